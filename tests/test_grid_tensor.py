"""GridTensor / Annotator / Registry behaviour (scenarios of the reference's
test/python/grid_tensor_test.py:13-71), CPU only."""
import pytest
import torch
import torch.nn as nn

import brt
from brt.runtime.grid_tensor import GridTensor, init_grid_tensor, deinit_grid_tensor
from brt.runtime import Registry


def test_annotator_shapes_and_initial_stacks():
    x = torch.randn(2, 3, 4, 5)
    a = brt.Annotator([0])(x)
    assert isinstance(a, GridTensor) and a.shape == (2, 3, 4, 5)
    assert a.tag_stack == [None] and a.load_stack == [None] and a.stack_size == 1
    b = brt.Annotator([0, 1])(x)
    assert b.shape == (6, 4, 5)
    c = brt.Annotator([1, 3])(x)  # cell dims moved to the front, rest = cell shape
    assert c.shape == (15, 2, 4)
    assert torch.equal(c[0 * 5 + 1], x[:, 0, :, 1])
    d = brt.Annotator([0], cell_shape=[60])(x)
    assert d.shape == (2, 60)
    e = brt.Annotator([0], gridding=False)(x)
    assert not isinstance(e, GridTensor)
    assert brt.Annotator([0])(a).stack_size == 2  # annotating twice pushes a level


def test_pack_unpack_and_deep_variants():
    t = init_grid_tensor(torch.arange(6.0).view(3, 2))
    assert t.annotation_empty()
    tag, load = torch.tensor([1, 2, 3]), torch.tensor([3])
    t.pack(tag, load, extra=7)
    assert t.tag is tag and t.load is load and t.get_extra_attr("extra") == 7
    t.set_extra_attr("extra", 8)
    _, tag2, load2, extra = t.unpack("extra")
    assert tag2 is tag and load2 is load and extra == {"extra": 8} and t.annotation_empty()
    t.deep_pack([tag, None], [load, None])
    assert t.stack_size == 2
    plain, tags, loads, _ = deinit_grid_tensor(t)
    assert type(plain) is torch.Tensor and tags == [tag, None] and loads == [load, None]
    with pytest.raises(AssertionError):
        init_grid_tensor(torch.zeros(1)).unpack()


@pytest.mark.parametrize("shallow", [True, False])
def test_stacks_travel_through_torch_ops(shallow):
    old = GridTensor.SHALLOW_TRANSPORT
    GridTensor.SHALLOW_TRANSPORT = shallow
    try:
        x = brt.Annotator([0])(torch.randn(4, 10))
        tag = torch.arange(1, 5, dtype=torch.int32)
        x.tag, x.load = tag, torch.tensor([4])
        y = nn.Linear(10, 3)(x)
        z = torch.relu(y) + 1
        assert isinstance(z, GridTensor) and z.tag is tag
        assert (z.tag_stack is x.tag_stack) == shallow
        a, b = z.split(2, dim=0)
        assert isinstance(a, GridTensor) and b.tag is tag
        plain = brt.to_torch_tensor(z)
        assert type(plain) is torch.Tensor
        again = brt.to_grid_tensor(plain, *brt.to_torch_tensor(z, True)[1:])
        assert again.tag is tag
    finally:
        GridTensor.SHALLOW_TRANSPORT = old


def test_registry_names():
    from brt.router.base import RouterBase
    from brt.router.fabric import FabricBase, make_fabric
    from brt.router.protocol import ProtocolBase, make_protocol

    routers = Registry.sub_cls_registries[RouterBase]
    assert {"scatter", "gather", "swin_moe_scatter", "task_scatter"} <= set(routers)
    fabrics = Registry.sub_cls_registries[FabricBase]
    assert {"dispatch", "combine", "fused_dispatch", "fused_combine", "identity_dispatch",
            "identity_combine", "single_cell_dispatch", "single_cell_combine",
            "placeholder_combine", "distributed_fused_dispatch",
            "distributed_fused_combine"} <= set(fabrics)
    protocols = Registry.sub_cls_registries[ProtocolBase]
    assert {"topk", "switch_top1", "threshold", "residual_threshold", "binary_threshold", "hash",
            "task", "swin_moe", "label", "identity", "decoder_greedy_search"} <= set(protocols)
    assert make_protocol("topk", {"top_k": 2}).top_k == 2
    assert make_fabric("fused_combine", {"flow_num": 1}).is_tag_index is False
    assert make_fabric("combine", {"flow_num": 1}).is_tag_index is True
    with pytest.raises(ValueError):
        make_fabric("dispatch", {1: 2})
    assert brt.router.is_router(brt.router.ScatterRouter)


def test_router_defaults():
    from brt.router import GatherRouter, ScatterRouter, SwinMoEScatterRouter

    s = ScatterRouter()
    assert s.protocol_kwargs == {"top_k": 1}
    assert s.fabric_kwargs == {"flow_num": 1, "route_logic": "1d", "transform": False}
    s = ScatterRouter(dispatch_score=True, protocol_type="threshold")
    assert s.protocol_kwargs == {"threshold": 0.0, "residual_path": -1}
    assert s.fabric_kwargs == {"flow_num": 2, "route_logic": ["1d", "2d"], "transform": [False, False]}
    g = GatherRouter()
    assert g.fabric_kwargs == {"flow_num": 1, "reduction": "add", "sparse": False}
    w = SwinMoEScatterRouter(protocol_kwargs={"capacity_factor": 1.25})
    assert w.protocol.top_k == 1 and w.fabric.max_path_load == 0
    assert w.protocol.runtime_capacity(100352, 8) == 15680


def test_protocol_masks_on_cpu():
    from brt.router.protocol import make_protocol

    score = torch.tensor([[0.1, 0.7, 0.2], [0.6, 0.3, 0.1], [0.2, 0.2, 0.6]])
    assert make_protocol("topk", {"top_k": 1})(score).tolist() == [[0, 1, 0], [1, 0, 0], [0, 0, 1]]
    assert make_protocol("topk", {"top_k": 2})(score).sum(1).tolist() == [2, 2, 2]
    m = make_protocol("threshold", {"threshold": 0.5})(score)
    assert m.dtype == torch.int32 and m.tolist() == [[0, 1, 0], [1, 0, 0], [0, 0, 1]]
    m = make_protocol("threshold", {"threshold": 0.65, "residual_path": 2})(score)
    assert m.tolist() == [[0, 1, 0], [0, 0, 1], [0, 0, 1]]
    m = make_protocol("switch_top1", {})(torch.eye(3).view(1, 3, 3))
    assert m.dtype == torch.int32 and m.shape == (3, 3)
    m = make_protocol("label", {"path_num": 4})(torch.tensor([3, 0]))
    assert m.tolist() == [[0, 0, 0, 1], [1, 0, 0, 0]]
    m = make_protocol("task", {"num_tasks": 3})(torch.tensor([2, 2, 0]))
    assert m.tolist() == [[0, 0, 1], [0, 0, 1], [1, 0, 0]]
    h = make_protocol("hash", {"num_tasks": 4, "placement_aware": True})
    assert h(torch.tensor([3])).tolist() == [[1, 0, 0, 1]]
    m = make_protocol("residual_threshold", {"threshold": 0.0, "residual_path": 0})(
        torch.tensor([[-1.0, 0.0], [1.0, 0.0]]))
    assert m.tolist() == [[1, 0], [0, 1]]  # below the threshold -> path 0 (the residual path)
    m = make_protocol("binary_threshold", {"threshold": 0.9, "selected_path": 1})(
        torch.tensor([[10.0, 0.0], [0.1, 0.0]]))
    assert m.tolist() == [[0, 1], [1, 0]]  # confident rows take the selected path


def test_module_paths_of_the_reference_resolve():
    """Code written against the reference imports its classes from the modules it keeps them in
    (python/brt/router/fabric/fused.py, protocol/topk.py, ...)."""
    import importlib

    for path, attr in (("brt.router.fabric.fused", "FusedDispatchFabric"),
                       ("brt.router.fabric.generic", "DispatchFabric"),
                       ("brt.router.fabric.base", "make_fabric"),
                       ("brt.router.fabric.distributed", "DistributedFusedCombineFabric"),
                       ("brt.router.protocol.topk", "TopKProtocol"),
                       ("brt.router.protocol.swin_moe", "SwinMoEProtocol"),
                       ("brt.router.protocol.base", "make_protocol"),
                       ("brainstorm_amd.router.protocol.hashed", "HashProtocol")):
        module = importlib.import_module(path)
        assert hasattr(module, attr), path
    from brt.router.fabric.fused import FusedCombineFabric  # noqa: F401
    from brt.router.protocol.switch import SwitchTop1Protocol  # noqa: F401


def test_deferred_buffer_fills_itself_before_any_read_and_not_for_metadata():
    """Host logic of the deferred dispatch (no GPU: the dispatch itself is replaced by a counter).
    Shape, dtype, device leave the buffer alone; an operator on the plain tensor or on the
    GridTensor that wraps it fills it first, and so does anything that hands out its address
    (data_ptr, stride, storage_offset: a foreign kernel could read through them); afterwards
    nothing is deferred any more."""
    import brt
    from brainstorm_amd.runtime import deferred

    class State(deferred.DeferredState):
        __slots__ = ("fills",)

        def materialize(self):
            if not self.done:
                self.fills += 1
                self.buffer.fill_(7.0)
                self.done = True

    def make():
        cells = torch.zeros(4, 3)
        state = State(cells, route=None, buffer=torch.empty(6, 3), key="brt_deferred_0")
        state.fills = 0
        grid = brt.to_grid_tensor(state.buffer, [torch.zeros(1)], [torch.zeros(1)], {"brt_deferred_0": state})
        return state, grid

    state, grid = make()
    assert tuple(grid.shape) == (6, 3) and grid.dtype == torch.float32 and state.fills == 0
    plain, tags, loads, extra = brt.to_torch_tensor(grid, retrieve_attr=True)
    assert isinstance(plain, deferred.DeferredRows) and deferred.state_of(plain) is state
    assert plain.shape[0] == 6 and plain.device.type == "cpu" and plain.is_contiguous() and state.fills == 0
    total = plain.sum()                      # a read: the dispatch runs first
    assert state.fills == 1 and float(total) == 7.0 * 18 and deferred.state_of(plain) is None
    assert type(plain + 1) is torch.Tensor   # results are ordinary tensors
    again = brt.to_torch_tensor(grid)        # nothing pending any more: a plain tensor
    assert type(again) is torch.Tensor and state.fills == 1

    state, grid = make()
    doubled = grid * 2                       # an operator on the GridTensor fills it too
    assert state.fills == 1 and float(brt.to_torch_tensor(doubled).sum()) == 14.0 * 18
    assert isinstance(doubled, brt.GridTensor) and doubled.extra_attr_dict["brt_deferred_0"] is state

    for read in (lambda t: t.data_ptr(), lambda t: t.stride(), lambda t: t.storage_offset()):
        state, grid = make()
        read(grid)                           # the address of the GridTensor: filled first
        assert state.fills == 1
        state, grid = make()
        plain = brt.to_torch_tensor(grid)
        assert state.fills == 0
        read(plain)                          # ... and of the plain tensor
        assert state.fills == 1
    state, grid = make()
    assert deferred.pending_of(grid) is state and deferred.pending_of(brt.to_torch_tensor(grid)) is state
    assert deferred.pending_of(torch.ones(2)) is None and state.fills == 0

    state, grid = make()
    product = torch.matmul(input=grid, other=torch.ones(3, 2))  # operands passed by keyword only
    assert state.fills == 1 and float(product.sum()) == 7.0 * 3 * 12
    assert isinstance(product, brt.GridTensor) and product.extra_attr_dict["brt_deferred_0"] is state

    state, grid = make()
    other = torch.ones(6, 3)
    assert deferred.pending_state(grid.extra_attr_dict, other) is None  # another tensor is not the buffer
    assert deferred.wrap_if_pending(other, grid.extra_attr_dict) is other and state.fills == 0
