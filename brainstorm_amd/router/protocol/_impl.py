"""Protocols: gate scores -> int32 hot mask ``[cells, paths]``.

Registry names, constructor arguments and return conventions follow
python/brt/router/protocol/*.py of the reference.  The masks themselves are
built with ordinary torch ops (as in the reference); the capacity throttle of
the Swin-MoE protocol runs the HIP ``throttle_hotmask`` kernel.
"""
import os
from typing import Any, Callable, Dict

import torch
import torch.nn as nn

from brainstorm_amd._C import router as c_router
from brainstorm_amd.router.utils import make_kwargs
from brainstorm_amd.runtime import Registry


class ProtocolBase(nn.Module):
    """protocol/base.py:17-47."""

    def __init__(self, **kwargs):
        super().__init__()
        self.debug = os.environ.get("BRT_DEBUG", "False").lower() in ("true", "1")

    #: True when the protocol never routes a cell to more than one path; the hot mask is
    #: then marked so that the fabrics can use the tag-driven combine
    single_path = False

    def forward(self, score: torch.Tensor, *args, **kwargs):
        decisions = self.make_route_decision(score, *args, **kwargs)
        if self.debug:
            self.check_decision(decisions, score)
        if self.single_path:
            hot_mask = decisions[0] if isinstance(decisions, (tuple, list)) else decisions
            hot_mask._brt_single_path = True
        return decisions

    def make_route_decision(self, score, **kwargs):
        raise NotImplementedError("make_route_decision has to be implemented by user")

    def check_decision(self, decisions, scores: torch.Tensor) -> None:
        hot_mask = decisions[0] if isinstance(decisions, (tuple, list)) else decisions
        assert hot_mask.size(0) == scores.size(0), (
            "indices and scores should have the same size in the first dimension")

    def check_compatibility(self, kwargs: Dict[str, Any]) -> None:
        pass


def register_protocol(protocol_type: str) -> Callable:
    return Registry.register_sub_cls(protocol_type, ProtocolBase)


def make_protocol(protocol_type: str, kwargs: Dict[str, Any]) -> ProtocolBase:
    protocol_cls = Registry.get_sub_cls(protocol_type, ProtocolBase)
    if protocol_cls is None:
        raise ValueError(f"Protocol type: {protocol_type} is not registered.")
    return protocol_cls(**make_kwargs(kwargs))


class CompactHotMask:
    """The decision of a top-k protocol kept as ``k`` path ids per cell instead of a
    ``[cells, paths]`` int32 mask (an extension: python/brt/router/protocol/topk.py:26-31 builds the
    mask with ``topk`` + ``zeros_like`` + ``scatter_``).  Only a fused dispatch fabric built with
    ``compact_route=True`` receives one; it reads ``path_ids`` and never needs the mask.
    ``dense()`` is the mask the reference would have built."""

    dtype = torch.int32

    def __init__(self, path_ids: torch.Tensor, scores: torch.Tensor, path_num: int):
        self.path_ids = path_ids   # [cells, k] int32, in the order of torch.topk
        self.scores = scores       # [cells, k] fp32: the scores of the chosen paths
        self.shape = torch.Size((path_ids.shape[0], int(path_num)))
        self.device = path_ids.device
        self.is_cuda = path_ids.is_cuda
        self._dense = None

    def size(self, dim=None):
        return self.shape if dim is None else self.shape[dim]

    def dim(self):
        return 2

    def numel(self):
        return self.shape[0] * self.shape[1]

    def dense(self) -> torch.Tensor:
        if self._dense is None:
            self._dense = torch.zeros(tuple(self.shape), dtype=torch.int32, device=self.device).scatter_(
                1, self.path_ids.long(), 1)
            if getattr(self, "_brt_single_path", False):
                self._dense._brt_single_path = True
        return self._dense


def _one_hot_int32(indices: torch.Tensor, like: torch.Tensor) -> torch.Tensor:
    """int32 mask with ones at ``indices`` (``[cells, k]``) along dim 1."""
    return torch.zeros(like.shape, dtype=torch.int32, device=like.device).scatter_(1, indices, 1)


def _topk_hot_mask(score, top_k):
    """int32 mask with ones at the ``top_k`` largest scores of every row (``torch.topk`` +
    ``zeros_like`` + ``scatter_``, protocol/topk.py:26-31): one kernel where the score is a 2-d
    device tensor of up to 1024 paths, the three torch launches otherwise."""
    if (score.is_cuda and score.dim() == 2 and score.shape[1] <= 1024
            and score.dtype in (torch.float32, torch.float16, torch.bfloat16)):
        return c_router.topk_hot_mask(score, top_k)
    return _one_hot_int32(torch.topk(score, top_k, dim=1).indices, score)


@register_protocol("topk")
class TopKProtocol(ProtocolBase):
    """protocol/topk.py:13-31."""

    def __init__(self, top_k=1):
        super().__init__()
        self.top_k = top_k
        self.single_path = top_k == 1
        #: set by a ScatterRouter whose fabric takes the compact route: the decision is handed
        #: over as path ids (one kernel, k words per cell) instead of the [cells, paths] mask
        self.compact = False

    def make_route_decision(self, score):
        if (self.compact and score.is_cuda and score.dim() == 2 and 0 < self.top_k <= score.shape[1] <= 1024
                and score.dtype in (torch.float32, torch.float16, torch.bfloat16)):
            path_ids, scores = c_router.gate_topk(score, self.top_k)
            return CompactHotMask(path_ids, scores, score.shape[1])
        return _topk_hot_mask(score, self.top_k)


@register_protocol("switch_top1")
class SwitchTop1Protocol(ProtocolBase):
    """protocol/switch.py:13-33: the score already is the (capacity-masked) hot mask.

    ``one_hot=True`` (an extension) is the caller's promise that no row of the mask has more than
    one nonzero, which lets the fabrics use the tag-driven combine and the deferred dispatch.  The
    mask comes from the caller, so nothing is assumed by default: a row with several ones is
    routed to all of them and summed, as in the reference."""

    def __init__(self, one_hot: bool = False, **kwargs):
        super().__init__(**kwargs)
        self.single_path = bool(one_hot)

    def make_route_decision(self, score):
        mask = score.reshape(-1, score.shape[-1]).to(torch.int32, non_blocking=True)
        # never the caller's own tensor object: the single-path mark is set on what is returned
        return mask.view_as(mask) if mask is score else mask

    def update(self, supported_capacities):
        self.supported_capacities = supported_capacities


@register_protocol("threshold")
class ThresholdProtocol(ProtocolBase):
    """protocol/threshold.py:13-40."""

    def __init__(self, threshold=0.0, residual_path=-1, **kwargs):
        super().__init__(**kwargs)
        self.threshold = threshold
        self.residual_path = residual_path

    def make_route_decision(self, score: torch.Tensor):
        hot_mask = (score > self.threshold).to(torch.int32)
        if self.residual_path >= 0:  # cells no path took go to the residual path
            orphan = (hot_mask.sum(dim=1, keepdim=True) == 0).to(torch.int32)
            where = torch.full_like(orphan, self.residual_path, dtype=torch.int64)
            hot_mask = torch.scatter_add(hot_mask, 1, where, orphan)
        return hot_mask.to(torch.int32)


def _binary_mask(picks_second: torch.Tensor, first_is_default: bool, score: torch.Tensor):
    """Two-path mask: row i routes to path 1 where ``picks_second[i]``, else path 0
    (``first_is_default``), or the complement."""
    idx = picks_second.to(torch.int64).view(-1, 1)
    if first_is_default:
        base = torch.ones(score.size(0), 2, dtype=torch.int32, device=score.device)
        return base.scatter_(1, idx, 0)
    base = torch.zeros(score.size(0), 2, dtype=torch.int32, device=score.device)
    return base.scatter_(1, idx, 1)


@register_protocol("residual_threshold")
class ResidualThresholdProtocol(ProtocolBase):
    """protocol/threshold.py:43-66."""

    def __init__(self, threshold=0.0, residual_path=0, **kwargs):
        super().__init__(**kwargs)
        self.threshold = threshold
        self.residual_path = residual_path

    def make_route_decision(self, score: torch.Tensor):
        below = score.sum(dim=1, keepdim=True) < self.threshold
        if self.residual_path not in (0, 1):
            raise ValueError("residual_path should be 0 or 1")
        return _binary_mask(below, self.residual_path == 0, score)


@register_protocol("binary_threshold")
class BinaryThresholdProtocol(ProtocolBase):
    """protocol/threshold.py:69-94."""

    def __init__(self, threshold=0.0, selected_path=0, **kwargs):
        super().__init__(**kwargs)
        self.threshold = threshold
        self.selected_path = selected_path
        self.softmax = nn.Softmax(dim=1)

    def make_route_decision(self, score: torch.Tensor):
        confident = self.softmax(score).max(dim=1).values >= self.threshold
        if self.selected_path not in (0, 1):
            raise ValueError("selected_path should be 0 or 1 for a binary threshold protocol")
        return _binary_mask(confident, self.selected_path == 0, score)


@register_protocol("hash")
class HashProtocol(ProtocolBase):
    """protocol/hashed.py:15-59: two fixed destinations per task id."""

    def __init__(self, num_tasks: int, placement_aware: bool = False, seed: int = 0, **kwargs):
        super().__init__(**kwargs)
        self.num_tasks = num_tasks
        self.placement_aware = placement_aware
        if placement_aware:
            first = torch.arange(num_tasks, dtype=torch.int64).view(-1, 1)
            second = (first + 1) % num_tasks
        else:
            torch.random.manual_seed(seed)
            first = torch.randperm(num_tasks, dtype=torch.int64).view(-1, 1)
            second = torch.flip(first, dims=[0])
        self.register_buffer("hash_indices", torch.cat([first, second], dim=1))
        self.check_hash_indices()

    def make_route_decision(self, task_ids: torch.Tensor):
        like = torch.empty((task_ids.size(0), self.num_tasks), device=task_ids.device)
        return _one_hot_int32(self.hash_indices[task_ids], like)

    def check_hash_indices(self):
        assert tuple(self.hash_indices.shape) == (self.num_tasks, 2)


@register_protocol("task")
class TaskProtocol(ProtocolBase):
    """protocol/hashed.py:62-91: cell of task i goes to path i."""

    def __init__(self, num_tasks: int, supported_capacities: torch.Tensor = None, **kwargs):
        super().__init__(**kwargs)
        self.supported_capacities = supported_capacities
        self.num_tasks = num_tasks
        self.register_buffer("task_indices", torch.arange(num_tasks, dtype=torch.int64).view(-1, 1))

    def make_route_decision(self, task_ids: torch.Tensor):
        like = torch.empty((task_ids.size(0), self.num_tasks), device=task_ids.device)
        return _one_hot_int32(self.task_indices[task_ids], like)


@register_protocol("label")
class LabelProtocol(ProtocolBase):
    """protocol/label.py:13-33: ``score`` is a 1-d tensor of path labels."""

    def __init__(self, path_num: int, **kwargs):
        super().__init__(**kwargs)
        self.path_num = path_num

    def make_route_decision(self, score):
        return torch.nn.functional.one_hot(score, num_classes=self.path_num)


@register_protocol("identity")
class IdentityProtocol(ProtocolBase):
    """protocol/identity.py:7-14."""

    def __init__(self, **kwargs):
        self.check_compatibility(kwargs)
        super().__init__(**kwargs)

    def make_route_decision(self, score, **kwargs):
        return None, None, None


def throttle_to_capacity(hot_mask, prefix, capacity, by_score=False, score=None):
    """Keeps at most ``capacity[e] - prefix[e]`` cells per path, first come first
    served, or highest score first (protocol/swin_moe.py:47-60)."""
    if not by_score:
        return c_router.throttle_hotmask(hot_mask, prefix, capacity)
    order = (-score.max(dim=1)[0]).argsort(dim=0)
    throttled, prefix = c_router.throttle_hotmask(hot_mask[order].contiguous(), prefix, capacity)
    return throttled[order.argsort(dim=0)], prefix


@register_protocol("swin_moe")
class SwinMoEProtocol(ProtocolBase):
    """protocol/swin_moe.py:69-144 (the maintained ``make_route_decision``)."""

    single_path = True  # only the first of the top-k choices is routed (swin_moe.py:138-144)

    def __init__(self, top_k=2, capacity_factor=0, gate_noise=0.0, group=None, is_postscore=True,
                 batch_prioritized_routing=False, normalize_gate=True, is_gshard_loss=True,
                 alignment=1, **kwargs):
        super().__init__(**kwargs)
        self.top_k = top_k
        self.capacity_factor = capacity_factor
        self.gate_noise = gate_noise
        self.normalize_gate = normalize_gate
        self.batch_prioritized_routing = batch_prioritized_routing
        self.is_postscore = is_postscore
        self.group = group
        self.is_gshard_loss = is_gshard_loss
        self.alignment = alignment

    def runtime_capacity(self, cells: int, paths: int) -> int:
        if self.capacity_factor <= 0:
            raise NotImplementedError("capacity_factor must be greater than 0")
        per_path = (int(cells) + paths - 1) // paths
        return self.top_k * int(self.capacity_factor * per_path)  # swin_moe.py:112-119

    def make_route_decision(self, score, logits_wo_noise, logits):
        paths = score.size(1)
        mask = _topk_hot_mask(score, 1)  # the first of the top-k choices (swin_moe.py:101-107)
        loss = self.generate_auxiliary(score, logits_wo_noise, logits, None)
        cap = self.runtime_capacity(score.size(0), paths)
        runtime_capacities = torch.full((paths,), cap, dtype=torch.int32, device=score.device)
        prefix = torch.zeros((paths,), dtype=torch.int32, device=score.device)
        hot_mask, _ = throttle_to_capacity(
            mask, prefix, runtime_capacities, self.batch_prioritized_routing, score)
        return hot_mask, runtime_capacities, score, loss

    def generate_auxiliary(self, score, logits_wo_noise, logits, topk_ids):
        return None  # the reference's auxiliary loss is commented out (swin_moe.py:241-252)


class DecoderProtocol(ProtocolBase):
    """protocol/decoder.py:9-28."""

    def __init__(self, index_format: str, pad_token_id: int, eos_token_id: int,
                 skip_eos_check: bool = False):
        super().__init__()
        self.eos_token_id = eos_token_id
        self.pad_token_id = pad_token_id
        self.skip_eos_check = skip_eos_check
        if skip_eos_check:
            self.default_path = 0
        self.sorted_sequence_length = None
        self.iteration = 0

    def update(self, seqence_length: torch.Tensor):
        self.sorted_sequence_length = seqence_length.unique(sorted=True).cpu().numpy()
        self.checking_sequence_length = self.sorted_sequence_length[0]
        self.next_sequence_length_id = 1
        self.iteration = 0

    def _advance(self) -> bool:
        """True while no sequence can have finished yet (skip_eos_check only)."""
        self.iteration += 1
        if self.iteration == self.checking_sequence_length:
            self.checking_sequence_length = self.sorted_sequence_length[self.next_sequence_length_id]
            self.next_sequence_length_id += 1
        return self.iteration + 1 < self.checking_sequence_length


@register_protocol("decoder_greedy_search")
class DecoderGreedySearchProtocol(DecoderProtocol):
    """protocol/decoder.py:31-75: path 0 = unfinished sequences, path 1 = finished."""

    def make_route_decision(self, score: torch.Tensor):
        if self.skip_eos_check and self._advance():
            n = score.size(0)
            route_indices = torch.zeros(n, 2, dtype=torch.int64, device=score.device)
            route_indices[:, self.default_path] = torch.arange(n, dtype=torch.int64, device=score.device)
            loads = torch.tensor([n, 0], dtype=torch.int64, device=score.device)
            return route_indices, loads, loads
        unfinished = (score != self.eos_token_id).long()
        hot_mask = torch.cat([unfinished, 1 - unfinished], dim=1)
        _, loads = c_router.generate_indices_and_loads(hot_mask.to(torch.int32))
        return hot_mask, loads, loads


@register_protocol("decoder_beam_search")
class DecoderBeamSearchProtocol(DecoderProtocol):
    def make_route_decision(self, score: torch.Tensor):
        raise NotImplementedError("DecoderBeamSearchProtocol not completed yet")  # decoder.py:97
