"""Grouped expert GEMM against the library routine it must reproduce: per-expert
``torch.nn.functional.linear`` on the expert's row slice (test/python/jit_test.py:183-203),
evaluated in fp32 on the bf16-rounded operands.  Tolerance 1e-2 relative (bf16 output)."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

ACT = {"none": 0, "gelu": 1, "relu": 2}


def reference(x, ws, bs, loads, act):
    outs, start = [], 0
    for e, m in enumerate(loads):
        y = torch.nn.functional.linear(x[start:start + m].float(), ws[e].float(),
                                       None if bs is None else bs[e].float())
        if act == "gelu":
            y = torch.nn.functional.gelu(y)
        elif act == "relu":
            y = torch.relu(y)
        outs.append(y)
        start += m
    return torch.cat(outs) if outs else x.new_zeros((0, ws[0].shape[0]))


def run(loads, K, N, act="none", bias=False, seed=0, slack=0):
    from brainstorm_amd import _lib

    g = torch.Generator().manual_seed(seed)
    E, rows = len(loads), sum(loads)
    P = rows + slack  # the buffer may be larger than the sum of the loads
    x = torch.randn(P, K, generator=g).to(torch.bfloat16).cuda()
    ws = [(torch.randn(N, K, generator=g) * 0.05).to(torch.bfloat16).cuda() for _ in range(E)]
    bs = [torch.randn(N, generator=g).to(torch.bfloat16).cuda() for _ in range(E)] if bias else None
    out = torch.full((P, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    wt = torch.tensor([w.data_ptr() for w in ws], dtype=torch.int64, device="cuda")
    bt = torch.tensor([b.data_ptr() for b in bs], dtype=torch.int64, device="cuda") if bias else None
    d_loads = torch.tensor(loads, dtype=torch.int32, device="cuda")
    _lib.check(_lib.lib().brt_hip_grouped_gemm(
        x.data_ptr(), wt.data_ptr(), None if bt is None else bt.data_ptr(), out.data_ptr(),
        d_loads.data_ptr(), E, P, K, N, ACT[act], torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    want = reference(x, ws, bs, loads, act)
    got = out[:rows].float()
    assert torch.isfinite(got).all(), "rows of an expert were left unwritten"
    if slack:
        assert torch.isnan(out[rows:].float()).all(), "rows beyond the loads were written"
    scale = want.abs().max().clamp_min(1e-6)
    err = (got - want).abs().max() / scale
    assert err < 1e-2, f"max error {err:.4f} relative to {scale:.3f}"
    return err


@pytest.mark.parametrize("loads,K,N", [
    ([16, 2], 512, 1024),                        # jit_test.py:157-203 shape
    ([2, 8, 4, 2], 512, 1024),                   # jit_test.py:310-355
    ([128] * 8, 768, 3072),
    ([160, 0, 1, 129, 127, 255, 300, 31], 768, 384),
    ([0, 0, 5, 0], 64, 128),
    ([1000, 3, 0, 700], 1024, 256),
    ([77, 200], 72, 200),                        # K and N tails
    ([33] * 70, 128, 128),                       # more than 64 experts
])
def test_grouped_gemm_matches_per_expert_linear(loads, K, N):
    run(loads, K, N)
    run(loads, K, N, act="gelu", bias=True, seed=1)
    run(loads, K, N, act="relu", bias=False, seed=2, slack=5)


def test_make_jit_kernel_homo_fuse_contract():
    import torch.nn as nn
    from brt.jit import make_jit_kernel

    linears = nn.ModuleList(nn.Linear(512, 1024) for _ in range(4)).cuda().to(torch.bfloat16)
    kernel = make_jit_kernel(linears, sample_inputs=[torch.randn(2 ** i, 512) for i in range(5)],
                             opt_level="homo_fuse")
    shared = [torch.randn(18, 512, device="cuda").to(torch.bfloat16),
              torch.empty(18, 1024, device="cuda", dtype=torch.bfloat16)]
    standalone = []
    for lin in linears:
        standalone += [lin.weight, lin.bias]
    capacities = torch.tensor([16, 2], dtype=torch.int32, device="cuda")
    kernel(shared, standalone, capacities)
    want = torch.cat([linears[0](shared[0][:16]), linears[1](shared[0][16:18])]).float()
    assert torch.allclose(shared[1].float(), want, atol=2e-2, rtol=1e-2)
    with pytest.raises(NotImplementedError):
        make_jit_kernel(linears, None, opt_level="hetero_fuse")
    with pytest.raises(NotImplementedError):
        kernel([shared[0].float(), shared[1].float()], standalone, capacities)


def test_full_size_switch_ffn():
    # BASELINE configs[1]: 64 experts, 768 -> 3072 -> 768, ~128 rows per expert
    rng = np.random.default_rng(2)
    loads = np.minimum(rng.multinomial(8192, [1 / 64] * 64), 160).tolist()
    run(loads, 768, 3072, act="gelu")
    run(loads, 3072, 768)


def test_ragged_dirichlet_loads_task_moe_shape():
    # BASELINE configs[4] at reduced size: loads ~ Dirichlet(0.3) (many empty experts, a few
    # with hundreds of rows), one launch over the ragged batches, both FFN shapes
    rng = np.random.default_rng(4)
    E, rows = 48, 4096
    loads = rng.multinomial(rows, rng.dirichlet(np.full(E, 0.3))).tolist()
    assert min(loads) == 0 and max(loads) > 320
    run(loads, 512, 2048, act="gelu", bias=True)
    run(loads, 2048, 512, slack=3)
