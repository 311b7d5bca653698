"""The torch CPU path timed as cpu_baseline computes what the C oracle computes."""
import numpy as np
import pytest
import torch

import oracle
from oracle import torch_path
from routing_cases import softmax, topk_mask


@pytest.mark.parametrize("T,E,k,caps,pad", [
    (1024, 16, 1, [64], False), (2048, 64, 1, [40], True), (512, 8, 2, None, False),
    (300, 5, 2, [10, 100, 200], True), (300, 5, 2, [10, 100, 200], False),
])
def test_torch_path_matches_c_oracle(T, E, k, caps, pad):
    mask, logits = topk_mask(T, E, k, seed=T + E)
    mask[:, E - 1] = 0  # an empty path
    x = np.random.default_rng(T).standard_normal((T, 24)).astype(np.float32)
    gates = softmax(logits).astype(np.float32)
    o_idx, o_loads = oracle.generate_indices_and_loads(mask, caps, pad)
    idx, loads = torch_path.generate_indices_and_loads(torch.from_numpy(mask), caps, pad)
    assert np.array_equal(idx.numpy(), o_idx) and np.array_equal(loads.numpy(), o_loads)
    for g in (None, gates):
        tg = None if g is None else torch.from_numpy(g)
        y = torch_path.dispatch(torch.from_numpy(x), idx, loads, tg)
        o_y, _ = oracle.dispatch(x, o_idx, o_loads, gates=g)
        assert np.array_equal(y.numpy(), o_y)
        res = np.random.default_rng(1).standard_normal((T, 24)).astype(np.float32)
        for r in (None, res):
            out = torch_path.combine(y, idx, loads, tg, None if r is None else torch.from_numpy(r))
            o_out = oracle.combine(o_y, o_idx, o_loads, gates=g, out_data=r)
            assert np.array_equal(out.numpy(), o_out)
