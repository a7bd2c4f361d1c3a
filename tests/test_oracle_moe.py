"""CPU: pins the oracle's MoE statements (float64 brute force, dense == sparse identity)."""
import numpy as np
import torch

from oracle import moe, router
from helpers import randn


def test_sparse_statement_matches_explicit_loops():
    E, T, H, I, K = 2, 3, 32, 32, 1
    w1 = torch.randn(E, 2 * I, H, dtype=torch.float64) * 0.2
    w2 = torch.randn(E, H, I, dtype=torch.float64) * 0.2
    x = torch.randn(T, H, dtype=torch.float64)
    ids = np.array([[0], [1], [0]])
    wts = np.array([[0.5], [1.0], [0.25]])
    a = moe.moe_expected(x, w1, w2, ids, wts)
    b = moe.moe_expected_loops(x, w1, w2, ids, wts)
    assert np.allclose(a, b, rtol=1e-12, atol=1e-12)


def test_dense_masked_sum_equals_sparse_gather():
    E, T, H, I, K = 8, 12, 128, 128, 2
    w1 = randn((E, 2 * I, H), torch.float32, 0.1, 1)
    w2 = randn((E, H, I), torch.float32, 0.1, 2)
    x = randn((T, H), torch.float32, 1.0, 3)
    logits = randn((T, E), torch.float32, 1.0, 4)
    dense = moe.torch_path_fused_moe(x, w1, w2, logits, K, renormalize=True)
    # same routing, restated independently
    p = torch.softmax(logits, dim=-1)
    wts, ids = torch.topk(p, K, dim=-1)
    wts = wts / wts.sum(dim=-1, keepdim=True)
    sparse = moe.moe_expected(x, w1, w2, ids, wts)
    assert np.allclose(dense.double().numpy(), sparse, rtol=1e-4, atol=1e-5)


def test_torch_path_router_agrees_with_kernel_rules_without_ties():
    T, E, K = 64, 8, 2
    logits = randn((T, E), torch.bfloat16, 1.0, 9)
    ids, wts = router.route(logits, 0, 1, 1, K)
    wts = router.renormalize(wts)
    p = torch.softmax(logits, dim=-1, dtype=torch.bfloat16)
    tw, ti = torch.topk(p, K, dim=-1)
    for t in range(T):
        srt = torch.sort(p[t].float(), descending=True).values
        if srt[K - 1] == srt[K] or srt[0] == srt[1]:
            continue
        assert sorted(ti[t].tolist()) == ids[t].tolist()


def test_dropped_pairs_contribute_nothing():
    E, T, H, I = 4, 5, 32, 32
    w1 = torch.randn(E, 2 * I, H, dtype=torch.float64)
    w2 = torch.randn(E, H, I, dtype=torch.float64)
    x = torch.randn(T, H, dtype=torch.float64)
    ids = np.array([[0, 1]] * T)
    wts = np.ones((T, 2))
    emap = np.array([0, -1, 1, 2])
    full = moe.moe_expected(x, w1, w2, ids, wts, expert_map=emap)
    only0 = moe.moe_expected(x, w1, w2, ids[:, :1], wts[:, :1])
    assert np.allclose(full, only0)
