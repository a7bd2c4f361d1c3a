"""CPU: pins the oracle's MoE statements (float64 brute force, dense == sparse identity)."""
import numpy as np
import pytest
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


def _deepseek_case(dtype, seed, with_bias, score_func):
    """64 experts in 8 groups, 4 groups kept, top-8; experts with an odd global id are not local."""
    T, E, K, H, I = 24, 64, 8, 64, 32
    x = randn((T, H), dtype, 1.0, seed)
    logits = randn((T, E), dtype, 1.5, seed + 1)
    bias = randn((E,), dtype, 0.1, seed + 2).abs() if with_bias else None
    emap = torch.tensor([e // 2 if e % 2 == 0 else -1 for e in range(E)])
    w1 = randn((E // 2, 2 * I, H), dtype, 0.3, seed + 3)
    w2 = randn((E // 2, H, I), dtype, 0.3, seed + 4)
    return T, E, K, x, logits, bias, emap, w1, w2


def _tie_free_rows(logits, score_fun, bias, n_groups, topk_group, topk):
    """Rows on which no rule about ties is needed: group scores distinct across the keep / drop line and
    selection scores distinct across the pick / no-pick line (after the group mask)."""
    dtype = logits.dtype
    p = router.scores(logits, score_fun)
    sel = p if bias is None else (p + bias.reshape(1, -1)).to(dtype)
    T, E = sel.shape
    ok = []
    for t in range(T):
        g = sel[t].float().view(n_groups, -1)
        if bias is None:
            gs = g.max(dim=-1).values
        else:
            top2 = g.topk(2, dim=-1).values.to(dtype)
            gs = (top2[:, 0] + top2[:, 1]).float()
        gsort = torch.sort(gs, descending=True)
        if gsort.values[topk_group - 1] == gsort.values[topk_group]:
            continue
        mask = torch.zeros(n_groups, dtype=torch.bool)
        mask[gsort.indices[:topk_group]] = True
        masked = torch.where(mask[:, None].expand_as(g), g, torch.zeros_like(g)).reshape(-1)
        ssort = torch.sort(masked, descending=True).values
        if ssort[topk - 1] == ssort[topk] or ssort[topk - 1] <= 0:
            continue
        ok.append(t)
    return ok


@pytest.mark.parametrize("with_bias", [False, True])
@pytest.mark.parametrize("score_func", ["softmax", "sigmoid"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_torch_path_grouped_branches_against_router_and_sparse_statement(dtype, score_func, with_bias):
    """The dense torch path (oracle restatement and the helper the package ships), run through
    group mask, top-2-sum group score, bias-for-selection, renormalisation and an expert map,
    equals `router.route` + the sparse float64 statement on rows that need no tie rule."""
    from muxi_native_layout_kernels_amd import utils as shipped
    T, E, K, x, logits, bias, emap, w1, w2 = _deepseek_case(dtype, 40, with_bias, score_func)
    sf = 0 if score_func == "softmax" else 1
    rows = _tie_free_rows(logits, sf, bias, 8, 4, K)
    assert len(rows) >= T // 2
    ids, wts = router.route(logits, sf, 8, 4, K, bias)
    wts = router.renormalize(wts)
    want = moe.moe_expected(x, w1, w2, ids, wts, expert_map=emap.numpy())
    dense_a = moe.torch_path_fused_moe(x, w1, w2, logits, K, num_expert_group=8, topk_group=4, renormalize=True,
                                       bias=bias, score_func=score_func, expert_map=emap)
    dense_b = shipped.fused_moe(x, w1, w2, logits, K, num_expert_group=8, topk_group=4, global_num_experts=E,
                                expert_map=emap, renormalize=True, e_score_correction_bias=bias,
                                score_func=score_func)
    assert torch.equal(dense_a, dense_b)          # the two restatements of utils.py:131-244 agree exactly
    got = dense_a.double().numpy()
    tol = 1e-4 if dtype == torch.float32 else 6e-2   # bf16: the dense path rounds every intermediate to bf16
    scale = np.abs(want[rows]).max()
    assert scale > 0.5                               # the comparison sees a signal
    assert np.abs(got[rows] - want[rows]).max() <= tol * scale
    # negative control: the same comparison rejects the sparse statement with the last pick removed
    fewer = moe.moe_expected(x, w1, w2, ids[:, :K - 1], wts[:, :K - 1], expert_map=emap.numpy())
    assert np.abs(got[rows] - fewer[rows]).max() > tol * scale


@pytest.mark.parametrize("with_bias", [False, True])
def test_torch_path_selection_equals_router_ids_without_ties(with_bias):
    """Expert ids picked by the library top-k of the torch path == `router.route` ids as sets, bf16 scores."""
    T, E, K, x, logits, bias, emap, w1, w2 = _deepseek_case(torch.bfloat16, 60, with_bias, "sigmoid")
    from muxi_native_layout_kernels_amd import utils as shipped
    wts_t, ids_t = shipped._select_experts(logits, K, 8, 4, True, bias, "sigmoid", torch.bfloat16)
    ids, wts = router.route(logits, 1, 8, 4, K, bias)
    wts = router.renormalize(wts)
    rows = _tie_free_rows(logits, 1, bias, 8, 4, K)
    assert len(rows) >= T // 2
    for t in rows:
        assert sorted(ids_t[t].tolist()) == sorted(ids[t].tolist())
        by_id = dict(zip(ids[t].tolist(), wts[t].float().tolist()))
        for e, w in zip(ids_t[t].tolist(), wts_t[t].float().tolist()):
            assert abs(by_id[e] - w) <= 2 ** -7 * abs(w)     # one bf16 ulp: the library sums the weights in another order
