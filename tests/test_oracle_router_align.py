"""CPU: pins the oracle's router and alignment statements."""
import json
import os

import numpy as np
import pytest
import torch

from oracle import router, align
from helpers import randn

GOLD = os.path.join(os.path.dirname(__file__), "golden")


def _brute(p_row, k):
    return sorted(range(len(p_row)), key=lambda j: (-p_row[j], j))[:k]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("score_fun", [0, 1])
def test_router_matches_brute_force_ranking(dtype, score_fun):
    logits = randn((64, 8), dtype, 1.0, 7)
    ids, w = router.route(logits, score_fun, 1, 1, 2)
    p = router.scores(logits, score_fun).double().numpy()
    for t in range(64):
        want = _brute(p[t], 2)
        got = ids[t].tolist()
        assert (sorted(want) == got) if score_fun == 0 else (want == got)
        for k in range(2):
            assert w[t, k].double().item() == p[t, ids[t, k]]


def test_router_special_cases():
    eq = torch.zeros((3, 16), dtype=torch.bfloat16)
    ids, w = router.route(eq, 0, 1, 1, 4)
    assert ids.tolist() == [[0, 1, 2, 3]] * 3
    assert torch.all(w.float() == 1.0 / 16)
    hot = torch.full((2, 8), -20.0, dtype=torch.float16)
    hot[0, 5] = 10.0
    hot[1, 2] = 10.0
    ids, w = router.route(hot, 0, 1, 1, 1)
    assert ids.reshape(-1).tolist() == [5, 2] and torch.all(w.float() == 1.0)
    ids, _ = router.route(hot, 1, 1, 1, 1)
    assert ids.reshape(-1).tolist() == [5, 2]


def test_router_agrees_with_library_topk_when_no_ties():
    logits = randn((256, 64), torch.bfloat16, 2.0, 11)
    ids, w = router.route(logits, 0, 1, 1, 6)
    p = router.scores(logits, 0).float()
    top = torch.topk(p, 7, dim=-1)
    ok = top.values[:, 5] != top.values[:, 6]
    # also require the six picked values to be distinct so library order is defined
    for t in range(256):
        if not ok[t] or len(set(top.values[t, :6].tolist())) < 6:
            continue
        assert sorted(top.indices[t, :6].tolist()) == ids[t].tolist()


def test_router_softmax_scores_match_library():
    logits = randn((32, 128), torch.float16, 1.5, 3)
    p = router.scores(logits, 0).float()
    lib = torch.softmax(logits.double(), dim=-1)
    assert torch.allclose(p.double(), lib, rtol=2e-3, atol=1e-6)
    assert torch.allclose(router.scores(logits, 1).double(), torch.sigmoid(logits.double()), rtol=2e-3, atol=1e-6)


def test_router_grouped_with_bias_brute_force():
    torch.manual_seed(0)
    logits = randn((40, 32), torch.bfloat16, 1.0, 5)
    bias = randn((32,), torch.bfloat16, 0.1, 6).abs()
    ids, w = router.route(logits, 1, 8, 4, 8, bias=bias)
    p = router.scores(logits, 1)
    sel = (p + bias.reshape(1, -1)).to(torch.bfloat16)
    for t in range(40):
        s = sel[t].float()
        g = s.view(8, 4)
        top2 = g.topk(2, dim=-1).values
        gs = (top2[:, 0].to(torch.bfloat16) + top2[:, 1].to(torch.bfloat16)).float()
        kept = sorted(range(8), key=lambda j: (-gs[j].item(), j))[:4]
        masked = s.clone()
        for j in range(8):
            if j not in kept:
                masked[j * 4:(j + 1) * 4] = 0
        want = _brute(masked.tolist(), 8)
        assert want == ids[t].tolist()            # sigmoid variant keeps pick order
        assert torch.equal(w[t], p[t][ids[t].long()])


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("score_fun", [0, 1])
@pytest.mark.parametrize("E,n_groups,topk_groups,K", [(32, 8, 4, 8), (256, 8, 4, 8), (64, 4, 2, 6), (48, 6, 1, 3)])
def test_router_grouped_without_bias_brute_force(dtype, score_fun, E, n_groups, topk_groups, K):
    """No bias: the group score is the largest score of the group (fused_topK.h:136-171).  Independent
    ranking: groups by (-max, group id), then the experts of the kept groups by (-score, id)."""
    T = 48
    logits = randn((T, E), dtype, 1.5, 100 + E)
    ids, w = router.route(logits, score_fun, n_groups, topk_groups, K)
    p = router.scores(logits, score_fun).double().numpy()
    per = E // n_groups
    for t in range(T):
        gmax = [p[t, g * per:(g + 1) * per].max() for g in range(n_groups)]
        kept = sorted(range(n_groups), key=lambda g: (-gmax[g], g))[:topk_groups]
        cand = [j for j in range(E) if j // per in kept]
        want = sorted(cand, key=lambda j: (-p[t, j], j))[:K]
        got = ids[t].tolist()
        assert (sorted(want) == got) if score_fun == 0 else (want == got)
        assert all(g // per in kept for g in got)
        for k in range(K):
            assert w[t, k].double().item() == p[t, got[k]]


def test_router_grouped_one_group_equals_plain():
    logits = randn((32, 64), torch.bfloat16, 1.0, 8)
    a = router.route(logits, 1, 1, 1, 6)
    b = router.route(logits, 1, 8, 8, 6)          # every group kept: the mask removes nothing
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])


def test_renormalize():
    w = torch.tensor([[0.25, 0.5], [0.125, 0.125]], dtype=torch.bfloat16)
    r = router.renormalize(w)
    assert r.tolist() == [[0.333984375, 0.66796875], [0.5, 0.5]]
    assert torch.equal(r, (w / w.sum(dim=-1, keepdim=True)))


def _check_invariants(ids, out, E, block=16, emap=None):
    flat = np.asarray(ids).reshape(-1)
    n = flat.size
    local = np.array([e if emap is None else emap[e] for e in flat])
    s = out["sorted_token_ids"]
    assert s.size == n + E * (block - 1)
    seen = s[s != n]
    assert sorted(seen.tolist()) == [i for i in range(n) if local[i] != -1]
    cs = out["cumsum"]
    assert cs[0] == 0 and all(c % block == 0 for c in cs)
    for e in range(E):
        seg = s[cs[e]:cs[e + 1]]
        real = seg[seg != n]
        assert all(local[i] == e for i in real)
        assert list(real) == sorted(real)                       # ascending flat index
        assert all(v == n for v in seg[len(real):])             # padding at the tail of the segment
        assert cs[e + 1] - cs[e] == (out["counts"][e] + block - 1) // block * block
        for b in range(cs[e] // block, cs[e + 1] // block):
            assert out["experts_ids"][b] == e
        assert out["cursors"][e] == cs[e] + out["counts"][e]
    assert out["padded_num_blocks"] == cs[E] // block
    assert all(v == n for v in s[cs[E]:])


def test_align_reference_example():
    ex = json.load(open(os.path.join(GOLD, "align_example_topk_ids.json")))
    out = align.align_tokens(ex["topk_ids"], ex["num_experts"])
    _check_invariants(ex["topk_ids"], out, ex["num_experts"])
    # brute force: expert 45 appears at flat indices 3, 9, 16, 40, 56
    cs = out["cumsum"]
    assert out["sorted_token_ids"][cs[45]:cs[45] + 5].tolist() == [3, 9, 16, 40, 56]
    assert out["counts"][45] == 5 and out["counts"][2] == 0
    assert out["padded_num_blocks"] == len(set(ex["topk_ids"]))  # every used expert has < 16 pairs


@pytest.mark.parametrize("T,K,E", [(1, 2, 8), (16, 2, 8), (64, 2, 8), (256, 2, 8), (33, 8, 256), (100, 6, 64)])
def test_align_invariants_random(T, K, E):
    rng = np.random.default_rng(T * 31 + K)
    ids = np.stack([rng.choice(E, size=K, replace=False) for _ in range(T)])
    _check_invariants(ids, align.align_tokens(ids, E), E)


def test_align_expert_map_drops_pairs():
    rng = np.random.default_rng(1)
    ids = np.stack([rng.choice(16, size=4, replace=False) for _ in range(20)])
    emap = np.array([e // 2 if e % 2 == 0 else -1 for e in range(16)])
    out = align.align_tokens(ids, 8, experts_map=emap)
    _check_invariants(ids, out, 8, emap=emap)
    assert out["counts"].sum() == int((ids % 2 == 0).sum())
