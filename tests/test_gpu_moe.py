"""GPU parity: router, alignment and the fused MoE layer against the oracle, through the C ABI.
Indices and the permutation are bit-exact; layer outputs within rtol = atol = 1e-2 of the float64
statement on the un-packed weights."""
import json
import os

import numpy as np
import pytest
import torch

from oracle import router as orouter, align as oalign, moe as omoe, layouts
from helpers import randn, pack_a, fp8_codes, assert_close

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(__file__), "golden")
RTOL = ATOL = 1e-2


def _route_gpu(mlk, logits, score_fun, n_groups, topk_groups, topk, bias=None, renorm=False):
    T = logits.shape[0]
    ids = torch.empty(T, topk, dtype=torch.int32, device="cuda")
    w = torch.empty(T, topk, dtype=logits.dtype, device="cuda")
    mlk.fused_routing_gate(logits.cuda(), score_fun, T, 4096, n_groups, topk_groups, ids, w, topk,
                           None if bias is None else bias.cuda(), renormalize=renorm)
    return ids.cpu(), w.cpu()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("score_fun", [0, 1])
@pytest.mark.parametrize("T,E,K", [(1, 8, 2), (16, 8, 2), (256, 8, 2), (77, 64, 6), (33, 256, 8), (5, 16, 16)])
def test_router_plain(mlk, dtype, score_fun, T, E, K):
    logits = randn((T, E), dtype, 1.0, 2025 + T)
    ids, w = _route_gpu(mlk, logits, score_fun, 1, 1, K)
    ids_o, w_o = orouter.route(logits, score_fun, 1, 1, K)
    assert torch.equal(ids, ids_o)
    assert torch.equal(w.view(torch.int16), w_o.view(torch.int16))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("score_fun", [0, 1])
@pytest.mark.parametrize("with_bias", [False, True])
def test_router_grouped_deepseek_configuration(mlk, dtype, score_fun, with_bias):
    T, E = 64, 256
    logits = randn((T, E), dtype, 1.0, 31)
    bias = randn((E,), dtype, 0.05, 32).abs() if with_bias else None
    ids, w = _route_gpu(mlk, logits, score_fun, 8, 4, 8, bias)
    ids_o, w_o = orouter.route(logits, score_fun, 8, 4, 8, bias)
    assert torch.equal(ids, ids_o)
    assert torch.equal(w.view(torch.int16), w_o.view(torch.int16))


@pytest.mark.parametrize("E,n_groups,topk_groups,K,score_fun,signed_bias", [
    (256, 128, 70, 8, 1, False),     # more than 64 groups: a lane holds several groups
    (256, 256, 40, 32, 0, False),    # one expert per group, the largest top-k
    (96, 3, 2, 7, 0, True),          # E not a power of two, bias of both signs (negative selection scores)
    (12, 4, 1, 3, 1, True),          # fewer candidates than picks inside the kept group: zeros are re-picked
    (200, 8, 8, 10, 0, False),
])
def test_router_general_groupings(mlk, E, n_groups, topk_groups, K, score_fun, signed_bias):
    T = 37
    logits = randn((T, E), torch.bfloat16, 2.0, 900 + E)
    bias = randn((E,), torch.bfloat16, 0.3, 901 + E) if signed_bias else None
    for renorm in (False, True):
        ids, w = _route_gpu(mlk, logits, score_fun, n_groups, topk_groups, K, bias, renorm=renorm)
        ids_o, w_o = orouter.route(logits, score_fun, n_groups, topk_groups, K, bias)
        assert torch.equal(ids, ids_o)
        w_o = orouter.renormalize(w_o) if renorm else w_o
        assert torch.equal(w.view(torch.int16), w_o.view(torch.int16))


def test_router_special_cases_and_renorm(mlk):
    eq = torch.zeros((3, 16), dtype=torch.bfloat16)
    ids, w = _route_gpu(mlk, eq, 0, 1, 1, 4)
    assert ids.tolist() == [[0, 1, 2, 3]] * 3
    logits = randn((128, 8), torch.bfloat16, 1.0, 5)
    ids, w = _route_gpu(mlk, logits, 0, 1, 1, 2, renorm=True)
    ids_o, w_o = orouter.route(logits, 0, 1, 1, 2)
    assert torch.equal(ids, ids_o)
    assert torch.equal(w.view(torch.int16), orouter.renormalize(w_o).view(torch.int16))
    # the same division done by torch on the GPU, as the reference's caller does it
    _, w_plain = _route_gpu(mlk, logits, 0, 1, 1, 2)
    wp = w_plain.cuda()
    assert torch.equal(w.cuda(), wp / wp.sum(dim=-1, keepdim=True))


def _align_gpu(mlk, ids, E, K, emap=None):
    T = ids.shape[0]
    n = T * K
    padded = n + E * 15
    dev = "cuda"
    s = torch.empty(padded, dtype=torch.int32, device=dev)
    cs = torch.empty(E + 1, dtype=torch.int32, device=dev)
    pn = torch.empty(1, dtype=torch.int32, device=dev)
    ei = torch.empty((padded + 15) // 16, dtype=torch.int32, device=dev)
    mlk.batched_routed_activation_indexed_to_expert_block_indexed(
        T, E, K, 16, ids.to(torch.int32).cuda(), s, cs, pn, ei,
        None if emap is None else torch.as_tensor(emap, dtype=torch.int32).cuda())
    return s.cpu().numpy(), cs.cpu().numpy(), int(pn.item()), ei.cpu().numpy()


def _compare_align(got, want):
    s, cs, pn, ei = got
    assert np.array_equal(s, want["sorted_token_ids"])
    assert np.array_equal(cs[:-1], want["cursors"][:-1]) and cs[-1] == want["cumsum"][-1]
    assert pn == want["padded_num_blocks"]
    assert np.array_equal(ei, want["experts_ids"])


def test_align_reference_example(mlk):
    ex = json.load(open(os.path.join(GOLD, "align_example_topk_ids.json")))
    ids = torch.tensor(ex["topk_ids"]).reshape(ex["tokens"], ex["topk"])
    _compare_align(_align_gpu(mlk, ids, ex["num_experts"], ex["topk"]),
                   oalign.align_tokens(ex["topk_ids"], ex["num_experts"]))


@pytest.mark.parametrize("T,K,E", [(1, 2, 8), (16, 2, 8), (64, 2, 8), (256, 2, 8), (33, 8, 256), (2048, 8, 256),
                                   (1000, 6, 64), (3, 1, 5)])
def test_align_random(mlk, T, K, E):
    rng = np.random.default_rng(T * 31 + K)
    ids = torch.from_numpy(np.stack([rng.choice(E, size=K, replace=False) for _ in range(T)]))
    _compare_align(_align_gpu(mlk, ids, E, K), oalign.align_tokens(ids.numpy(), E))


def test_align_expert_map(mlk):
    rng = np.random.default_rng(1)
    ids = torch.from_numpy(np.stack([rng.choice(16, size=4, replace=False) for _ in range(200)]))
    emap = np.array([e // 2 if e % 2 == 0 else -1 for e in range(16)])
    _compare_align(_align_gpu(mlk, ids, 8, 4, emap), oalign.align_tokens(ids.numpy(), 8, experts_map=emap))


def _pack_experts(w):
    return torch.stack([pack_a(w[e]) for e in range(w.shape[0])]).reshape(w.shape)


def _rel_l2(got, want64):
    g = got.detach().cpu().to(torch.float64).numpy()
    return float(np.linalg.norm(g - want64) / max(np.linalg.norm(want64), 1e-30))


def _outside(got, want64, rtol=RTOL, atol=ATOL):
    """Fraction of elements the element-wise check would reject."""
    g = got.detach().cpu().to(torch.float64).numpy()
    return float((np.abs(g - want64) > atol + rtol * np.abs(want64)).mean())


def _moe_case(mlk, T, E, K, H, I, dtype, seed, score="softmax", fp8=False, groups=None, bias=None, emap=None):
    """One fused_moe call against the float64 statement.  Weights are drawn so that the outputs are of order
    one (gate/up rows ~ N(0, 1/H), down rows ~ N(0, 4/I)): the tolerances then see every routed pair.  The
    same check is run against the expected value with the last pick of every token removed and must reject it."""
    from muxi_native_layout_kernels_amd.moe_planC import fused_moe
    x = randn((T, H), dtype, 1.0, seed)
    logits = randn((T, E), dtype, 1.0, seed + 1)
    std1, std2 = 1.0 / np.sqrt(H), 2.0 / np.sqrt(I)
    kw = {}
    if fp8:
        c1 = fp8_codes((E, 2 * I, H), seed + 2, std=1.0)
        c2 = fp8_codes((E, H, I), seed + 3, std=1.0)
        g = torch.Generator().manual_seed(seed + 4)
        s1 = ((torch.rand((E, 2 * I // 128, H // 128), generator=g) + 0.5) * std1).float()
        s2 = ((torch.rand((E, H // 128, I // 128), generator=g) + 0.5) * std2).float()
        w1u = omoe.dequant_experts(c1.numpy(), s1.numpy())
        w2u = omoe.dequant_experts(c2.numpy(), s2.numpy())
        w1p, w2p = _pack_experts(c1), _pack_experts(c2)
        kw = dict(w1_scale=s1.cuda(), w2_scale=s2.cuda(), block_shape=[128, 128], soft_fp8=True)
    else:
        w1u = randn((E, 2 * I, H), dtype, std1, seed + 2)
        w2u = randn((E, H, I), dtype, std2, seed + 3)
        w1p, w2p = _pack_experts(w1u), _pack_experts(w2u)
    n_groups, tk_groups = groups if groups else (1, 1)
    y = fused_moe(x.cuda(), w1p.cuda(), w2p.cuda(), logits.cuda(), K, True, use_grouped_topk=groups is not None,
                  num_expert_group=n_groups, topk_group=tk_groups, gating_bias=None if bias is None else bias.cuda(),
                  score_func=score, experts_map=None if emap is None else torch.as_tensor(emap).cuda(), **kw)
    assert y.shape == x.shape and y.dtype == dtype
    ids, wts = orouter.route(logits, 0 if score == "softmax" else 1, n_groups, tk_groups, K, bias)
    wts = orouter.renormalize(wts)
    want = omoe.moe_expected(x, w1u, w2u, ids, wts, round_h_to=dtype, expert_map=emap)
    assert_close(y, want, RTOL, ATOL, "fused_moe T=%d" % T)
    assert _rel_l2(y, want) <= 1e-2
    assert np.abs(want).mean() > 0.05, "the expected output carries no signal"
    if K > 1 and emap is None:
        # negative control: without the last pick of every token the same check must fail
        fewer = omoe.moe_expected(x, w1u, w2u, ids[:, :K - 1], wts[:, :K - 1], round_h_to=dtype)
        assert _outside(y, fewer) > 0.2 and _rel_l2(y, fewer) > 1e-2, "the check cannot see a dropped pick"
    return y


@pytest.mark.parametrize("T", [1, 2, 16, 17, 40, 64, 70, 90, 100, 128, 256, 300])
def test_fused_moe_small_shape(mlk, T):
    _moe_case(mlk, T, 8, 2, 256, 384, torch.bfloat16, 100 + T)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_fused_moe_dtypes_and_determinism(mlk, dtype):
    y1 = _moe_case(mlk, 40, 8, 2, 512, 256, dtype, 7)
    y2 = _moe_case(mlk, 40, 8, 2, 512, 256, dtype, 7)
    assert torch.equal(y1, y2)


@pytest.mark.parametrize("T", [1, 16, 70, 130])
def test_fused_moe_soft_fp8(mlk, T):
    _moe_case(mlk, T, 8, 2, 256, 384, torch.bfloat16, 300 + T, fp8=True)


@pytest.mark.parametrize("T,E,K,H,I", [
    (256, 8, 2, 256, 384),      # six token blocks per task: panels of 96 tokens
    (300, 4, 2, 512, 384),      # eight blocks (panels of 128 tokens), then a pass of 44 tokens on the row-shared kernels
    (200, 2, 1, 768, 128),      # one k window per slice boundary case: I = 128
    (256, 3, 3, 256, 1024),     # every token on every expert: tasks of 256 tokens in two panels each
])
def test_fused_moe_soft_fp8_panel_kernels(mlk, T, E, K, H, I):
    """Soft-FP8 weights with more than 64 tokens per pass over an expert run the panel kernels (32x32x16 products);
    switching them off (experiment switch 9) must give the row-shared kernels' result to the same tolerance."""
    from muxi_native_layout_kernels_amd import _lib
    import ctypes
    lib = _lib.load()
    plan = (ctypes.c_int32 * 8)()
    assert lib.mlk_moe_plan(T, E, K, H, I, 2, ctypes.addressof(plan)) == 0 and plan[0] == 4, "this case must take the panel path"
    y1 = _moe_case(mlk, T, E, K, H, I, torch.bfloat16, 2100 + T, fp8=True)
    lib.mlk_set_tunable(9, 1)
    try:
        assert lib.mlk_moe_plan(T, E, K, H, I, 2, ctypes.addressof(plan)) == 0 and plan[0] == 3
        y2 = _moe_case(mlk, T, E, K, H, I, torch.bfloat16, 2100 + T, fp8=True)
    finally:
        lib.mlk_set_tunable(9, 0)
    assert_close(y1, y2.double().cpu().numpy(), RTOL, ATOL, "panel kernels vs row-shared kernels")


@pytest.mark.parametrize("switch", [1, 3, 17, 18, 20, 24])
def test_fused_moe_soft_fp8_panel_down_shapes(mlk, switch):
    """The panel down projection on the long LDS ring (one workgroup per CU) and on the short one (two per CU), in
    1 to 8 K slices, each asked for through experiment switch 10 (slices + 16 x short ring) and checked against
    the float64 statement."""
    from muxi_native_layout_kernels_amd import _lib
    import ctypes
    lib = _lib.load()
    T, E, K, H, I = 256, 8, 2, 256, 1024
    plan = (ctypes.c_int32 * 8)()
    lib.mlk_set_tunable(10, switch)
    try:
        assert lib.mlk_moe_plan(T, E, K, H, I, 2, ctypes.addressof(plan)) == 0 and plan[0] == 4
        assert (plan[4], plan[5]) == (switch & 15, 2 if switch >> 4 else 1)
        _moe_case(mlk, T, E, K, H, I, torch.bfloat16, 2300 + switch, fp8=True)
    finally:
        lib.mlk_set_tunable(10, 0)


def test_fused_moe_soft_fp8_panel_down_two_per_cu(mlk):
    """A shape whose down projection fills two workgroups per CU by itself (8 row tiles x 8 experts x 8 K slices):
    the plan picks the short-ring kernel, and the result is checked against the float64 statement."""
    from muxi_native_layout_kernels_amd import _lib
    import ctypes
    T, E, K, H, I = 256, 8, 2, 2048, 4096
    plan = (ctypes.c_int32 * 8)()
    assert _lib.load().mlk_moe_plan(T, E, K, H, I, 2, ctypes.addressof(plan)) == 0
    assert plan[0] == 4 and (plan[4], plan[5]) == (8, 2), list(plan)
    _moe_case(mlk, T, E, K, H, I, torch.bfloat16, 2400, fp8=True)


def test_fused_moe_grouped_sigmoid_bias(mlk):
    E = 64
    bias = randn((E,), torch.bfloat16, 0.05, 9).abs()
    _moe_case(mlk, 24, E, 8, 256, 128, torch.bfloat16, 500, score="sigmoid", groups=(8, 4), bias=bias)


def test_fused_moe_expert_map(mlk):
    emap = np.array([0, -1, 1, -1, 2, -1, 3, -1], dtype=np.int32)
    # local experts 0..3 hold the weights of global experts 0, 2, 4, 6
    from muxi_native_layout_kernels_amd.moe_planC import fused_moe
    T, E, K, H, I = 32, 8, 2, 256, 256
    dtype = torch.bfloat16
    x = randn((T, H), dtype, 1.0, 1)
    logits = randn((T, E), dtype, 1.0, 2)
    w1 = randn((4, 2 * I, H), dtype, 1.0 / np.sqrt(H), 3)
    w2 = randn((4, H, I), dtype, 2.0 / np.sqrt(I), 4)
    y = fused_moe(x.cuda(), _pack_experts(w1).cuda(), _pack_experts(w2).cuda(), logits.cuda(), K, True,
                  experts_map=torch.as_tensor(emap).cuda())
    ids, wts = orouter.route(logits, 0, 1, 1, K)
    want = omoe.moe_expected(x, w1, w2, ids, orouter.renormalize(wts), round_h_to=dtype, expert_map=emap)
    assert_close(y, want, RTOL, ATOL, "expert map")
    # negative control: treating the absent experts as present (weights of local expert e // 2) must fail the check
    wrong = omoe.moe_expected(x, w1, w2, ids, orouter.renormalize(wts), round_h_to=dtype,
                              expert_map=np.arange(8) // 2)
    assert _outside(y, wrong) > 0.2


@pytest.mark.parametrize("dtype,fp8,E,K,H,I", [
    (torch.float16, False, 8, 2, 256, 384),
    (torch.bfloat16, False, 16, 6, 512, 256),
    (torch.bfloat16, True, 16, 8, 384, 512),
    (torch.bfloat16, False, 64, 16, 128, 128),
    (torch.bfloat16, False, 32, 20, 256, 128),      # top-k above 16: the general decode kernels
])
def test_fused_moe_single_token(mlk, dtype, fp8, E, K, H, I):
    """One token runs GeMV-style kernels; switching them off must give the grouped kernels' result
    to the same tolerance."""
    from muxi_native_layout_kernels_amd import _lib
    y1 = _moe_case(mlk, 1, E, K, H, I, dtype, 900 + K, fp8=fp8)
    _lib.load().mlk_moe_set_tile_path(3)
    try:
        y2 = _moe_case(mlk, 1, E, K, H, I, dtype, 900 + K, fp8=fp8)
    finally:
        _lib.load().mlk_moe_set_tile_path(1)
    assert_close(y1, y2.double().cpu().numpy(), RTOL, ATOL, "single-token kernels vs grouped kernels")


@pytest.mark.parametrize("dtype,fp8,T,E,K,score,groups,with_bias", [
    (torch.bfloat16, False, 1, 8, 2, "softmax", None, False),       # the Mixtral routing
    (torch.float16, False, 1, 8, 2, "softmax", None, False),
    (torch.bfloat16, True, 7, 8, 2, "softmax", None, False),
    (torch.bfloat16, False, 33, 64, 8, "sigmoid", (8, 4), True),
    (torch.bfloat16, True, 1, 48, 6, "softmax", (4, 2), False),     # expert count that is no power of two
])
def test_whole_layer_call_leaves_the_routing_in_its_buffers(mlk, dtype, fp8, T, E, K, score, groups, with_bias):
    """`mlk_fused_moe` (one library call per layer) writes the router's picks into the ids / weights buffers it is
    given: they must be the oracle's bit for bit, and the layer output must pass the same check as ever."""
    from muxi_native_layout_kernels_amd import moe_planC
    H, I = 256, 384
    bias = randn((E,), dtype, 0.05, 55).abs() if with_bias else None
    n_groups, tk_groups = groups if groups else (1, 1)
    ids_buf, w_buf = moe_planC._routing_buffers(T, K, dtype, torch.device("cuda", torch.cuda.current_device()))
    ids_buf.fill_(-7)
    w_buf.zero_()
    _moe_case(mlk, T, E, K, H, I, dtype, 4000 + T, score=score, fp8=fp8, groups=groups, bias=bias)
    logits = randn((T, E), dtype, 1.0, 4000 + T + 1)
    ids_o, w_o = orouter.route(logits, 0 if score == "softmax" else 1, n_groups, tk_groups, K, bias)
    assert torch.equal(ids_buf.cpu(), ids_o)
    assert torch.equal(w_buf.cpu().view(torch.int16), orouter.renormalize(w_o).view(torch.int16))


@pytest.mark.parametrize("slices", [2, 4])
@pytest.mark.parametrize("T,E,K,fp8", [(3, 8, 2, False), (16, 16, 8, False), (9, 8, 2, True)])
def test_fused_moe_decode_k_sliced_down(mlk, slices, T, E, K, fp8):
    """Up to 16 tokens the down projection may slice K across workgroups (the last one to arrive folds
    the slices in slice order): same result to tolerance, identical from call to call."""
    from muxi_native_layout_kernels_amd import _lib
    lib = _lib.load()
    lib.mlk_set_tunable(7, slices)
    try:
        y1 = _moe_case(mlk, T, E, K, 256, 384, torch.bfloat16, 700 + T, fp8=fp8)
        y2 = _moe_case(mlk, T, E, K, 256, 384, torch.bfloat16, 700 + T, fp8=fp8)
    finally:
        lib.mlk_set_tunable(7, 0)
    assert torch.equal(y1, y2)


@pytest.mark.parametrize("T,E,K,H,I,fp8", [
    (1, 4, 1, 128, 128, False),      # one pick: all 16 waves of the down kernel on one pair
    (1, 8, 3, 256, 640, False),      # 15 of 16 waves used, 5 K slices per pair, 20 k tiles
    (1, 8, 5, 128, 384, True),       # fp8 tiles of 64 k: 6 tiles over 3 waves per pair
    (1, 16, 16, 128, 256, True),     # one wave per pair
    (2, 3, 3, 128, 128, False),      # every token picks every expert
    (5, 4, 2, 384, 128, True),       # K-sliced fp8 down projection with 4 k tiles per slice... (I/32 = 4)
    (16, 2, 1, 128, 256, False),
    (13, 64, 5, 256, 128, True),     # 65 routed pairs: one more than the in-kernel alignment takes
])
def test_fused_moe_odd_shapes(mlk, T, E, K, H, I, fp8):
    _moe_case(mlk, T, E, K, H, I, torch.bfloat16, 1000 + T + K, fp8=fp8)


@pytest.mark.parametrize("T", [1, 4, 16, 40])
@pytest.mark.parametrize("fp8", [False, True])
def test_fused_moe_deepseek_style_routing(mlk, T, fp8):
    """256 experts in 8 groups, 4 groups kept, top-8, sigmoid scores with a selection bias - the only routing
    configuration the reference's own router accepts (fused_gating.h:22-34, test_muxi_moe.py:41-50)."""
    E = 256
    bias = randn((E,), torch.bfloat16, 0.05, 77).abs()
    _moe_case(mlk, T, E, 8, 256, 128, torch.bfloat16, 1200 + T, score="sigmoid", groups=(8, 4), bias=bias, fp8=fp8)


def test_fused_moe_single_token_expert_map(mlk):
    """A routed expert that is not held locally contributes nothing."""
    from muxi_native_layout_kernels_amd.moe_planC import fused_moe
    E, K, H, I = 8, 4, 256, 256
    dtype = torch.bfloat16
    emap = np.array([0, -1, 1, -1, 2, -1, 3, -1], dtype=np.int32)
    w1 = randn((4, 2 * I, H), dtype, 1.0 / np.sqrt(H), 3)
    w2 = randn((4, H, I), dtype, 2.0 / np.sqrt(I), 4)
    w1p, w2p = _pack_experts(w1).cuda(), _pack_experts(w2).cuda()
    for seed in range(4):
        x = randn((1, H), dtype, 1.0, 10 + seed)
        logits = randn((1, E), dtype, 1.0, 20 + seed)
        y = fused_moe(x.cuda(), w1p, w2p, logits.cuda(), K, True, experts_map=torch.as_tensor(emap).cuda())
        ids, wts = orouter.route(logits, 0, 1, 1, K)
        want = omoe.moe_expected(x, w1, w2, ids, orouter.renormalize(wts), round_h_to=dtype, expert_map=emap)
        assert_close(y, want, RTOL, ATOL, "single token, expert map")


def test_fused_moe_matches_torch_path_on_gpu(mlk):
    """The reference's own test recipe: compare with the pure-torch MoE run on the GPU in the same dtype,
    atol 0.1 / rtol 0.05 (benchmark_and_test/test_muxi_moe.py:111)."""
    from muxi_native_layout_kernels_amd.moe_planC import fused_moe
    from muxi_native_layout_kernels_amd import utils
    T, E, K, H, I = 48, 8, 2, 512, 768
    dtype = torch.bfloat16
    x = (torch.rand((T, H), generator=torch.Generator().manual_seed(1)) / 100).to(dtype)
    logits = randn((T, E), dtype, 1.0, 2)
    w1 = (torch.rand((E, 2 * I, H), generator=torch.Generator().manual_seed(3)) / 10).to(dtype)
    w2 = (torch.rand((E, H, I), generator=torch.Generator().manual_seed(4)) / 10).to(dtype)
    y = fused_moe(x.cuda(), _pack_experts(w1).cuda(), _pack_experts(w2).cuda(), logits.cuda(), K, True)
    ref = utils.fused_moe(x.cuda(), w1.cuda(), w2.cuda(), logits.cuda(), K, num_expert_group=1, topk_group=1,
                          global_num_experts=E, renormalize=True)
    torch.testing.assert_close(y, ref, atol=0.1, rtol=0.05)


def test_low_level_fused_experts_compute_signature(mlk):
    """Call sequence of the reference's Python entry (muxi_moe_planC.py:44-146) on the low-level ops."""
    T, E, K, H, I = 20, 8, 2, 256, 256
    dtype = torch.float16
    x = randn((T, H), dtype, 1.0, 1).cuda()
    logits = randn((T, E), dtype, 1.0, 2).cuda()
    w1u = randn((E, 2 * I, H), dtype, 1.0 / np.sqrt(H), 3)
    w2u = randn((E, H, I), dtype, 2.0 / np.sqrt(I), 4)
    w1, w2 = _pack_experts(w1u).cuda(), _pack_experts(w2u).cuda()
    ids = torch.empty(T, K, dtype=torch.int32, device="cuda")
    wts = torch.empty(T, K, dtype=dtype, device="cuda")
    mlk.fused_routing_gate(logits, 0, T, H, 1, 1, ids, wts, K, None)
    wts = wts / wts.sum(dim=-1, keepdim=True)
    padded = K * T + E * 15
    sorted_ids = torch.full((padded,), T * K, dtype=torch.int32, device="cuda")
    cumsum = torch.empty(E + 1, dtype=torch.int32, device="cuda")
    pn = torch.empty(1, dtype=torch.int32, device="cuda")
    eids = torch.empty((padded + 15) // 16, dtype=torch.int32, device="cuda")
    C = torch.zeros(K * 2 * I * T, dtype=dtype, device="cuda")
    y = torch.zeros_like(x)
    mlk.fused_experts_compute(w1, w2, x, T, E, K, ids, wts, sorted_ids, cumsum, pn, eids, C, y, APerWarp=2, splitK=3,
                              tile_m_2=128, tile_n_2=16, tile_k_2=128, block_dim_x_gemm=256, experts_map=None)
    want = omoe.moe_expected(x.cpu(), w1u, w2u, ids.cpu(), wts.cpu(), round_h_to=dtype)
    assert_close(y, want, RTOL, ATOL, "low-level")
    assert int(pn.item()) == oalign.align_tokens(ids.cpu().numpy(), E)["padded_num_blocks"]


class _Lazy:
    """Per-expert weights fetched on demand (only the experts the sampled tokens use reach the host)."""

    def __init__(self, fetch, shape):
        self.fetch, self.shape, self.cache = fetch, shape, {}

    def __getitem__(self, e):
        if e not in self.cache:
            self.cache[e] = self.fetch(e)
        return self.cache[e]


def _sample_tokens(T):
    return list(range(T)) if T <= 4 else sorted({0, T // 2 + 1, T - 1})


def _whole_tensor_against_torch_path(y, x, w1, w2, logits, K, E):
    """Every token of `y` against the shipped pure-torch MoE run on the GPU in the same dtype, with the reference's
    own tolerances (benchmark_and_test/test_muxi_moe.py:111: atol 0.1, rtol 0.05).  The torch path breaks ties
    between equal T-rounded scores as `torch.topk` pleases, the kernels take the lower expert id; with N(0, 0.02)
    weights a different expert is a different output, so tokens whose two selections differ are left to the float64
    check of the sampled tokens, and there may only be a few of them."""
    from muxi_native_layout_kernels_amd import utils
    ref = utils.fused_moe(x, w1, w2, logits, K, num_expert_group=1, topk_group=1, global_num_experts=E, renormalize=True)
    _, ids_torch = utils._select_experts(logits, K, 1, 1, True, None, "softmax", x.dtype)
    ids_ours, _ = orouter.route(logits.cpu(), 0, 1, 1, K)
    same = (ids_torch.sort(dim=-1).values.cpu() == ids_ours.sort(dim=-1).values.to(ids_torch.dtype)).all(dim=-1)
    assert int(same.sum()) >= 0.9 * y.shape[0], "too many routing ties: %d of %d tokens" % (int((~same).sum()), y.shape[0])
    rows = same.nonzero().flatten().cuda()
    torch.testing.assert_close(y[rows], ref[rows], atol=0.1, rtol=0.05)
    return int(same.sum())


@pytest.mark.parametrize("T", [1, 16, 64, 256])
def test_fused_moe_mixtral_shape(mlk, T):
    """E=8, top-2, H=4096, I=14336, bf16 weights ~ N(0, 0.02) at full size; the oracle evaluates sampled tokens
    (from different token blocks) on the experts they select.  64 and 256 tokens run the row-shared kernels
    and the combine kernel."""
    from muxi_native_layout_kernels_amd.moe_planC import fused_moe
    E, K, H, I = 8, 2, 4096, 14336
    dtype = torch.bfloat16
    x = randn((T, H), dtype, 1.0, 2025)
    logits = randn((T, E), dtype, 1.0, 2026)
    g = torch.Generator(device="cuda").manual_seed(2027)
    w1u = (torch.randn((E, 2 * I, H), generator=g, device="cuda") * 0.02).to(dtype)
    w2u = (torch.randn((E, H, I), generator=g, device="cuda") * 0.02).to(dtype)
    w1p = mlk.pack_layout_a(w1u).view(E, 2 * I, H)
    w2p = mlk.pack_layout_a(w2u).view(E, H, I)
    y = fused_moe(x.cuda(), w1p, w2p, logits.cuda(), K, True)
    y2 = fused_moe(x.cuda(), w1p, w2p, logits.cuda(), K, True)
    assert torch.equal(y, y2)
    ids, wts = orouter.route(logits, 0, 1, 1, K)
    wts = orouter.renormalize(wts)
    tok = _sample_tokens(T)
    want = omoe.moe_expected(x[tok], _Lazy(lambda e: w1u[e].cpu(), (E, 2 * I, H)), _Lazy(lambda e: w2u[e].cpu(), (E, H, I)),
                             ids[tok], wts[tok], round_h_to=dtype)
    assert_close(y[tok], want, RTOL, ATOL, "mixtral T=%d" % T)
    assert _rel_l2(y[tok], want) <= 1e-2 and np.abs(want).mean() > 0.3
    fewer = omoe.moe_expected(x[tok], _Lazy(lambda e: w1u[e].cpu(), (E, 2 * I, H)),
                              _Lazy(lambda e: w2u[e].cpu(), (E, H, I)), ids[tok][:, :1], wts[tok][:, :1], round_h_to=dtype)
    assert _outside(y[tok], fewer) > 0.2
    # every token is finite and of the expected size (the sampled ones are checked exactly)
    yn = y.float()
    assert torch.isfinite(yn).all() and 0.2 < float(yn.abs().mean()) < 20.0
    # and every token against the torch path on the GPU, as the reference's own test compares whole outputs
    _whole_tensor_against_torch_path(y, x.cuda(), w1u, w2u, logits.cuda(), K, E)


@pytest.mark.parametrize("T,unit_scales", [(1, False), (16, True), (16, False), (64, False), (256, False)])
def test_fused_moe_mixtral_shape_soft_fp8(mlk, T, unit_scales):
    """The soft-FP8 variant of the same layer: e4m3 bytes from N(0, 1) * 16 clipped to +-448, one fp32 scale per
    128 x 128 block (random factors around 1e-3, the general widening path; or all ones, which are powers of two and
    take the scaled converter)."""
    from muxi_native_layout_kernels_amd.moe_planC import fused_moe
    from oracle import softfp8
    E, K, H, I = 8, 2, 4096, 14336
    dtype = torch.bfloat16
    x = randn((T, H), dtype, 1.0, 3025)
    logits = randn((T, E), dtype, 1.0, 3026)
    g = torch.Generator(device="cuda").manual_seed(3027)
    c1 = (torch.randn((E, 2 * I, H), generator=g, device="cuda") * 16).clamp_(-448, 448).to(torch.float8_e4m3fn).view(torch.uint8)
    c2 = (torch.randn((E, H, I), generator=g, device="cuda") * 16).clamp_(-448, 448).to(torch.float8_e4m3fn).view(torch.uint8)
    if unit_scales:
        s1 = torch.ones((E, 2 * I // 128, H // 128), dtype=torch.float32, device="cuda")
        s2 = torch.ones((E, H // 128, I // 128), dtype=torch.float32, device="cuda")
    else:
        s1 = (torch.rand((E, 2 * I // 128, H // 128), generator=g, device="cuda") + 0.5) * 1.0e-3
        s2 = (torch.rand((E, H // 128, I // 128), generator=g, device="cuda") + 0.5) * 1.3e-3
    w1p = mlk.pack_layout_a(c1).view(E, 2 * I, H)
    w2p = mlk.pack_layout_a(c2).view(E, H, I)
    y = fused_moe(x.cuda(), w1p, w2p, logits.cuda(), K, True, w1_scale=s1, w2_scale=s2, block_shape=[128, 128],
                  soft_fp8=True)
    y2 = fused_moe(x.cuda(), w1p, w2p, logits.cuda(), K, True, w1_scale=s1, w2_scale=s2, block_shape=[128, 128],
                   soft_fp8=True)
    assert torch.equal(y, y2)
    ids, wts = orouter.route(logits, 0, 1, 1, K)
    wts = orouter.renormalize(wts)
    tok = _sample_tokens(T)
    w1l = _Lazy(lambda e: softfp8.dequant_weight_f32(c1[e].cpu().numpy(), s1[e].cpu().numpy()), (E, 2 * I, H))
    w2l = _Lazy(lambda e: softfp8.dequant_weight_f32(c2[e].cpu().numpy(), s2[e].cpu().numpy()), (E, H, I))
    want = omoe.moe_expected(x[tok], w1l, w2l, ids[tok], wts[tok], round_h_to=dtype)
    # outputs are huge with unit scales (weights ~ N(0, 16)): the check is relative, the absolute term is scaled up
    scale = max(1.0, float(np.abs(want).mean()))
    assert_close(y[tok], want, RTOL, ATOL * scale, "mixtral soft-FP8 T=%d" % T)
    assert _rel_l2(y[tok], want) <= 1e-2
    fewer = omoe.moe_expected(x[tok], w1l, w2l, ids[tok][:, :1], wts[tok][:, :1], round_h_to=dtype)
    assert _outside(y[tok], fewer, RTOL, ATOL * scale) > 0.2
    assert torch.isfinite(y.float()).all()
    if not unit_scales:
        # every token against the torch path on weights widened and scaled in bf16 beforehand, the reference's
        # recipe for soft-FP8 (benchmark_and_test/test_muxi_moe_softfp8.py:113-129)
        from muxi_native_layout_kernels_amd import utils
        w1w = utils.scale_whole_tensor(c1.view(torch.float8_e4m3fn), s1)
        w2w = utils.scale_whole_tensor(c2.view(torch.float8_e4m3fn), s2)
        _whole_tensor_against_torch_path(y, x.cuda(), w1w, w2w, logits.cuda(), K, E)


# -------------------------------------------------------------- the reference's own test grid
def _pack_view_permute(w):
    """The packing loop of the reference's tests (test_muxi_moe.py:73-81) for all experts at once."""
    e, n, k = w.shape
    return w.view(e, n // 16, 16, k // 8, 8).permute(0, 1, 3, 2, 4).contiguous().view(e, n, k)


@pytest.mark.parametrize("m", [8, 16, 64, 256, 272, 384, 512, 1024, 2048])
@pytest.mark.parametrize("n,k,e", [(256, 7168, 256), (768, 2048, 128)])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_reference_grid(mlk, m, n, k, e, dtype):
    """benchmark_and_test/test_muxi_moe.py:14-111 at its own shapes and with its own recipe: top-8, sigmoid, 8 groups
    of which 4 are kept, renormalised, `rand / 100` activations, `rand / 10` weights, `rand` logits, compared with
    the pure-torch MoE run on the GPU in the same dtype to atol 0.1 / rtol 0.05.  On top of that, sampled tokens
    are checked against the float64 statement with the router's own tie rule to rtol = atol = 1e-2."""
    from muxi_native_layout_kernels_amd.moe_planC import fused_moe
    from muxi_native_layout_kernels_amd import utils
    topk = 8
    torch.manual_seed(2025)
    a = torch.rand((m, k), device="cuda", dtype=dtype) / 100
    w1 = torch.rand((e, 2 * n, k), device="cuda", dtype=dtype) / 10
    w2 = torch.rand((e, k, n), device="cuda", dtype=dtype) / 10
    score = torch.rand((m, e), device="cuda", dtype=dtype)
    out = fused_moe(a, _pack_view_permute(w1), _pack_view_permute(w2), score, topk, renormalize=True,
                    use_grouped_topk=True, num_expert_group=8, topk_group=4, gating_bias=None, score_func="sigmoid")
    ref = utils.fused_moe(a.clone(), w1, w2, score, topk, 8, 4, global_num_experts=e, renormalize=True,
                          e_score_correction_bias=None, score_func="sigmoid")
    torch.testing.assert_close(out, ref, atol=0.1, rtol=0.05)
    assert float(ref.float().abs().mean()) > 1.0            # the recipe gives outputs far above the tolerance
    # float64 statement on sampled tokens
    tok = sorted({0, m // 2, m - 1})
    ids, wts = orouter.route(score[tok].cpu(), 1, 8, 4, topk)      # rows are routed independently
    wts = orouter.renormalize(wts)
    w1l = _Lazy(lambda i: w1[i].cpu(), (e, 2 * n, k))
    w2l = _Lazy(lambda i: w2[i].cpu(), (e, k, n))
    want = omoe.moe_expected(a[tok].cpu(), w1l, w2l, ids, wts, round_h_to=dtype)
    assert_close(out[tok], want, RTOL, ATOL, "reference grid m=%d" % m)
    fewer = omoe.moe_expected(a[tok].cpu(), w1l, w2l, ids[:, :topk - 1], wts[:, :topk - 1], round_h_to=dtype)
    assert _outside(out[tok], fewer) > 0.5


@pytest.mark.parametrize("m", [8, 64, 244, 256, 272, 512, 1024, 2048])
@pytest.mark.parametrize("n,k,e", [(256, 7168, 256), (768, 2048, 128)])
def test_reference_grid_soft_fp8(mlk, m, n, k, e):
    """benchmark_and_test/test_muxi_moe_softfp8.py:57-129: the same grid with float8_e4m3fn weights and
    `rand * 2` block scales, expected value from `scale_whole_tensor` + the pure-torch MoE in bf16."""
    from muxi_native_layout_kernels_amd.moe_planC import fused_moe
    from muxi_native_layout_kernels_amd import utils
    from oracle import softfp8
    topk, dtype = 8, torch.bfloat16
    torch.manual_seed(2025)
    a = torch.rand((m, k), device="cuda", dtype=dtype) / 100
    w1 = (torch.rand((e, 2 * n, k), device="cuda", dtype=dtype) / 10).to(torch.float8_e4m3fn)
    w2 = (torch.rand((e, k, n), device="cuda", dtype=dtype) / 10).to(torch.float8_e4m3fn)
    w1_scale = torch.rand((e, 2 * n // 128, k // 128), device="cuda", dtype=torch.float32) * 2
    w2_scale = torch.rand((e, k // 128, n // 128), device="cuda", dtype=torch.float32) * 2
    score = torch.rand((m, e), device="cuda", dtype=dtype)
    out = fused_moe(a, _pack_view_permute(w1.view(torch.uint8)), _pack_view_permute(w2.view(torch.uint8)), score, topk,
                    renormalize=True, use_grouped_topk=True, num_expert_group=8, topk_group=4, gating_bias=None,
                    score_func="sigmoid", w1_scale=w1_scale, w2_scale=w2_scale, block_shape=[128, 128], soft_fp8=True)
    ref = utils.fused_moe(a.clone(), utils.scale_whole_tensor(w1, w1_scale), utils.scale_whole_tensor(w2, w2_scale),
                          score, topk, 8, 4, global_num_experts=e, renormalize=True, e_score_correction_bias=None,
                          score_func="sigmoid")
    torch.testing.assert_close(out, ref, atol=0.1, rtol=0.05)
    assert float(ref.float().abs().mean()) > 1.0
    tok = sorted({0, m // 2, m - 1})
    ids, wts = orouter.route(score[tok].cpu(), 1, 8, 4, topk)
    wts = orouter.renormalize(wts)
    c1, c2 = w1.view(torch.uint8), w2.view(torch.uint8)
    w1l = _Lazy(lambda i: softfp8.dequant_weight_f32(c1[i].cpu().numpy(), w1_scale[i].cpu().numpy()), (e, 2 * n, k))
    w2l = _Lazy(lambda i: softfp8.dequant_weight_f32(c2[i].cpu().numpy(), w2_scale[i].cpu().numpy()), (e, k, n))
    want = omoe.moe_expected(a[tok].cpu(), w1l, w2l, ids, wts, round_h_to=dtype)
    assert_close(out[tok], want, RTOL, ATOL, "reference grid soft-FP8 m=%d" % m)


@pytest.mark.parametrize("T", [171, 172, 244, 256, 500])
def test_fused_moe_soft_fp8_many_experts_near_a_full_pass(mlk, T):
    """256 experts, top-8, soft-FP8 with 170 to 256 tokens in a pass: one token block per task, so the decode down
    kernel runs with an output tile of up to 256 tokens; the rows per wave are chosen so that it fits the LDS."""
    E = 256
    bias = randn((E,), torch.bfloat16, 0.05, 78).abs()
    _moe_case(mlk, T, E, 8, 512, 256, torch.bfloat16, 1500 + T, score="sigmoid", groups=(8, 4), bias=bias, fp8=True)
