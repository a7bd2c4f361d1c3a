"""GPU parity on seeded random shapes through the public entry points: whatever the tables, the borrowed rows, the
heuristics for unscanned shapes and the guards choose for a shape must give the oracle's result (rtol = atol = 1e-2
for the products; bit-exact for the relayouts).  The fixed cases elsewhere pin named kernels; these pin the dispatch."""
import warnings

import numpy as np
import pytest
import torch

from oracle import gemm as ogemm, layouts, router as orouter, moe as omoe
from helpers import randn, pack_a, pack_b, fp8_codes, assert_close, bits

pytestmark = pytest.mark.gpu
RTOL = ATOL = 1e-2


def _shapes(seed, count, n_max, k_max, m_max):
    rng = np.random.RandomState(seed)
    out = []
    for _ in range(count):
        n = 128 * int(rng.randint(1, n_max // 128 + 1))
        k = 128 * int(rng.randint(1, k_max // 128 + 1))
        m = int(rng.choice([1, 2, 3, 5, 8, 15, 16, 17, 31, 32, 33, 48, 63, 64, 65, 80, 100, 128, 130, 200, 256, 300]))
        out.append((n, k, min(m, m_max)))
    return out


@pytest.mark.parametrize("n,k,m", _shapes(11, 14, 2048, 2048, 300))
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_gemm_layout_a_random_shapes(mlk, n, k, m, dtype):
    w = randn((n, k), dtype, 0.05, n + k)
    b = randn((m, k), dtype, 1.0, n + k + m)
    bias = randn((1, n), dtype, 1.0, 7)
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        c = mlk.gemm_layoutA(pack_a(w).cuda(), b.cuda(), alpha=0.5, bias=bias.cuda())
    assert_close(c, ogemm.linear_expected(w, b, 0.5, bias), RTOL, ATOL, "gemm_layoutA %dx%d M=%d" % (n, k, m))


@pytest.mark.parametrize("n,k,m", _shapes(12, 10, 2048, 2048, 200))
def test_gemm_soft_fp8_random_shapes(mlk, n, k, m):
    codes = fp8_codes((n, k), n + k)
    g = torch.Generator().manual_seed(n + m)
    scale = (torch.rand((n // 128, k // 128), generator=g) * 0.02 + 0.001).float()
    b = randn((m, k), torch.bfloat16, 1.0, k + m)
    c = mlk.gemm_layoutA_linear(pack_a(codes).cuda(), b.cuda(), scale_matrix=scale.cuda())
    assert_close(c, ogemm.softfp8_linear_expected(codes.numpy(), scale.numpy(), b), RTOL, ATOL,
                 "soft-fp8 gemm %dx%d M=%d" % (n, k, m))


@pytest.mark.parametrize("n,k,m", [(n, k, 16 * max(1, m // 16)) for n, k, m in _shapes(13, 10, 2048, 2048, 256)])
def test_native_chain_random_shapes(mlk, n, k, m):
    """layoutB -> gemm_layoutABC -> reLayoutC equals gemm_layoutAB_ContinuousC bit for bit and the oracle to tolerance."""
    dtype = torch.bfloat16
    w = randn((n, k), dtype, 0.05, n + 3 * k)
    b = randn((m, k), dtype, 1.0, n + k + 5 * m)
    a = pack_a(w).cuda()
    bn = mlk.layoutB(b.cuda())
    assert torch.equal(bn.cpu().view(torch.int16), pack_b(b).view(torch.int16).reshape(bn.shape))
    c_rm = mlk.gemm_layoutAB_ContinuousC(a, bn)
    c_nat = mlk.gemm_layoutABC(a, bn)
    assert torch.equal(mlk.reLayoutC(c_nat), c_rm)
    assert_close(c_rm, ogemm.linear_expected(w, b), RTOL, ATOL, "native chain %dx%d M=%d" % (n, k, m))


def _gemv_shapes(seed, count):
    rng = np.random.RandomState(seed)
    return [(16 * int(rng.randint(1, 257)), 64 * int(rng.randint(1, 65))) for _ in range(count)]


@pytest.mark.parametrize("n,k", _gemv_shapes(14, 12))
def test_gemv_random_shapes(mlk, n, k):
    for dtype in (torch.float16, torch.bfloat16):
        w = randn((n, k), dtype, 0.05, n + k)
        x = randn((1, k), dtype, 1.0, n)
        assert_close(mlk.gemv_layoutA(pack_a(w).cuda(), x.cuda()), ogemm.linear_expected(w, x), RTOL, ATOL,
                     "gemv %dx%d" % (n, k))
    codes = fp8_codes((n, k), n * 3 + k)
    g = torch.Generator().manual_seed(k)
    scale = (torch.rand(((n + 127) // 128, (k + 127) // 128), generator=g) * 0.02 + 0.001).float()
    x = randn((1, k), torch.bfloat16, 1.0, n + 1)
    assert_close(mlk.gemv_layoutA(pack_a(codes).cuda(), x.cuda(), scale_matrix=scale.cuda()),
                 ogemm.softfp8_linear_expected(codes.numpy(), scale.numpy(), x), RTOL, ATOL, "soft-fp8 gemv %dx%d" % (n, k))


def _moe_shapes(seed, count):
    rng = np.random.RandomState(seed)
    out = []
    for _ in range(count):
        e = int(rng.choice([2, 4, 8, 16, 32, 64, 128]))
        k = int(rng.randint(1, min(e, 8) + 1))
        h = 128 * int(rng.randint(1, 5))
        i = 128 * int(rng.randint(1, 5))
        t = int(rng.choice([1, 2, 7, 16, 17, 33, 64, 100, 257, 300]))
        out.append((t, e, k, h, i, bool(rng.randint(0, 2)), bool(rng.randint(0, 2))))
    return out


@pytest.mark.parametrize("T,E,K,H,I,fp8,sigmoid", _moe_shapes(15, 14))
def test_fused_moe_random_shapes(mlk, T, E, K, H, I, fp8, sigmoid):
    from muxi_native_layout_kernels_amd.moe_planC import fused_moe
    dtype = torch.bfloat16
    x = randn((T, H), dtype, 1.0, T + E)
    logits = randn((T, E), dtype, 1.0, T + E + 1)
    std1, std2 = 1.0 / np.sqrt(H), 2.0 / np.sqrt(I)
    pack = lambda w: torch.stack([pack_a(w[e]) for e in range(w.shape[0])]).reshape(w.shape)     # noqa: E731
    kw = {}
    if fp8:
        c1, c2 = fp8_codes((E, 2 * I, H), E + 2, std=1.0), fp8_codes((E, H, I), E + 3, std=1.0)
        g = torch.Generator().manual_seed(E + 4)
        s1 = ((torch.rand((E, 2 * I // 128, H // 128), generator=g) + 0.5) * std1).float()
        s2 = ((torch.rand((E, H // 128, I // 128), generator=g) + 0.5) * std2).float()
        w1u, w2u = omoe.dequant_experts(c1.numpy(), s1.numpy()), omoe.dequant_experts(c2.numpy(), s2.numpy())
        w1p, w2p = pack(c1), pack(c2)
        kw = dict(w1_scale=s1.cuda(), w2_scale=s2.cuda(), block_shape=[128, 128], soft_fp8=True)
    else:
        w1u, w2u = randn((E, 2 * I, H), dtype, std1, E + 2), randn((E, H, I), dtype, std2, E + 3)
        w1p, w2p = pack(w1u), pack(w2u)
    score = "sigmoid" if sigmoid else "softmax"
    y = fused_moe(x.cuda(), w1p.cuda(), w2p.cuda(), logits.cuda(), K, True, score_func=score, **kw)
    y2 = fused_moe(x.cuda(), w1p.cuda(), w2p.cuda(), logits.cuda(), K, True, score_func=score, **kw)      # launch plan
    assert torch.equal(y, y2)
    ids, wts = orouter.route(logits, 1 if sigmoid else 0, 1, 1, K)
    want = omoe.moe_expected(x, w1u, w2u, ids, orouter.renormalize(wts), round_h_to=dtype)
    assert_close(y, want, RTOL, ATOL, "fused_moe T=%d E=%d K=%d H=%d I=%d fp8=%d" % (T, E, K, H, I, fp8))
