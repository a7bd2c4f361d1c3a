"""GPU parity: narrow GeMM (layoutA / layoutAB_ContinuousC / layoutABC, soft-FP8) against the
oracle's float64 product on the un-packed weights, rtol = atol = 1e-2, through the C ABI."""
import numpy as np
import pytest
import torch

from oracle import gemm as ogemm, layouts
from helpers import randn, pack_a, pack_b, fp8_codes, assert_close, bits

pytestmark = pytest.mark.gpu

RTOL = ATOL = 1e-2


@pytest.mark.parametrize("m", [1, 8, 16, 32, 64])
def test_gemm_layout_a_fp16_config(mlk, m):
    n, k = 11008, 4096
    w = randn((n, k), torch.float16, 0.02, 2025)
    b = randn((m, k), torch.float16, 1.0, 2026 + m)
    c = mlk.gemm_layoutA(pack_a(w).cuda(), b.cuda())
    assert c.shape == (m, n) and c.dtype == torch.float16
    assert_close(c, ogemm.linear_expected(w, b), RTOL, ATOL, "gemm_layoutA M=%d" % m)


@pytest.mark.parametrize("m", [1, 3, 15, 17, 33, 48, 63, 65, 100, 130])
def test_gemm_layout_a_ragged_tokens(mlk, m):
    n, k = 256, 512
    w = randn((n, k), torch.bfloat16, 0.05, 1)
    b = randn((m, k), torch.bfloat16, 1.0, 2)
    c = mlk.gemm_layoutA(pack_a(w).cuda(), b.cuda())
    assert_close(c, ogemm.linear_expected(w, b), RTOL, ATOL, "ragged M=%d" % m)


@pytest.mark.parametrize("p1,p2,p3", [(1, 1, 1), (1, 4, 1), (2, 2, 1), (4, 4, 1), (1, 16, 1), (2, 8, 1), (1, 1, 4),
                                      (2, 4, 3), (4, 2, 8), (1, 2, 64)])
@pytest.mark.parametrize("m", [16, 40, 64])
def test_gemm_launch_parameters(mlk, p1, p2, p3, m):
    n, k = 512, 2048
    w = randn((n, k), torch.bfloat16, 0.02, 3)
    b = randn((m, k), torch.bfloat16, 1.0, 4)
    bias = randn((1, n), torch.bfloat16, 1.0, 5)
    a = pack_a(w).cuda()
    want = ogemm.linear_expected(w, b, 0.75, bias)
    c = mlk.gemm_layoutA_wapper(a, b.cuda(), n, m, k, alpha=0.75, kernelParam1=p1, kernelParam2=p2, kernelParam3=p3,
                                kernelId=1, bias=bias.cuda())
    assert_close(c, want, RTOL, ATOL, "params")
    c2 = mlk.gemm_layoutA_wapper(a, b.cuda(), n, m, k, alpha=0.75, kernelParam1=p1, kernelParam2=p2,
                                 kernelParam3=p3, kernelId=1, bias=bias.cuda())
    assert torch.equal(c, c2), "K split across workgroups must be deterministic and leave its counters clean"


@pytest.mark.parametrize("p1,p3", [(1, 1), (2, 1), (4, 1), (1, 2), (2, 4), (4, 8)])
@pytest.mark.parametrize("m", [16, 33, 48, 64, 100])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_gemm_tile_kernel(mlk, p1, p3, m, dtype):
    """kernelId 2: row-shared tile kernel, row-major and native operands, K split across workgroups."""
    n, k = 1024, 2048
    w = randn((n, k), dtype, 0.02, 13)
    b = randn((m, k), dtype, 1.0, 14)
    bias = randn((1, n), dtype, 1.0, 15)
    a = pack_a(w).cuda()
    want = ogemm.linear_expected(w, b, 1.25, bias)
    c = mlk.gemm_layoutA_wapper(a, b.cuda(), n, m, k, alpha=1.25, kernelParam1=p1, kernelParam2=1, kernelParam3=p3,
                                kernelId=2, bias=bias.cuda())
    assert_close(c, want, RTOL, ATOL, "tile kernel")
    assert torch.equal(c, mlk.gemm_layoutA_wapper(a, b.cuda(), n, m, k, alpha=1.25, kernelParam1=p1, kernelParam2=1,
                                                  kernelParam3=p3, kernelId=2, bias=bias.cuda()))
    if m % 16 == 0:
        b_nat = mlk.layoutB(b.cuda())
        c_rm = mlk.gemm_layoutAB_ContinuousC_wapper(a, b_nat, n, m, k, alpha=1.25, kernelParam1=p1, kernelParam3=p3,
                                                    kernelId=2, bias=bias.cuda())
        c_nat = mlk.gemm_layoutABC_wapper(a, b_nat, n, m, k, alpha=1.25, kernelParam1=p1, kernelParam3=p3, kernelId=2,
                                          bias=bias.cuda())
        assert torch.equal(c_rm, c) and torch.equal(mlk.reLayoutC(c_nat), c)


def test_gemm_tile_kernel_soft_fp8(mlk):
    n, k, m = 1024, 2048, 40
    codes = fp8_codes((n, k), 21)
    b = randn((m, k), torch.bfloat16, 1.0, 22)
    g = torch.Generator().manual_seed(23)
    scale = (torch.rand((n // 128, k // 128), generator=g) * 0.02 + 0.001).float()
    c = mlk.gemm_layoutA_soft_fp8_wapper(pack_a(codes).cuda(), scale.cuda(), b.cuda(), n, m, k, kernelParam1=2,
                                         kernelParam3=2, kernelId=2)
    assert_close(c, ogemm.softfp8_linear_expected(codes.numpy(), scale.numpy(), b), RTOL, ATOL, "tile fp8")


@pytest.mark.parametrize("kid", [12, 14, 16, 18])
@pytest.mark.parametrize("p1,p2,p3", [(1, 1, 1), (4, 2, 1), (2, 8, 2), (1, 16, 1), (8, 4, 1), (8, 2, 2)])
@pytest.mark.parametrize("m", [1, 7, 16, 40])
def test_gemm_ring_depth_kernel_ids(mlk, kid, p1, p2, p3, m):
    """kernelId 12..18: kernel 1 with 2..8 k tiles in flight per wave.  The summation order does not depend
    on the depth, so the result is bit-equal to kernel 1's; above 16 tokens the ids mean kernel 1."""
    n, k = 512, 1024 + 32 * 5                    # 37 k tiles: fewer than, equal to and more than the ring at some split
    w = randn((n, k), torch.float16, 0.02, 31)
    b = randn((m, k), torch.float16, 1.0, 32)
    a = pack_a(w).cuda()
    c = mlk.gemm_layoutA_wapper(a, b.cuda(), n, m, k, kernelParam1=p1, kernelParam2=p2, kernelParam3=p3, kernelId=kid)
    assert_close(c, ogemm.linear_expected(w, b), RTOL, ATOL, "ring depth id %d" % kid)
    c1 = mlk.gemm_layoutA_wapper(a, b.cuda(), n, m, k, kernelParam1=p1, kernelParam2=p2, kernelParam3=p3, kernelId=1)
    assert torch.equal(c, c1)


def test_gemm_ring_depth_soft_fp8(mlk):
    n, k, m = 512, 1024, 9
    codes = fp8_codes((n, k), 41)
    b = randn((m, k), torch.bfloat16, 1.0, 42)
    g = torch.Generator().manual_seed(43)
    scale = (torch.rand((n // 128, k // 128), generator=g) * 0.02 + 0.001).float()
    for kid in (12, 14, 16, 18):
        for p1 in (2, 8):         # eight row groups per wave = one 128-row scale block
            c = mlk.gemm_layoutA_soft_fp8_wapper(pack_a(codes).cuda(), scale.cuda(), b.cuda(), n, m, k, kernelParam1=p1,
                                                 kernelParam2=4, kernelParam3=1, kernelId=kid)
            assert_close(c, ogemm.softfp8_linear_expected(codes.numpy(), scale.numpy(), b), RTOL, ATOL, "fp8 depth")


@pytest.mark.parametrize("m", [65, 100, 128, 130, 200, 256, 300])
@pytest.mark.parametrize("p1,p3", [(1, 1), (2, 1), (2, 2), (4, 4)])
def test_gemm_tile_kernel_wide_passes(mlk, m, p1, p3):
    """More than 64 tokens with kernelId 2 on row-major operands: passes of up to 128 tokens over the weights."""
    n, k = 512, 1024
    w = randn((n, k), torch.bfloat16, 0.02, 51)
    b = randn((m, k), torch.bfloat16, 1.0, 52)
    bias = randn((1, n), torch.bfloat16, 1.0, 53)
    a = pack_a(w).cuda()
    c = mlk.gemm_layoutA_wapper(a, b.cuda(), n, m, k, alpha=0.5, kernelParam1=p1, kernelParam2=1, kernelParam3=p3,
                                kernelId=2, bias=bias.cuda())
    assert_close(c, ogemm.linear_expected(w, b, 0.5, bias), RTOL, ATOL, "wide passes M=%d" % m)
    c2 = mlk.gemm_layoutA_wapper(a, b.cuda(), n, m, k, alpha=0.5, kernelParam1=p1, kernelParam2=1, kernelParam3=p3,
                                 kernelId=2, bias=bias.cuda())
    assert torch.equal(c, c2)


def test_gemm_wide_default_parameters(mlk):
    """A shape that is in no table, above 64 tokens: the heuristic picks the panel kernel (K % 128 == 0)."""
    n, k, m = 768, 512, 150
    w = randn((n, k), torch.float16, 0.02, 61)
    b = randn((m, k), torch.float16, 1.0, 62)
    c = mlk.gemm_layoutA(pack_a(w).cuda(), b.cuda())
    assert_close(c, ogemm.linear_expected(w, b), RTOL, ATOL, "wide default")
    codes = fp8_codes((n, k), 63)
    g = torch.Generator().manual_seed(64)
    scale = (torch.rand((n // 128, k // 128), generator=g) * 0.02 + 0.001).float()
    bb = randn((m, k), torch.bfloat16, 1.0, 65)
    c8 = mlk.gemm_layoutA_linear(pack_a(codes).cuda(), bb.cuda(), scale_matrix=scale.cuda())
    assert_close(c8, ogemm.softfp8_linear_expected(codes.numpy(), scale.numpy(), bb), RTOL, ATOL, "wide default fp8")


@pytest.mark.parametrize("m", [1, 65, 128, 129, 200, 256, 300, 640])
@pytest.mark.parametrize("n,k,p3", [(512, 256, 1), (272, 384, 1), (272, 384, 3), (1040, 1024, 2), (256, 128, 4)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_gemm_panel_kernel(mlk, m, n, k, p3, dtype):
    """kernelId 3: 256-row x 128-token panels with MFMA 32x32x16; ragged token counts, row counts that are not
    a multiple of 256 (or of 32: 272 = 17 row groups), K slices that do not divide the windows evenly, one
    window per slice, more slices than windows."""
    w = randn((n, k), dtype, 0.05, 91)
    b = randn((m, k), dtype, 1.0, 92)
    bias = randn((1, n), dtype, 1.0, 93)
    a = pack_a(w).cuda()
    # (rows, tokens) of a panel: 128 x 128, 256 x 128, 256 x 256, both chosen by the library
    for rg, width in ((2, 1), (4, 1), (4, 2), (1, 4)):
        c = mlk.gemm_layoutA_wapper(a, b.cuda(), n, m, k, alpha=0.5, kernelParam1=rg, kernelParam2=width, kernelParam3=p3,
                                    kernelId=3, bias=bias.cuda())
        assert c.shape == (m, n) and c.dtype == dtype
        assert_close(c, ogemm.linear_expected(w, b, 0.5, bias), RTOL, ATOL, "panel n=%d k=%d M=%d" % (n, k, m))
        c2 = mlk.gemm_layoutA_wapper(a, b.cuda(), n, m, k, alpha=0.5, kernelParam1=rg, kernelParam2=width,
                                     kernelParam3=p3, kernelId=3, bias=bias.cuda())
        assert torch.equal(c, c2)


@pytest.mark.parametrize("m", [100, 256, 385])
@pytest.mark.parametrize("scaled", [False, True])
def test_gemm_panel_kernel_soft_fp8(mlk, m, scaled):
    n, k = 640, 512
    codes = fp8_codes((n, k), 95)
    g = torch.Generator().manual_seed(96)
    scale = (torch.rand((n // 128, k // 128), generator=g) * 0.02 + 0.001).float() if scaled else None
    b = randn((m, k), torch.bfloat16, 1.0, 97)
    for p3, rg, width in ((1, 2, 1), (2, 2, 1), (2, 4, 1), (1, 4, 2), (2, 4, 2)):
        c = mlk.gemm_layoutA_soft_fp8_wapper(pack_a(codes).cuda(), None if scale is None else scale.cuda(), b.cuda(),
                                             n, m, k, kernelParam1=rg, kernelParam2=width, kernelParam3=p3, kernelId=3)
        want = ogemm.softfp8_linear_expected(codes.numpy(), None if scale is None else scale.numpy(), b)
        assert_close(c, want, RTOL, ATOL, "panel fp8 M=%d slices=%d width=%d" % (m, p3, width))


@pytest.mark.parametrize("n,m,k,p1,p2,p3", [
    (5504, 1024, 256, 2, 1, 2),      # 43 row tiles x 8 token tiles of 128 x 128: one whole round of 256 panels + 88 sliced
    (5520, 1000, 512, 2, 1, 3),      # ragged rows and tokens, three uneven slices of four windows
    (16640, 1024, 256, 4, 2, 2),     # 65 row tiles x 4 token tiles of 256 x 256: 256 whole + 4 sliced
    (11008, 1024, 128, 4, 1, 2),     # one window: a single slice does all the work
    (5504, 384, 256, 2, 1, 2),       # three token tiles do not divide an XCD's CUs: every panel whole
    (2048, 1024, 256, 2, 1, 2),      # exactly one round: nothing left over, no slices
    (1024, 200, 512, 4, 1, 4),       # less than a round: every panel sliced, as with kernelId 3
])
def test_gemm_panel_kernel_last_round_slices(mlk, n, m, k, p1, p2, p3):
    """kernelId 5: the panel kernel with K slices only on the panels left over after whole rounds of one panel per
    CU; bit-equal on a second run, and equal to the oracle like kernelId 3."""
    dtype = torch.bfloat16
    w = randn((n, k), dtype, 0.05, 191)
    b = randn((m, k), dtype, 1.0, 192)
    bias = randn((1, n), dtype, 1.0, 193)
    a = pack_a(w).cuda()
    c = mlk.gemm_layoutA_wapper(a, b.cuda(), n, m, k, alpha=0.5, kernelParam1=p1, kernelParam2=p2, kernelParam3=p3,
                                kernelId=5, bias=bias.cuda())
    assert c.shape == (m, n) and c.dtype == dtype
    assert_close(c, ogemm.linear_expected(w, b, 0.5, bias), RTOL, ATOL, "panel, last round sliced n=%d M=%d" % (n, m))
    c2 = mlk.gemm_layoutA_wapper(a, b.cuda(), n, m, k, alpha=0.5, kernelParam1=p1, kernelParam2=p2, kernelParam3=p3,
                                 kernelId=5, bias=bias.cuda())
    assert torch.equal(c, c2)


def test_gemm_panel_kernel_last_round_slices_soft_fp8(mlk):
    n, k, m = 5504, 512, 1024
    codes = fp8_codes((n, k), 195)
    g = torch.Generator().manual_seed(196)
    scale = (torch.rand((n // 128, k // 128), generator=g) * 0.02 + 0.001).float()
    b = randn((m, k), torch.bfloat16, 1.0, 197)
    c = mlk.gemm_layoutA_soft_fp8_wapper(pack_a(codes).cuda(), scale.cuda(), b.cuda(), n, m, k, kernelParam1=2,
                                         kernelParam2=1, kernelParam3=2, kernelId=5)
    assert_close(c, ogemm.softfp8_linear_expected(codes.numpy(), scale.numpy(), b), RTOL, ATOL, "panel fp8, last round sliced")


@pytest.mark.parametrize("fp8", [False, True])
def test_gemm_panel_kernel_band_and_chunk_mapping(mlk, fp8):
    """256 x 256 panels computed whole: the workgroup ids walk bands of eight groups of row tiles in chunks of four token
    tiles.  73 row tiles = ten groups (a band of eight and one of two, the last group with one row tile) and six token
    tiles (a chunk of four and one of two, the last tile ragged): every output element is checked."""
    n, k, m = 18560, 256, 1300
    b = randn((m, k), torch.bfloat16, 1.0, 292)
    if fp8:
        codes = fp8_codes((n, k), 293)
        g = torch.Generator().manual_seed(294)
        scale = (torch.rand((n // 128, k // 128), generator=g) * 0.02 + 0.001).float()
        c = mlk.gemm_layoutA_soft_fp8_wapper(pack_a(codes).cuda(), scale.cuda(), b.cuda(), n, m, k, kernelParam1=4,
                                             kernelParam2=2, kernelParam3=1, kernelId=3)
        want = ogemm.softfp8_linear_expected(codes.numpy(), scale.numpy(), b)
    else:
        w = randn((n, k), torch.bfloat16, 0.05, 291)
        bias = randn((1, n), torch.bfloat16, 1.0, 295)
        c = mlk.gemm_layoutA_wapper(pack_a(w).cuda(), b.cuda(), n, m, k, alpha=0.5, kernelParam1=4, kernelParam2=2,
                                    kernelParam3=1, kernelId=3, bias=bias.cuda())
        want = ogemm.linear_expected(w, b, 0.5, bias)
    assert c.shape == (m, n)
    assert_close(c, want, RTOL, ATOL, "band / chunk mapping fp8=%s" % fp8)


def test_gemm_panel_kernel_is_the_wide_default(mlk):
    """Above 64 tokens the heuristic for unscanned shapes picks the panel kernel; a K that is no
    multiple of 128 keeps the row-shared kernel, and the panel kernel refuses it when asked for by id."""
    from muxi_native_layout_kernels_amd import arg_selector
    # 4224 rows: a weight shape that no packaged table holds
    assert arg_selector.selector("layoutA_gemm").get_args((4224, 300, 1024))[0] == 3
    assert arg_selector.selector("layoutA_soft_fp8_gemm").get_args((4224, 300, 1024))[0] == 3
    assert arg_selector.selector("layoutA_gemm").get_args((4224, 300, 1088))[0] == 2
    assert arg_selector.selector("layout_gemm").get_args((4224, 304, 1024))[0] == 2       # native operands
    n, k, m = 4224, 1024, 300
    w = randn((n, k), torch.bfloat16, 0.02, 98)
    b = randn((m, k), torch.bfloat16, 1.0, 99)
    c = mlk.gemm_layoutA_linear(pack_a(w).cuda(), b.cuda())
    assert_close(c, ogemm.linear_expected(w, b), RTOL, ATOL, "panel default")
    with pytest.raises(RuntimeError, match="K % 128"):
        mlk.gemm_layoutA_wapper(pack_a(w[:, :960].contiguous()).cuda(), b[:, :960].contiguous().cuda(), n, m, 960,
                                kernelParam1=1, kernelParam2=1, kernelParam3=1, kernelId=3)
    with pytest.raises(RuntimeError, match="row-major"):
        mlk.gemm_layoutABC_wapper(pack_a(w).cuda(), mlk.layoutB(b[:288].contiguous().cuda()), n, 288, k, kernelParam1=1,
                                  kernelParam2=1, kernelParam3=1, kernelId=3)


@pytest.mark.parametrize("n", [16 * 300, 16 * 384, 16 * 688, 16 * 768, 16 * 1000])
@pytest.mark.parametrize("m", [1, 7, 16, 32, 40, 48, 57, 64])
def test_gemm_balanced_rows_kernel(mlk, n, m):
    """kernelId 4: one workgroup per CU, the row groups dealt out evenly (one to four per workgroup, uneven
    deals included).  From three token blocks on the activations of a k window are shared through LDS; shapes
    it does not take run as kernel 1."""
    k = 256
    w = randn((n, k), torch.bfloat16, 0.05, 71)
    b = randn((m, k), torch.bfloat16, 1.0, 72)
    bias = randn((1, n), torch.bfloat16, 1.0, 73)
    a = pack_a(w).cuda()
    for p2 in (1, 2, 8):
        c = mlk.gemm_layoutA_wapper(a, b.cuda(), n, m, k, alpha=2.0, kernelParam1=1, kernelParam2=p2, kernelParam3=1,
                                    kernelId=4, bias=bias.cuda())
        assert_close(c, ogemm.linear_expected(w, b, 2.0, bias), RTOL, ATOL, "balanced rows n=%d m=%d" % (n, m))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("k", [192, 1024, 1152, 4096])
@pytest.mark.parametrize("m", [20, 32, 33, 48, 50, 64])
def test_gemm_balanced_rows_kernel_shared_windows(mlk, dtype, k, m):
    """kernelId 4 at two (eight waves), three and four token blocks over short and long K: K = 192 (six k tiles, no whole
    windows: the plain wave kernel takes it), 1024 and 4096 (the unrolled loop with its lead-in), 1152 (36 k
    tiles: nine windows, an odd tail), on 688 row groups (three and two per workgroup on 256 CUs); twice, and the
    two runs must agree bit for bit."""
    n = 16 * 688
    w = randn((n, k), dtype, 0.02, 74)
    b = randn((m, k), dtype, 1.0, 75)
    bias = randn((1, n), dtype, 1.0, 76)
    a = pack_a(w).cuda()
    for p2 in (8, 4, 2):
        c = mlk.gemm_layoutA_wapper(a, b.cuda(), n, m, k, alpha=0.5, kernelParam1=1, kernelParam2=p2, kernelParam3=1,
                                    kernelId=4, bias=bias.cuda())
        assert_close(c, ogemm.linear_expected(w, b, 0.5, bias), RTOL, ATOL, "balanced shared k=%d m=%d p2=%d" % (k, m, p2))
        c2 = mlk.gemm_layoutA_wapper(a, b.cuda(), n, m, k, alpha=0.5, kernelParam1=1, kernelParam2=p2, kernelParam3=1,
                                     kernelId=4, bias=bias.cuda())
        assert torch.equal(c, c2)


@pytest.mark.parametrize("n", [11008, 12288, 4736, 18432, 22016, 28672, 32768])
@pytest.mark.parametrize("m", [20, 32, 40, 64])
def test_gemm_balanced_rows_kernel_soft_fp8(mlk, n, m):
    """kernelId 4 with soft-FP8 weights from two token blocks on (eight waves share staged windows): two to eight
    row groups per workgroup (on 256 CUs: three or two for 11008 rows, five or four for 18432, six or five for 22016,
    seven for 28672, eight for 32768) that start anywhere, so they straddle two 128-row blocks of scales; every block
    has its own random scale.  With two waves at two token blocks the id means kernel 1."""
    k = 1024
    codes = fp8_codes((n, k), 91)
    g = torch.Generator().manual_seed(92)
    scale = (torch.rand((n // 128, k // 128), generator=g) * 0.02 + 0.001).float()
    b = randn((m, k), torch.bfloat16, 1.0, 93)
    a = pack_a(codes).cuda()
    want = ogemm.softfp8_linear_expected(codes.numpy(), scale.numpy(), b)
    for p2 in (8, 4, 2):
        c = mlk.gemm_layoutA_soft_fp8_wapper(a, scale.cuda(), b.cuda(), n, m, k, kernelParam1=1, kernelParam2=p2,
                                             kernelParam3=1, kernelId=4)
        assert_close(c, want, RTOL, ATOL, "balanced fp8 n=%d m=%d p2=%d" % (n, m, p2))


def test_gemm_balanced_rows_fallbacks(mlk):
    """Soft-FP8 weights at one token block and native operands are outside kernel 4: the id then means kernel 1."""
    n, k, m = 16 * 300, 512, 16
    codes = fp8_codes((n - n % 128, k), 81)
    n8 = codes.shape[0]
    g = torch.Generator().manual_seed(82)
    scale = (torch.rand((n8 // 128, k // 128), generator=g) * 0.02 + 0.001).float()
    b = randn((m, k), torch.bfloat16, 1.0, 83)
    c = mlk.gemm_layoutA_soft_fp8_wapper(pack_a(codes).cuda(), scale.cuda(), b.cuda(), n8, m, k, kernelParam1=1,
                                         kernelParam2=4, kernelParam3=1, kernelId=4)
    assert_close(c, ogemm.softfp8_linear_expected(codes.numpy(), scale.numpy(), b), RTOL, ATOL, "kernel 4 on fp8")
    w = randn((n, k), torch.float16, 0.05, 84)
    bh = randn((m, k), torch.float16, 1.0, 85)
    a = pack_a(w).cuda()
    c_rm = mlk.gemm_layoutAB_ContinuousC_wapper(a, mlk.layoutB(bh.cuda()), n, m, k, kernelParam1=1, kernelParam2=4,
                                                kernelParam3=1, kernelId=4)
    assert_close(c_rm, ogemm.linear_expected(w, bh), RTOL, ATOL, "kernel 4 on native B")


def test_gemm_special_cases(mlk):
    n = k = 256
    eye = torch.eye(n, dtype=torch.float16)
    b = randn((32, k), torch.float16, 1.0, 6)
    assert torch.equal(mlk.gemm_layoutA(pack_a(eye).cuda(), b.cuda()).cpu(), b)
    bias = randn((1, n), torch.float16, 1.0, 7)
    c0 = mlk.gemm_layoutA(pack_a(eye).cuda(), b.cuda(), alpha=0.0, bias=bias.cuda())
    assert torch.equal(c0.cpu(), bias.expand(32, n))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("m", [32, 48, 64])
def test_native_chain_balanced_rows_kernel(mlk, dtype, m):
    """kernelId 4 on layout-B activations from two token blocks on (eight and four waves share staged windows):
    layout-C output + reLayoutC equals the row-major output bit for bit, the layout-C tensor equals the oracle's
    relayout of it, and both match the oracle; 688 and 512 row groups (three / two and two per workgroup)."""
    for n, k in ((16 * 688, 1024), (8192, 512)):
        w = randn((n, k), dtype, 0.02, 18)
        b = randn((m, k), dtype, 1.0, 19)
        a, b_nat = pack_a(w).cuda(), mlk.layoutB(b.cuda())
        for p2 in (8, 4):
            c_rm = mlk.gemm_layoutAB_ContinuousC_wapper(a, b_nat, n, m, k, kernelParam1=1, kernelParam2=p2, kernelParam3=1,
                                                        kernelId=4)
            c_nat = mlk.gemm_layoutABC_wapper(a, b_nat, n, m, k, kernelParam1=1, kernelParam2=p2, kernelParam3=1,
                                              kernelId=4)
            assert torch.equal(mlk.reLayoutC(c_nat), c_rm)
            assert torch.equal(c_nat.cpu().view(torch.int16), ogemm.layout_c_of(c_rm.cpu()).view(torch.int16))
            assert_close(c_rm, ogemm.linear_expected(w, b), RTOL, ATOL, "native balanced n=%d m=%d p2=%d" % (n, m, p2))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_native_chain_bit_exact(mlk, dtype):
    """layoutB -> gemm_layoutABC -> reLayoutC equals gemm_layoutAB_ContinuousC bit for bit (same launch
    parameters, hence same accumulation order), and both match the oracle."""
    n, k, m = 1024, 2048, 32
    w = randn((n, k), dtype, 0.02, 8)
    b = randn((m, k), dtype, 1.0, 9)
    a = pack_a(w).cuda()
    b_nat = mlk.layoutB(b.cuda())
    assert np.array_equal(bits(b_nat.cpu()), layouts.pack_layout_b(bits(b)))
    for (p1, p2, p3) in [(1, 4, 1), (2, 2, 2)]:
        c_nat = mlk.gemm_layoutABC_wapper(a, b_nat, n, m, k, kernelParam1=p1, kernelParam2=p2, kernelParam3=p3)
        assert c_nat.shape == (n // 32, m // 16, 4, 16, 8)
        c_rm = mlk.gemm_layoutAB_ContinuousC_wapper(a, b_nat, n, m, k, kernelParam1=p1, kernelParam2=p2,
                                                    kernelParam3=p3)
        assert torch.equal(mlk.reLayoutC(c_nat), c_rm)
        # layout-C of the result is layout-B of the row-major result
        assert np.array_equal(bits(c_nat.cpu()), layouts.pack_layout_c(bits(c_rm.cpu())))
        c_a = mlk.gemm_layoutA_wapper(a, b.cuda(), n, m, k, kernelParam1=p1, kernelParam2=p2, kernelParam3=p3)
        assert torch.equal(c_a, c_rm)
        assert_close(c_rm, ogemm.linear_expected(w, b), RTOL, ATOL, "native chain")


def test_native_chain_config(mlk):
    n = k = 8192
    m = 32
    w = randn((n, k), torch.bfloat16, 0.02, 2025)
    b = randn((m, k), torch.bfloat16, 1.0, 2026)
    a = pack_a(w).cuda()
    b_nat = mlk.layoutB(b.cuda())
    c_nat = mlk.gemm_layoutABC(a, b_nat)
    c = mlk.reLayoutC(c_nat)
    assert_close(c, ogemm.linear_expected(w, b), RTOL, ATOL, "ABC 8192")
    # the native output is layout-C of the row-major one (oracle permutation, bit for bit)
    assert torch.equal(c_nat.cpu(), ogemm.layout_c_of(c.cpu()))
    # chain a second product on the native output: C1 is the layout-B operand of the next layer
    w2 = randn((256, n), torch.bfloat16, 0.02, 2027)
    c2 = mlk.reLayoutC(mlk.gemm_layoutABC(pack_a(w2).cuda(), c_nat))
    assert_close(c2, ogemm.linear_expected(w2, c.cpu()), RTOL, ATOL, "chained")


@pytest.mark.parametrize("m", [1, 4, 16, 33])
@pytest.mark.parametrize("scaled", [False, True])
def test_gemm_soft_fp8(mlk, m, scaled):
    n, k = 1024, 2048
    codes = fp8_codes((n, k), 2025)
    b = randn((m, k), torch.bfloat16, 1.0, 2026)
    g = torch.Generator().manual_seed(3)
    scale = (torch.rand((n // 128, k // 128), generator=g) * 0.02 + 0.001).float() if scaled else \
        torch.ones((n // 128, k // 128))
    c = mlk.gemm_layoutA_soft_fp8(pack_a(codes).cuda(), scale.cuda(), b.cuda())
    assert_close(c, ogemm.softfp8_linear_expected(codes.numpy(), scale.numpy(), b), RTOL, ATOL, "soft-fp8 gemm")
    c2 = mlk.gemm_layoutA_linear(pack_a(codes).cuda(), b.cuda(), scale_matrix=scale.cuda())
    assert torch.equal(c, c2)


@pytest.mark.parametrize("m", [4, 16])
@pytest.mark.parametrize("scaled", [False, True])
def test_gemm_soft_fp8_config(mlk, m, scaled):
    """The third benchmark configuration at its full shape through the shipped table rows, with unit scales and
    with an arbitrary fp32 scale per 128 x 128 block (the general widening path, which is what the bench times)."""
    n, k = 28672, 8192
    codes = fp8_codes((n, k), 2025)
    b = randn((m, k), torch.bfloat16, 1.0, 2026)
    if scaled:
        g = torch.Generator().manual_seed(2027)
        scale = (torch.rand((n // 128, k // 128), generator=g) * 0.02 + 0.001).float()
    else:
        scale = torch.ones((n // 128, k // 128))
    c = mlk.gemm_layoutA_soft_fp8(pack_a(codes).cuda(), scale.cuda(), b.cuda())
    # float64 product in row chunks to bound host memory
    from oracle import softfp8
    got = c.cpu()
    for r0 in range(0, n, 4096):
        wchunk = softfp8.dequant_weight_f32(codes[r0:r0 + 4096].numpy(), scale[r0 // 128:(r0 + 4096) // 128].numpy() if scaled else None)
        assert_close(got[:, r0:r0 + 4096], ogemm.linear_expected(wchunk, b), RTOL, ATOL, "soft-fp8 config")


def test_gemm_errors(mlk):
    a = torch.zeros(8, 16, 16, 8, dtype=torch.bfloat16, device="cuda")   # 128 x 128
    b = torch.zeros(16, 128, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(RuntimeError, match="same k"):
        mlk.gemm_layoutA(a, torch.zeros(16, 256, dtype=torch.bfloat16, device="cuda"))
    with pytest.raises(RuntimeError, match="2D"):
        mlk.gemm_layoutA(a, b.view(1, 16, 128))
    with pytest.raises(RuntimeError, match="m % 128"):
        mlk.gemm_layoutA(torch.zeros(4, 16, 16, 8, dtype=torch.bfloat16, device="cuda"), b)
    with pytest.raises(RuntimeError, match="5D"):
        mlk.gemm_layoutABC(a, b)
    with pytest.raises(RuntimeError, match="data type"):
        mlk.gemm_layoutA(a, b.half())
    assert mlk.gemm_layoutA(a, b).shape == (16, 128)


def test_gemm_repeated_calls_take_the_launch_plan_and_keep_the_checks(mlk):
    """Second calls with the same shapes run from the launch plan: same results as the first, K-split workspace
    included, and the per-call checks (contiguity, beta) still raise."""
    n, k, m = 1024, 2048, 24
    w = randn((n, k), torch.float16, 0.02, 51)
    a = pack_a(w).cuda()
    b1, b2 = randn((m, k), torch.float16, 1.0, 52).cuda(), randn((m, k), torch.float16, 1.0, 53).cuda()
    c1 = mlk.gemm_layoutA(a, b1)
    c2 = mlk.gemm_layoutA(a, b2)                                  # planned
    c1b = mlk.gemm_layoutA(a, b1)                                 # planned
    assert torch.equal(c1, c1b)
    assert_close(c2, ogemm.linear_expected(w, b2.cpu()), RTOL, ATOL, "planned call")
    bn = mlk.layoutB(randn((32, k), torch.float16, 1.0, 54).cuda())
    for fn in (mlk.gemm_layoutABC, mlk.gemm_layoutAB_ContinuousC):
        assert torch.equal(fn(a, bn), fn(a, bn))
    assert torch.equal(mlk.reLayoutC(mlk.gemm_layoutABC(a, bn)), mlk.gemm_layoutAB_ContinuousC(a, bn))
    with pytest.raises(RuntimeError, match="beta"):
        mlk.gemm_layoutA(a, b1, beta=2)
    wide = torch.zeros((m, 2 * k), dtype=torch.float16, device="cuda")
    with pytest.raises(RuntimeError, match="contiguous"):
        mlk.gemm_layoutA(a, wide[:, ::2])
