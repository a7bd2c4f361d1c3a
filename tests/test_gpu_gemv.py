"""GPU parity: GeMV over layout-A weights against the oracle (float64 product on the
un-packed weights), rtol = atol = 1e-2, through the C ABI."""
import numpy as np
import pytest
import torch

from oracle import gemm as ogemm, softfp8
from helpers import randn, pack_a, fp8_codes, assert_close

pytestmark = pytest.mark.gpu

RTOL = ATOL = 1e-2


@pytest.mark.parametrize("n,k", [(16, 32), (4096, 4096), (1024, 14336), (11008, 4096), (160, 28672)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_gemv_16bit(mlk, n, k, dtype):
    w = randn((n, k), dtype, 0.02, 2025)
    x = randn((1, k), dtype, 1.0, 2026)
    y = mlk.gemv_layoutA(pack_a(w).cuda(), x.cuda())
    assert y.shape == (1, n) and y.dtype == dtype
    assert_close(y, ogemm.linear_expected(w, x), RTOL, ATOL, "gemv")


@pytest.mark.parametrize("block,p1,p2", [(64, 1, 1), (256, 1, 4), (256, 2, 2), (256, 4, 8), (512, 2, 6),
                                         (1024, 1, 4), (1024, 16, 2)])
def test_gemv_launch_parameters(mlk, block, p1, p2):
    n, k = 2048, 4096
    w = randn((n, k), torch.bfloat16, 0.02, 1)
    x = randn((1, k), torch.bfloat16, 1.0, 2)
    y = mlk.gemv_layoutA_wapper(pack_a(w).cuda(), x.cuda(), n, k, blockDimX=block, kernelId=1, kernelParam1=p1,
                                kernelParam2=p2)
    assert_close(y, ogemm.linear_expected(w, x), RTOL, ATOL, "gemv params")


def test_gemv_alpha_bias_and_special_cases(mlk):
    n, k = 256, 512
    w = randn((n, k), torch.bfloat16, 0.05, 3)
    x = randn((1, k), torch.bfloat16, 1.0, 4)
    bias = randn((1, n), torch.bfloat16, 1.0, 5)
    a = pack_a(w).cuda()
    y = mlk.gemv_layoutA(a, x.cuda(), alpha=0.5, bias=bias.cuda())
    assert_close(y, ogemm.linear_expected(w, x, 0.5, bias), RTOL, ATOL, "alpha+bias")
    # alpha = 0 leaves the bias exactly
    y0 = mlk.gemv_layoutA(a, x.cuda(), alpha=0.0, bias=bias.cuda())
    assert torch.equal(y0.cpu(), bias)
    # identity weights copy x exactly
    eye = torch.eye(512, dtype=torch.bfloat16)
    yi = mlk.gemv_layoutA(pack_a(eye).cuda(), x.cuda())
    assert torch.equal(yi.cpu(), x)
    with pytest.raises(RuntimeError, match="beta"):
        mlk.gemv_layoutA(a, x.cuda(), beta=1.0)


def test_gemv_is_deterministic(mlk):
    n, k = 4096, 4096
    a = pack_a(randn((n, k), torch.bfloat16, 0.02, 7)).cuda()
    x = randn((1, k), torch.bfloat16, 1.0, 8).cuda()
    y1 = mlk.gemv_layoutA(a, x)
    y2 = mlk.gemv_layoutA(a, x)
    assert torch.equal(y1, y2)


@pytest.mark.parametrize("n,k", [(128, 128), (4096, 4096), (28672, 8192), (2112, 7168)])
@pytest.mark.parametrize("scaled", [False, True])
def test_gemv_soft_fp8(mlk, n, k, scaled):
    codes = fp8_codes((n, k), 2025)
    x = randn((1, k), torch.bfloat16, 1.0, 2026)
    scale = None
    if scaled:
        g = torch.Generator().manual_seed(9)
        scale = (torch.rand(((n + 127) // 128, (k + 127) // 128), generator=g) * 0.02 + 0.001).float()
    y = mlk.gemv_layoutA(pack_a(codes).cuda(), x.cuda(), scale_matrix=None if scale is None else scale.cuda())
    want = ogemm.softfp8_linear_expected(codes.numpy(), None if scale is None else scale.numpy(), x)
    assert_close(y, want, RTOL, ATOL, "soft-fp8 gemv")


def test_gemv_soft_fp8_all_codes_exact(mlk):
    """Every finite e4m3 code, one per weight row, against the oracle's widening: with a one-hot x
    the output is the dequantised weight itself, so the comparison is bit-exact."""
    k = 64
    codes = torch.tensor([c for c in range(256) if c not in (0x7F, 0xFF)] + [0, 0], dtype=torch.uint8)  # 256 rows
    w = torch.zeros((256, k), dtype=torch.uint8)
    w[:, 5] = codes
    x = torch.zeros((1, k), dtype=torch.bfloat16)
    x[0, 5] = 1.0
    for s in (1.0, 0.37, 1.0 / 448.0, 0.5, 2.0 ** -7, 4.0):
        scale = torch.full((2, 1), s, dtype=torch.float32)
        y = mlk.gemv_layoutA(pack_a(w).cuda(), x.cuda(), scale_matrix=scale.cuda())
        want = softfp8.bf16_bits_to_f32(softfp8.dequant_bf16_bits(codes.numpy(), np.float32(s)))
        got = y.cpu().float().numpy().reshape(-1)
        assert np.array_equal(got, want)  # values, so that -0 (code 0x80) compares equal to the +0 a sum yields


def test_gemv_rows_2_to_4(mlk):
    n, k = 512, 1024
    w = randn((n, k), torch.float16, 0.02, 1)
    for m in (2, 3, 4):
        x = randn((m, k), torch.float16, 1.0, 10 + m)
        y = mlk.gemv_layoutA_wapper(pack_a(w).cuda(), x.cuda(), n, k, blockDimX=256, kernelParam1=1, kernelParam2=4)
        assert_close(y, ogemm.linear_expected(w, x), RTOL, ATOL, "gemv M=%d" % m)


def test_gemv_errors(mlk):
    a = torch.zeros(2, 4, 16, 8, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(RuntimeError, match="vector"):
        mlk.gemv_layoutA(a, torch.zeros(2, 32, dtype=torch.bfloat16, device="cuda"))
    with pytest.raises(RuntimeError, match="same k"):
        mlk.gemv_layoutA(a, torch.zeros(1, 64, dtype=torch.bfloat16, device="cuda"))
    with pytest.raises(RuntimeError, match="4D"):
        mlk.gemv_layoutA(a.view(2, 4, 128), torch.zeros(1, 32, dtype=torch.bfloat16, device="cuda"))
    with pytest.raises(RuntimeError, match="data type"):
        mlk.gemv_layoutA(a, torch.zeros(1, 32, dtype=torch.float16, device="cuda"))


@pytest.mark.parametrize("kind", ["bf16", "fp16", "fp8", "fp8_matrix_cores"])
@pytest.mark.parametrize("n,k,block,per_cu,depth", [
    (4096, 4096, 1024, 1, 2),      # one row group per workgroup
    (11008, 4096, 512, 2, 4),      # uneven deal: two or three row groups per workgroup
    (28672, 2048, 256, 1, 8),      # seven row groups per workgroup, several 128-row scale blocks each
    (48, 192, 1024, 4, 2),         # fewer row groups than workgroups asked for, fewer tiles than waves
    (2112, 7168, 512, 4, 6),       # tiles not a multiple of the wave count
])
def test_gemv_persistent_kernels(mlk, kind, n, k, block, per_cu, depth):
    """Kernel id 2 (one uninterrupted stream per wave over a range of row groups) and, for soft-FP8 weights,
    kernel id 3 (the same with the products on the matrix cores) against the oracle, for 1 to 4 tokens."""
    fp8 = kind.startswith("fp8")
    if fp8 and k % 64:
        pytest.skip("soft-FP8 tiles cover 64 k")
    dtype = torch.float16 if kind == "fp16" else torch.bfloat16
    kid = 3 if kind == "fp8_matrix_cores" else 2
    scale = None
    if fp8:
        codes = fp8_codes((n, k), 77)
        g = torch.Generator().manual_seed(78)
        scale = (torch.rand(((n + 127) // 128, (k + 127) // 128), generator=g) * 0.02 + 0.001).float()
        a = pack_a(codes).cuda()
    else:
        w = randn((n, k), dtype, 0.02, 77)
        a = pack_a(w).cuda()
    for m in (1, 3, 4):
        x = randn((m, k), dtype, 1.0, 80 + m)
        bias = randn((1, n), dtype, 1.0, 90 + m)
        y = mlk.gemv_layoutA_wapper(a, x.cuda(), n, k, alpha=0.75, blockDimX=block, kernelId=kid, kernelParam1=per_cu,
                                    kernelParam2=depth, scale_matrix=None if scale is None else scale.cuda(),
                                    bias=bias.cuda())
        if fp8:
            want = ogemm.softfp8_linear_expected(codes.numpy(), scale.numpy(), x, 0.75, bias)
        else:
            want = ogemm.linear_expected(w, x, 0.75, bias)
        assert_close(y, want, RTOL, ATOL, "persistent gemv %s M=%d" % (kind, m))
        y2 = mlk.gemv_layoutA_wapper(a, x.cuda(), n, k, alpha=0.75, blockDimX=block, kernelId=kid, kernelParam1=per_cu,
                                     kernelParam2=depth, scale_matrix=None if scale is None else scale.cuda(),
                                     bias=bias.cuda())
        assert torch.equal(y, y2)


def test_gemv_matrix_core_variant_all_codes_exact(mlk):
    """Kernel id 3 widens with the same instructions as the other kernels: every finite e4m3 code comes back
    exactly through a one-hot activation vector (one code per weight row, in even and odd rows and octets)."""
    k = 128
    codes = torch.tensor([c for c in range(256) if c not in (0x7F, 0xFF)] + [0, 0], dtype=torch.uint8)
    for col in (5, 8, 77, 127):
        w = torch.zeros((256, k), dtype=torch.uint8)
        w[:, col] = codes
        x = torch.zeros((1, k), dtype=torch.bfloat16)
        x[0, col] = 1.0
        for s in (1.0, 0.37, 0.5):
            scale = torch.full((2, 1), s, dtype=torch.float32)
            y = mlk.gemv_layoutA_wapper(pack_a(w).cuda(), x.cuda(), 256, k, blockDimX=256, kernelId=3, kernelParam1=1,
                                        kernelParam2=2, scale_matrix=scale.cuda())
            want = softfp8.bf16_bits_to_f32(softfp8.dequant_bf16_bits(codes.numpy(), np.float32(s)))
            assert np.array_equal(y.cpu().float().numpy().reshape(-1), want)


def test_gemv_repeated_calls_take_the_launch_plan_and_keep_the_checks(mlk):
    """The second call with the same shapes and dtypes skips the shape checks and the table lookup (launch plan);
    what a shape does not tell is still checked on every call, and other values of alpha / bias go through."""
    n, k = 512, 1024
    w = randn((n, k), torch.bfloat16, 0.05, 41)
    a = pack_a(w).cuda()
    x1, x2 = randn((1, k), torch.bfloat16, 1.0, 42).cuda(), randn((1, k), torch.bfloat16, 1.0, 43).cuda()
    bias = randn((1, n), torch.bfloat16, 1.0, 44).cuda()
    y1 = mlk.gemv_layoutA(a, x1)
    y2 = mlk.gemv_layoutA(a, x2)                                  # planned
    assert_close(y1, ogemm.linear_expected(w, x1.cpu()), RTOL, ATOL, "first call")
    assert_close(y2, ogemm.linear_expected(w, x2.cpu()), RTOL, ATOL, "planned call")
    y3 = mlk.gemv_layoutA(a, x2, alpha=0.5, bias=bias)
    y4 = mlk.gemv_layoutA(a, x1, alpha=0.25, bias=bias)           # planned, other alpha
    assert_close(y3, ogemm.linear_expected(w, x2.cpu(), 0.5, bias.cpu()), RTOL, ATOL, "bias, first call")
    assert_close(y4, ogemm.linear_expected(w, x1.cpu(), 0.25, bias.cpu()), RTOL, ATOL, "bias, planned call")
    with pytest.raises(RuntimeError, match="beta"):
        mlk.gemv_layoutA(a, x1, beta=1)
    wide = torch.zeros((1, 2 * k), dtype=torch.bfloat16, device="cuda")
    with pytest.raises(RuntimeError, match="contiguous"):
        mlk.gemv_layoutA(a, wide[:, ::2])                         # same shape and dtype, not contiguous
