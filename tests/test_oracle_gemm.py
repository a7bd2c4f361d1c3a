"""CPU: pins the oracle's GeMV / GeMM statements against closed forms and library routines."""
import numpy as np
import pytest
import torch

from oracle import gemm as ogemm, layouts, softfp8
from helpers import randn, fp8_codes


def test_linear_expected_closed_forms():
    n, k, m = 48, 64, 5
    w = randn((n, k), torch.bfloat16, 0.5, 1)
    x = randn((m, k), torch.bfloat16, 1.0, 2)
    bias = randn((1, n), torch.bfloat16, 1.0, 3)
    # alpha = 0 leaves the bias; no bias and alpha = 0 leaves zero
    assert np.array_equal(ogemm.linear_expected(w, x, 0.0, bias), np.broadcast_to(bias.double().numpy(), (m, n)))
    assert not ogemm.linear_expected(w, x, 0.0).any()
    # identity weights return the activations, a permutation matrix permutes them, alpha scales
    eye = torch.eye(k, dtype=torch.bfloat16)
    assert np.array_equal(ogemm.linear_expected(eye, x), x.double().numpy())
    perm = torch.randperm(k, generator=torch.Generator().manual_seed(4))
    assert np.array_equal(ogemm.linear_expected(eye[perm], x, 2.0), 2.0 * x.double().numpy()[:, perm])
    # a single element: one term of the sum, checked by hand
    one = torch.zeros((16, 32), dtype=torch.float16)
    one[3, 7] = 1.5
    v = torch.zeros((1, 32), dtype=torch.float16)
    v[0, 7] = -2.0
    out = ogemm.linear_expected(one, v, 1.0)
    assert out[0, 3] == -3.0 and np.count_nonzero(out) == 1
    # agrees with the library product in float64 (independent summation order)
    lib = torch.nn.functional.linear(x.double(), w.double(), bias.double().reshape(-1)).numpy()
    assert np.allclose(ogemm.linear_expected(w, x, 1.0, bias), lib, rtol=1e-12, atol=1e-12)


def test_round_to_is_one_fp32_rounding_then_T():
    v = np.array([1.0 + 2.0 ** -9, 1.0 + 2.0 ** -8 + 2.0 ** -30, -3.0e-8])
    got = ogemm.round_to(v, torch.bfloat16)
    # the middle value sits just above a bf16 tie: fp32 drops the 2^-30, the tie then goes to even (1.0);
    # a direct rounding of the float64 value would give 1.0078125
    assert got.tolist() == [1.0, 1.0, torch.tensor(-3.0e-8).to(torch.bfloat16).item()]


def test_torch_path_linear_is_the_library_linear():
    w = randn((32, 64), torch.float32, 0.5, 5)
    x = randn((3, 64), torch.float32, 1.0, 6)
    assert np.allclose(ogemm.torch_path_linear(w, x).double().numpy(), ogemm.linear_expected(w, x), rtol=1e-5, atol=1e-5)


def test_softfp8_linear_expected_equals_product_on_dequantised_weights():
    codes = fp8_codes((256, 384), 7)
    scale = (torch.rand((2, 3), generator=torch.Generator().manual_seed(8)) * 0.1 + 0.01).float()
    x = randn((2, 384), torch.bfloat16, 1.0, 9)
    w = softfp8.dequant_weight_f32(codes.numpy(), scale.numpy())
    # block (1, 2) really uses scale[1, 2]
    dec = softfp8.decode_e4m3(codes.numpy()[128:, 256:]) * scale.numpy()[1, 2]
    trunc = (dec.astype(np.float32).view(np.uint32) >> 16 << 16).view(np.float32)
    assert np.array_equal(w[128:, 256:], trunc)
    assert np.array_equal(ogemm.softfp8_linear_expected(codes.numpy(), scale.numpy(), x), ogemm.linear_expected(w, x))


def test_torch_path_softfp8_weight_against_the_truncating_statement():
    """The reference's scripts build their expected soft-FP8 weights in bf16 (decode, then a bf16 product with
    the bf16-rounded scale, gemv_benchmark_soft_fp8.py:6-37); the kernels multiply in fp32 and truncate.  With
    power-of-two scales both are exact, hence equal; with any scale they differ by the rounding of the scale
    to bf16 (2^-9) plus one rounding / truncation of the product (2^-8 + 2^-7)."""
    from muxi_native_layout_kernels_amd import utils as shipped
    codes = fp8_codes((256, 256), 11)
    pow2 = torch.tensor([[0.5, 2.0], [0.0625, 1.0]])
    a = ogemm.torch_path_softfp8_weight(codes, pow2)
    b = softfp8.dequant_weight_f32(codes.numpy(), pow2.numpy())
    assert a.dtype == torch.bfloat16 and np.array_equal(a.float().numpy(), b)
    anyscale = torch.tensor([[0.013, 0.37], [1.7, 0.0009]])
    a = ogemm.torch_path_softfp8_weight(codes, anyscale).double().numpy()
    b = softfp8.dequant_weight_f32(codes.numpy(), anyscale.numpy()).astype(np.float64)
    assert np.all(np.abs(a - b) <= (2.0 ** -9 + 2.0 ** -8 + 2.0 ** -7) * np.abs(b))
    # and it is the block-scale helper the package ships under the reference's name (utils.py:14-25)
    w16 = codes.view(torch.float8_e4m3fn).to(torch.bfloat16)
    assert torch.equal(ogemm.torch_path_softfp8_weight(codes, anyscale), shipped.scale_tensor(w16, anyscale))
    # a ragged last block takes the last scale entry
    part = ogemm.torch_path_softfp8_weight(codes[:200, :130], anyscale)
    assert torch.equal(part, ogemm.torch_path_softfp8_weight(codes, anyscale)[:200, :130])


@pytest.mark.parametrize("m,n", [(16, 32), (48, 128)])
def test_layout_c_of_is_the_inverse_of_the_reference_closed_form(m, n):
    """gemm_benchmark.py:74-76 turns a layout-C tensor back into row-major [tokens, rows]:
    `C.view(rows//32, tokens//16, 4, 16, 8).permute(1, 3, 0, 2, 4).contiguous().view(tokens, rows)`."""
    c = randn((m, n), torch.float16, 1.0, 13)
    c_nat = ogemm.layout_c_of(c)
    assert tuple(c_nat.shape) == (n // 32, m // 16, 4, 16, 8) and c_nat.dtype == c.dtype
    back = c_nat.view(n // 32, m // 16, 4, 16, 8).permute(1, 3, 0, 2, 4).contiguous().view(m, n)
    assert torch.equal(back, c)
    assert np.array_equal(layouts.unpack_layout_c(c_nat.view(torch.int16).numpy()), c.view(torch.int16).numpy())
