"""GeMV / narrow GeMM expected values, restated on the CPU.

TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).

The reference's scripts take their expected value from a matrix product on the
UN-PACKED weights plus bias (benchmark_and_test/gemv_benchmark.py:20-41,
gemm_benchmark.py:74-76); the epilogue is `T(alpha * acc)` then `+ bias`
(csrc/layout_gemv_kernel.cuh:191-212, csrc/gemm_layout_A.cu:236-257).  `beta`
is accepted and never read by any kernel of the reference.

Pinned by the textbook product: float64 accumulation here, so any fp32
accumulation order is within the stated tolerance of it; special cases
(alpha = 0, identity weights) are closed forms checked in the tests.
"""
import numpy as np
import torch

from . import layouts, softfp8


def to_f64(t):
    """torch tensor (fp16 / bf16 / fp32) or ndarray -> float64 ndarray."""
    if isinstance(t, torch.Tensor):
        return t.detach().cpu().to(torch.float64).numpy()
    return np.asarray(t, dtype=np.float64)


def round_to(x64, dtype):
    """float64 ndarray -> torch tensor of `dtype` through one fp32 rounding
    (the kernels hold fp32 accumulators and convert once)."""
    return torch.from_numpy(np.asarray(x64, dtype=np.float64)).to(torch.float32).to(dtype)


def linear_expected(w, x, alpha=1.0, bias=None):
    """Exact (float64) alpha * x @ w^T + bias for w [N, K], x [M, K] -> [M, N]."""
    acc = to_f64(x) @ to_f64(w).T
    out = float(alpha) * acc
    if bias is not None:
        out = out + to_f64(bias).reshape(1, -1)
    return out


def softfp8_linear_expected(w_codes, scale, x, alpha=1.0, bias=None):
    """Same with W = trunc_bf16(e4m3 * scale[128x128 block]) (csrc/utils.cuh:80-99,
    scale layout csrc/gemm_layout_A_soft_fp8.cu:110-112, utils.py:14-25)."""
    w = softfp8.dequant_weight_f32(np.asarray(w_codes, dtype=np.uint8), scale)
    return linear_expected(w, x, alpha, bias)


def torch_path_linear(w, x, bias=None):
    """The reference's CPU-runnable path for GeMV / GeMM: a library linear on the
    un-packed weights in the configuration's dtype (gemv_benchmark.py:20-41 uses
    the vendor BLAS for the same product).  This is what the benchmark times on
    the host cores."""
    return torch.nn.functional.linear(x, w, bias)


def torch_path_softfp8_weight(w_codes_t, scale_t):
    """bytes -> float8_e4m3fn -> bf16 -> times the 128x128 block scale in bf16, as
    benchmark_and_test/gemv_benchmark_soft_fp8.py:6-37 builds its expected
    weights (`scale_tensor`, muxi_layout_kernels/utils.py:14-25)."""
    w = w_codes_t.view(torch.float8_e4m3fn).to(torch.bfloat16)
    n, k = w.shape
    s = scale_t.to(torch.bfloat16).repeat_interleave(128, 0)[:n].repeat_interleave(128, 1)[:, :k]
    return w * s


def layout_c_of(c_rowmajor_t):
    """Row-major [M, N] torch tensor -> layout-C tensor, via the oracle permutation."""
    bits = c_rowmajor_t.contiguous().view(torch.int16).numpy()
    return torch.from_numpy(layouts.pack_layout_c(bits)).view(c_rowmajor_t.dtype)
