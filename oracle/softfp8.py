"""Soft-FP8 widening: e4m3 bytes -> bf16 weights, restated on the CPU.

TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).

Restates `scalefp8tobf16` (csrc/utils.cuh:80-99, second copy :232-251, third
copy csrc/moe_kernels/group_gemm_utils.h:73-92) with integer and fp32 numpy
arithmetic:

    interm = sign << 31 | (byte & 0x7f) << 20          an fp32 equal to value * 2^-120
    bias   = fp32(2^120) * fp32(scale)                 0x7b800000 is 2^120
    out    = bits(fp32(bias * interm)) >> 16           truncation to bf16

Pinned by: for the 254 codes other than 0x7f / 0xff, `interm * 2^120` equals
the library decode of the byte as float8_e4m3fn exactly (tests compare with
torch's float8_e4m3fn view); the two NaN codes decode as +-480 = 1.875 * 2^8,
the closed form of "exponent 15, mantissa 7" without the NaN special case.
"""
import numpy as np

_TWO_POW_120_BITS = np.uint32(0x7B800000)


def widen_bits(codes):
    """e4m3 bytes -> fp32 bit patterns of value * 2^-120 (csrc/utils.cuh:87-97)."""
    c = np.asarray(codes, dtype=np.uint8).astype(np.uint32)
    return ((c & np.uint32(0x80)) << np.uint32(24)) | ((c & np.uint32(0x7F)) << np.uint32(20))


def decode_e4m3(codes):
    """e4m3 bytes -> float32 value as the reference decodes it (NaN codes -> +-480)."""
    small = widen_bits(codes).view(np.float32)
    two120 = np.array([_TWO_POW_120_BITS], dtype=np.uint32).view(np.float32)[0]
    with np.errstate(over="ignore"):
        return (small * two120).astype(np.float32)


def dequant_bf16_bits(codes, scale):
    """bytes, per-element fp32 scale (broadcastable) -> bf16 bit patterns (uint16).

    Order of operations as in csrc/utils.cuh:82-86: the scale is first folded
    into the 2^120 constant (one fp32 rounding), then multiplied by the widened
    value (second fp32 rounding), then the low 16 bits are dropped.
    """
    two120 = np.array([_TWO_POW_120_BITS], dtype=np.uint32).view(np.float32)[0]
    with np.errstate(over="ignore", invalid="ignore"):
        bias = (np.float32(two120) * np.asarray(scale, dtype=np.float32)).astype(np.float32)
        prod = (bias * widen_bits(codes).view(np.float32)).astype(np.float32)
    return (prod.view(np.uint32) >> np.uint32(16)).astype(np.uint16)


def bf16_bits_to_f32(bits):
    return (np.asarray(bits, dtype=np.uint16).astype(np.uint32) << np.uint32(16)).view(np.float32)


def expand_block_scale(scale, n, k, block=128):
    """[ceil(N/128), ceil(K/128)] fp32 -> [N, K]: one factor per 128x128 block.

    Block indexing as in `scale_tensor`, muxi_layout_kernels/utils.py:14-25, and
    the kernel's scale index csrc/layout_gemv_kernel_soft_fp8.cuh:129-134.
    """
    s = np.asarray(scale, dtype=np.float32)
    rows = np.arange(n) // block
    cols = np.arange(k) // block
    return s[np.ix_(rows, cols)]


def dequant_weight_f32(w_codes, scale=None, block=128):
    """uint8 [N, K] (+ block scale) -> float32 [N, K] holding the truncated-bf16 weights."""
    n, k = w_codes.shape
    full = np.ones((n, k), np.float32) if scale is None else expand_block_scale(scale, n, k, block)
    return bf16_bits_to_f32(dequant_bf16_bits(w_codes, full))
