"""Native layouts A / B / C and the fp8 byte repack, restated on the CPU.

TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).

All three layouts are permutations of 8-element granules.  Every function
works on numpy arrays of any itemsize (the permutation never looks inside an
element), so NaN payloads and arbitrary bit patterns survive.

Two independent statements are given for each layout: the closed form the
reference's own scripts hold (`*_closed`), and an element-by-element index
loop written from the kernels' address arithmetic (`*_loop`).  The tests
require them to agree; a transposed operand or a wrong stride fails there.
"""
import numpy as np


# ----------------------------------------------------------------- layout-A
def pack_layout_a(w):
    """[N, K] -> [N/16, K/8, 16, 8]:  A_nat[g, o, r, e] = A[16 g + r, 8 o + e].

    Closed form held by the reference: benchmark_and_test/gemv_benchmark.py:47-48
    (`A.view(m//16,16,k//8,8).permute(0,2,1,3).contiguous()`), same expression in
    gemm_benchmark.py:41-42 and test_muxi_moe.py:74-81.
    """
    n, k = w.shape
    assert n % 16 == 0 and k % 8 == 0
    return np.ascontiguousarray(w.reshape(n // 16, 16, k // 8, 8).transpose(0, 2, 1, 3))


def unpack_layout_a(a_nat):
    """Inverse of pack_layout_a: [N/16, K/8, 16, 8] -> [N, K]."""
    g, o, r, e = a_nat.shape
    assert r == 16 and e == 8
    return np.ascontiguousarray(a_nat.transpose(0, 2, 1, 3)).reshape(g * 16, o * 8)


def pack_layout_a_loop(w):
    """Index-loop statement of layout-A, following the host-side shape contract
    csrc/gemv_layout_a.cu:83-87 and the lane addressing `base + laneId` of
    csrc/layout_gemv_kernel.cuh:66-68 (lane = 16 q + r reads row r, octet q)."""
    n, k = w.shape
    out = np.empty((n // 16, k // 8, 16, 8), dtype=w.dtype)
    for row in range(n):
        for col in range(k):
            out[row // 16, col // 8, row % 16, col % 8] = w[row, col]
    return out


# ----------------------------------------------------------------- layout-B
def pack_layout_b(b):
    """[M, K] -> [K/32, M/16, 4, 16, 8]:  B_nat[c, g, q, r, e] = B[16 g + r, 32 c + 8 q + e].

    Closed form held by the reference: benchmark_and_test/transposeB_bench.py:10-11
    (`B.view(n//16,16,k//32,4,8).permute(2,0,3,1,4).contiguous()`); the device
    kernel is csrc/layout_b.cu:12-63 (offsets :34-46, output shape :73).
    """
    m, k = b.shape
    assert m % 16 == 0 and k % 32 == 0
    return np.ascontiguousarray(b.reshape(m // 16, 16, k // 32, 4, 8).transpose(2, 0, 3, 1, 4))


def unpack_layout_b(b_nat):
    """Inverse of pack_layout_b: [K/32, M/16, 4, 16, 8] -> [M, K]."""
    c, g, q, r, e = b_nat.shape
    assert (q, r, e) == (4, 16, 8)
    return np.ascontiguousarray(b_nat.transpose(1, 3, 0, 2, 4)).reshape(g * 16, c * 32)


def pack_layout_b_loop(b):
    """Index-loop statement following csrc/layout_b.cu:34-46: the source granule of
    (row 16 g + r, k-octet 4 c + q) goes to output granule (c * M/16 + g) * 64 + 16 q + r."""
    m, k = b.shape
    flat = np.empty((k // 32) * (m // 16) * 64 * 8, dtype=b.dtype)
    for row in range(m):
        for col in range(k):
            g, r = divmod(row, 16)
            c, rem = divmod(col, 32)
            q, e = divmod(rem, 8)
            granule = (c * (m // 16) + g) * 64 + 16 * q + r
            flat[granule * 8 + e] = b[row, col]
    return flat.reshape(k // 32, m // 16, 4, 16, 8)


# ----------------------------------------------------------------- layout-C
def pack_layout_c(c):
    """Row-major output C[M, N] -> [N/32, M/16, 4, 16, 8].

    Layout-C of a product is layout-B of the next product with k := N; store
    address arithmetic csrc/gemm_layout_abc.cu:78-90.
    """
    return pack_layout_b(c)


def unpack_layout_c(c_nat):
    """[N/32, M/16, 4, 16, 8] -> row-major [M, N].

    Closed form held by the reference: benchmark_and_test/gemm_benchmark.py:74-76
    (`C.view(m//32,n//16,4,16,8).permute(1,3,0,2,4).contiguous().view(n,m)`);
    device kernel csrc/re_layout_c.cu:12-61.
    """
    return unpack_layout_b(c_nat)


# ------------------------------------------------------- fp8 weight repack
def fp8_weight_repack(w_bytes):
    """Swap bytes 1 and 2 of every aligned 4-byte group of a uint8 array.

    csrc/fp8_weight_repack.cu:35-36:
    `(w & 0xff0000ff) | ((w & 0x00ff0000) >> 8) | ((w & 0x0000ff00) << 8)`.
    The reference only visits whole 256x256 blocks (:54); this statement covers
    every dword, which is the same result wherever the reference writes at all.
    """
    w = np.ascontiguousarray(w_bytes)
    assert w.dtype == np.uint8 and w.size % 4 == 0
    d = w.reshape(-1).view("<u4")
    out = (d & np.uint32(0xFF0000FF)) | ((d & np.uint32(0x00FF0000)) >> np.uint32(8)) | (
        (d & np.uint32(0x0000FF00)) << np.uint32(8))
    return out.view(np.uint8).reshape(w.shape)


def fp8_weight_repack_loop(w_bytes):
    """Byte-index statement: out[4 i + (0, 1, 2, 3)] = in[4 i + (0, 2, 1, 3)]."""
    w = np.ascontiguousarray(w_bytes).reshape(-1)
    out = np.empty_like(w)
    for i in range(0, w.size, 4):
        out[i], out[i + 1], out[i + 2], out[i + 3] = w[i], w[i + 2], w[i + 1], w[i + 3]
    return out.reshape(w_bytes.shape)
