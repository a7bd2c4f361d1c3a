"""Host-side mirror of the reference's operator interface for the hot path.

Same names, positional order, keyword names and defaults as the pybind module
of the reference (csrc/ffi.cu:32-143); each function checks its arguments the way
the reference's host launcher does, looks up launch parameters in the csv
tables, allocates the output and calls the C-ABI library on torch's current HIP
stream.  PyTorch is used for device memory and streams only.

Reference naming: `m` = weight rows (output features), `k` = reduction,
`n` = activation rows (tokens).
"""
import threading

import torch

from . import _lib, arg_selector

_KIND = {torch.float16: 0, torch.bfloat16: 1}
_FP8_KIND = 2


def _stream():
    return torch.cuda.current_stream().cuda_stream


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream_of(t):
    """Raw handle of torch's current stream on the tensor's device (the short way when torch offers it)."""
    if _raw_stream is not None:
        return _raw_stream(t.get_device())
    return torch.cuda.current_stream(t.device).cuda_stream


# Launch plans of the eager entry points.  The first call with a given combination of shapes, dtypes and device
# runs every argument check and the table lookup, and leaves the launch arguments here; later calls with the same
# combination only check what a shape does not tell (contiguity, alpha / beta), allocate the output and call the
# library.  A plan is a few integers: the cache is never cleared.
_plans = {}


def _ptr(t):
    return 0 if t is None else t.data_ptr()


def _check(cond, msg):
    if not cond:
        raise RuntimeError(msg)


def _is_fp8(t):
    return t.element_size() == 1


def _kind(t):
    if _is_fp8(t):
        return _FP8_KIND
    _check(t.dtype in _KIND, "Unsupported data type")
    return _KIND[t.dtype]


# --------------------------------------------------------------- workspaces
class WorkspacePool:
    """Device scratch handed to the kernels as raw pointers (cross-workgroup K-split partials and their
    arrival counters, the MoE alignment tables and intermediate).

    * One buffer per (device, stream): two calls that run side by side on different streams never share
      counters or partials.  Calls on one stream are ordered, so they can share.
    * A buffer that has been handed out stays allocated for the life of the process.  A HIP graph captured
      earlier replays with the pointer it was captured with; when a later call needs more room, a new, larger
      buffer takes over for new calls and the old one is retired, not freed.
    * `zero_prefix` bytes at the front are cleared when a buffer is created (the K-split kernels count
      arrivals there and leave the counters at zero).
    """

    def __init__(self, min_bytes, zero_prefix=False):
        self.min_bytes = int(min_bytes)
        self.zero_prefix = zero_prefix
        self._lock = threading.Lock()
        self._live = {}
        self._retired = []

    def get(self, device, stream, nbytes, prefix_bytes=0):
        key = (device.type, device.index, int(stream))
        with self._lock:
            buf = self._live.get(key)
            if buf is None or buf.numel() < nbytes:
                if buf is not None:
                    self._retired.append(buf)
                grown = 0 if buf is None else buf.numel() + buf.numel() // 2      # few retirements on a growing series
                size = max(int(nbytes), self.min_bytes, grown)
                buf = torch.empty(size, dtype=torch.uint8, device=device)
                if self.zero_prefix and prefix_bytes:
                    buf[:prefix_bytes].zero_()
                self._live[key] = buf
            return buf

    def owned(self):
        """Every buffer ever handed out (live and retired)."""
        with self._lock:
            return list(self._live.values()) + list(self._retired)

    def held_bytes(self):
        with self._lock:
            return sum(b.numel() for b in self._live.values()) + sum(b.numel() for b in self._retired)

    def release(self, retired_only=False):
        """Drop the retired buffers and, unless `retired_only`, the live ones too (they are re-created on the next
        call).  Only for callers that hold no captured graph which replays one of these pointers, and with no call
        of this library in flight on the device."""
        with self._lock:
            freed = sum(b.numel() for b in self._retired)
            self._retired = []
            if not retired_only:
                freed += sum(b.numel() for b in self._live.values())
                self._live = {}
        return freed


_gemm_pool = WorkspacePool(1 << 22, zero_prefix=True)
_moe_pool = WorkspacePool(1 << 20)


def workspace_bytes_held():
    """Device bytes the library's scratch pools hold right now (K-split partials, MoE tables and intermediates)."""
    return _gemm_pool.held_bytes() + _moe_pool.held_bytes()


def release_workspaces(retired_only=False):
    """Give the scratch memory of the K-split GeMMs and of the fused MoE back to torch's allocator and return the
    number of bytes released.  The pools keep one buffer per (device, stream) and never free by themselves, so that
    a HIP graph captured around a call replays with valid pointers; a caller that holds no such graph (or has
    dropped it) calls this after a burst of large batches, or when streams it used are gone.  `retired_only`
    releases just the buffers that a larger one has replaced.  Synchronize the device first."""
    return _gemm_pool.release(retired_only) + _moe_pool.release(retired_only)


def _workspace(device, nbytes, counter_bytes, stream=None):
    """Scratch for cross-workgroup K splits on `stream` (default: torch's current stream)."""
    return _gemm_pool.get(device, _stream() if stream is None else stream, nbytes, counter_bytes)


# ------------------------------------------------------------------ relayout
def pack_layout_a(weight):
    """[N, K] or [E, N, K] (16-bit or 1-byte elements) -> layout-A [.., N/16, K/8, 16, 8].

    Device counterpart of the offline `A.view(m//16,16,k//8,8).permute(0,2,1,3)`
    (benchmark_and_test/gemv_benchmark.py:47-48, test_muxi_moe.py:74-81)."""
    _check(weight.is_cuda, "weight must be a CUDA tensor")
    _check(weight.is_contiguous(), "weight must be contiguous")
    _check(weight.dim() in (2, 3), "weight must be 2D or 3D")
    n, k = weight.shape[-2], weight.shape[-1]
    _check(n % 16 == 0 and k % 8 == 0, "N % 16 and K % 8 must be 0")
    batch = weight.shape[0] if weight.dim() == 3 else 1
    out = torch.empty(tuple(weight.shape[:-2]) + (n // 16, k // 8, 16, 8), dtype=weight.dtype, device=weight.device)
    lib = _lib.load()
    _lib.check(lib.mlk_pack_layout_a(_ptr(weight), _ptr(out), batch, n, k, weight.element_size(), _stream()),
               "pack_layout_a")
    return out


def unpack_layout_a(a_nat):
    """layout-A [.., N/16, K/8, 16, 8] -> [.., N, K]."""
    _check(a_nat.is_cuda and a_nat.is_contiguous(), "A must be a contiguous CUDA tensor")
    _check(a_nat.dim() in (4, 5) and a_nat.shape[-2] == 16 and a_nat.shape[-1] == 8, "A must be in layout-A")
    n, k = a_nat.shape[-4] * 16, a_nat.shape[-3] * 8
    batch = a_nat.shape[0] if a_nat.dim() == 5 else 1
    out = torch.empty(tuple(a_nat.shape[:-4]) + (n, k), dtype=a_nat.dtype, device=a_nat.device)
    lib = _lib.load()
    _lib.check(lib.mlk_unpack_layout_a(_ptr(a_nat), _ptr(out), batch, n, k, a_nat.element_size(), _stream()),
               "unpack_layout_a")
    return out


def layoutB(B):
    """Row-major activations [n, k] -> layout-B [k/32, n/16, 4, 16, 8] (csrc/layout_b.cu:65-99)."""
    _check(B.is_cuda, "B must be a CUDA tensor")
    _check(B.is_contiguous(), "B must be contiguous")
    _check(B.dim() == 2, "B must be a 2D tensor")
    n, k = B.shape
    _check(n % 16 == 0, "n must be a multiple of 16")
    _check(k % 32 == 0, "k must be a multiple of 32")
    _check(B.dtype in _KIND, "Unsupported data type")
    out = torch.empty((k // 32, n // 16, 4, 16, 8), dtype=B.dtype, device=B.device)
    _lib.check(_lib.load().mlk_layout_b(_ptr(B), _ptr(out), n, k, _stream()), "layoutB")
    return out


def reLayoutC(C):
    """layout-C [m/32, n/16, 4, 16, 8] -> row-major [n, m] (csrc/re_layout_c.cu:63-95)."""
    _check(C.is_cuda, "C must be a CUDA tensor")
    _check(C.is_contiguous(), "C must be contiguous")
    _check(C.dim() == 5, "C must be a 5D tensor")
    _check(C.shape[2] == 4 and C.shape[3] == 16 and C.shape[4] == 8, "C must be in layout-C [m/32, n/16, 4, 16, 8]")
    _check(C.dtype in _KIND, "Unsupported data type")
    m, n = C.shape[0] * 32, C.shape[1] * 16
    out = torch.empty((n, m), dtype=C.dtype, device=C.device)
    _lib.check(_lib.load().mlk_re_layout_c(_ptr(C), _ptr(out), n, m, _stream()), "reLayoutC")
    return out


def fp8_weight_repack(weight):
    """Swap bytes 1 and 2 of every 4-byte group (csrc/fp8_weight_repack.cu:44-67)."""
    _check(weight.is_cuda, "weight must be a CUDA tensor")
    _check(weight.is_contiguous(), "weight must be contiguous")
    _check(weight.element_size() == 1, "weight must hold one byte per element")
    _check(weight.numel() % 4 == 0, "weight size must be a multiple of 4 bytes")
    out = torch.empty_like(weight)
    _lib.check(_lib.load().mlk_fp8_weight_repack(_ptr(weight), _ptr(out), weight.numel(), _stream()),
               "fp8_weight_repack")
    return out


# ---------------------------------------------------------------------- GeMV
def _check_beta(beta):
    # The reference accepts beta everywhere and no kernel of it ever reads it
    # (csrc/layout_gemv_kernel.cuh:377 only derives an unused flag); C is never an input.
    _check(float(beta) == 0.0, "beta != 0 is not supported: the output is never read (the reference ignores beta)")


def _layout_a_dims(A):
    _check(A.dim() == 4, "A must be a 4D tensor")
    _check(A.size(2) == 16, "A.shape[2] must be 16")
    _check(A.size(3) == 8, "A.shape[3] must be 8")
    return A.size(0) * 16, A.size(1) * 8


def gemv_layoutA_wapper(A, B, m, k, alpha=1, beta=0, blockDimX=256, kernelId=1, kernelParam1=1, kernelParam2=1,
                        scale_matrix=None, bias=None):
    """Run the GeMV with explicit launch parameters (csrc/gemv_layout_a.cu:17-71)."""
    _check_beta(beta)
    _check(A.is_cuda and B.is_cuda, "A and B must be CUDA tensors")
    _check(B.dtype in _KIND, "Unsupported data type")
    a_kind = _kind(A)
    if a_kind == _FP8_KIND:
        _check(B.dtype == torch.bfloat16, "Unsupported data type")
        if scale_matrix is not None:
            _check(scale_matrix.dtype == torch.float32 and scale_matrix.is_contiguous(),
                   "scale_matrix must be contiguous fp32")
            _check(tuple(scale_matrix.shape) == ((m + 127) // 128, (k + 127) // 128),
                   "scale_matrix must be [ceil(m/128), ceil(k/128)]")
    else:
        _check(A.dtype == B.dtype, "Unsupported data type")
        scale_matrix = None
    if bias is not None:
        _check(bias.dtype == B.dtype and bias.numel() == m, "bias must be [1, m] of the activation dtype")
    rows = B.size(0)
    C = torch.empty((rows, m), dtype=B.dtype, device=B.device)
    _lib.check(_lib.load().mlk_gemv_layout_a(_ptr(A), _ptr(B), _ptr(C), rows, m, k, a_kind, _KIND[B.dtype],
                                             float(alpha), _ptr(bias), _ptr(scale_matrix), int(blockDimX),
                                             int(kernelId), int(kernelParam1), int(kernelParam2), _stream()),
               "gemv_layoutA")
    return C


def gemv_layoutA(A, B, alpha=1, beta=0, scale_matrix=None, bias=None):
    """y[1, m] = alpha * B[1, k] . A^T (+ bias), A in layout-A (csrc/gemv_layout_a.cu:73-150)."""
    key = ("gemv", A.shape, B.shape, A.dtype, B.dtype, A.device, B.device,
           None if scale_matrix is None else (scale_matrix.shape, scale_matrix.dtype, scale_matrix.device),
           None if bias is None else (bias.shape, bias.dtype, bias.device))
    plan = _plans.get(key)
    if plan is not None and beta == 0 and A.is_contiguous() and B.is_contiguous() and \
            (scale_matrix is None or scale_matrix.is_contiguous()) and (bias is None or bias.is_contiguous()):
        m, k, a_kind, x_kind, block, kid, p1, p2, use_scale, fn = plan
        C = torch.empty((1, m), dtype=B.dtype, device=B.device)
        rc = fn(A.data_ptr(), B.data_ptr(), C.data_ptr(), 1, m, k, a_kind, x_kind, float(alpha),
                0 if bias is None else bias.data_ptr(), scale_matrix.data_ptr() if use_scale else 0,
                block, kid, p1, p2, _stream_of(B))
        if rc != 0:
            _lib.check(rc, "gemv_layoutA")
        return C
    C = _gemv_layoutA_checked(A, B, alpha, beta, scale_matrix, bias)
    m, k = A.size(0) * 16, A.size(1) * 8
    if _is_fp8(A) and B.dtype == torch.bfloat16:
        table = "gemv_soft_fp8"
    else:
        table = "gemv_fp16" if B.dtype == torch.float16 else "gemv_bf16"
    block, kid, p1, p2 = arg_selector.gemv_guard(arg_selector.selector(table).get_args((m, k)), m, k)
    _plans[key] = (m, k, _kind(A), _KIND[B.dtype], block, kid, p1, p2, _is_fp8(A) and scale_matrix is not None,
                   _lib.load().mlk_gemv_layout_a)
    return C


def _gemv_layoutA_checked(A, B, alpha=1, beta=0, scale_matrix=None, bias=None):
    """Every argument check of the reference's host launcher, the table lookup, the launch."""
    _check(A.is_cuda, "A must be a CUDA tensor")
    _check(B.is_cuda, "B must be a CUDA tensor")
    _check(A.is_contiguous(), "A must be contiguous")
    _check(B.is_contiguous(), "B must be contiguous")
    m, a_k = _layout_a_dims(A)
    _check(B.dim() == 2 and B.size(0) == 1, "B must be a vector")
    _check(a_k == B.size(1), "A and B must have the same k")
    k = a_k
    _check(m % 16 == 0, "GEMV m % 16(at least) must be 0")
    _check(k % 32 == 0, "GEMV k % 32(at least) must be 0")
    if _is_fp8(A) and B.dtype == torch.bfloat16:
        sel = arg_selector.selector("gemv_soft_fp8")
    elif B.dtype == torch.float16:
        sel = arg_selector.selector("gemv_fp16")
    elif B.dtype == torch.bfloat16:
        sel = arg_selector.selector("gemv_bf16")
    else:
        raise RuntimeError("Unsupported data type")
    block, kid, p1, p2 = arg_selector.gemv_guard(sel.get_args((m, k)), m, k)
    return gemv_layoutA_wapper(A, B, m, k, alpha, beta, block, kid, p1, p2, scale_matrix, bias)


# ---------------------------------------------------------------------- GEMM
_B_ROWMAJOR, _B_NATIVE = 0, 1
_C_ROWMAJOR, _C_NATIVE = 0, 1


def _gemm_call(A, A_Scale, B, m, n, k, alpha, beta, bias, b_mode, c_mode, kernel_id, p1, p2, p3, what):
    _check_beta(beta)
    _check(B.dtype in _KIND, "Unsupported data type")
    a_kind = _kind(A)
    if a_kind == _FP8_KIND:
        _check(B.dtype == torch.bfloat16, "soft-FP8 weights need bf16 activations")
        if A_Scale is not None:
            _check(A_Scale.dtype == torch.float32 and A_Scale.is_contiguous(), "A_Scale must be contiguous fp32")
            _check(tuple(A_Scale.shape) == ((m + 127) // 128, (k + 127) // 128),
                   "A_Scale must be [ceil(m/128), ceil(k/128)]")
    else:
        _check(A.dtype == B.dtype, "Unsupported data type")
        A_Scale = None
    if bias is not None:
        _check(bias.dtype == B.dtype and bias.numel() == m, "bias must be [1, m] of the activation dtype")
    if c_mode == _C_NATIVE:
        C = torch.empty((m // 32, n // 16, 4, 16, 8), dtype=B.dtype, device=B.device)
    else:
        C = torch.empty((n, m), dtype=B.dtype, device=B.device)
    lib = _lib.load()
    ws = None
    ws_bytes = 0
    if p3 > 1:
        ws_bytes = lib.mlk_gemm_workspace_bytes(n, m, int(p1), int(p3))
        ws = _workspace(B.device, ws_bytes, lib.mlk_gemm_counter_bytes())
        ws_bytes = ws.numel()
    _lib.check(lib.mlk_gemm_layout_a(_ptr(A), _ptr(B), _ptr(C), n, m, k, a_kind, _KIND[B.dtype], b_mode, c_mode,
                                     float(alpha), _ptr(bias), _ptr(A_Scale), int(kernel_id), int(p1), int(p2),
                                     int(p3), _ptr(ws), ws_bytes, _stream()), what)
    return C


def _gemm_guard(args, m):
    kid, p1, p2, p3 = args
    if kid not in (1, 2, 3, 4, 5, 12, 14, 16, 18) or p1 not in (1, 2, 4, 8) or \
            (kid not in (3, 5) and (m // 16) % p1 != 0) or \
            p2 not in (1, 2, 4, 8, 16) or p3 < 1:
        return (1, 1, 4, 1)
    return args


def _gemm_eager(tag, table, checked, A, A_Scale, B, alpha, beta, bias, b_mode, c_mode):
    """The table-driven GeMM entry points behind their launch plans (see `_plans`): `checked` is the function that
    runs every argument check, the table lookup and the launch for a combination not seen before."""
    key = (tag, A.shape, B.shape, A.dtype, B.dtype, A.device, B.device,
           None if A_Scale is None else (A_Scale.shape, A_Scale.dtype, A_Scale.device),
           None if bias is None else (bias.shape, bias.dtype, bias.device))
    plan = _plans.get(key)
    if plan is not None and beta == 0 and A.is_contiguous() and B.is_contiguous() and \
            (A_Scale is None or A_Scale.is_contiguous()) and (bias is None or bias.is_contiguous()):
        m, n, k, a_kind, x_kind, kid, p1, p2, p3, ws_need, counter_bytes, use_scale, c_shape, fn = plan
        C = torch.empty(c_shape, dtype=B.dtype, device=B.device)
        stream = _stream_of(B)
        ws_ptr = ws_len = 0
        if p3 > 1:
            ws = _gemm_pool.get(B.device, stream, ws_need, counter_bytes)
            ws_ptr, ws_len = ws.data_ptr(), ws.numel()
        rc = fn(A.data_ptr(), B.data_ptr(), C.data_ptr(), n, m, k, a_kind, x_kind, b_mode, c_mode, float(alpha),
                0 if bias is None else bias.data_ptr(), A_Scale.data_ptr() if use_scale else 0, kid, p1, p2, p3,
                ws_ptr, ws_len, stream)
        if rc != 0:
            _lib.check(rc, tag)
        return C
    C = checked()
    lib = _lib.load()
    m, k = A.size(0) * 16, A.size(1) * 8
    n = B.size(0) if b_mode == _B_ROWMAJOR else B.size(1) * 16
    kid, p1, p2, p3 = _gemm_guard(arg_selector.selector(table).get_args((m, n, k)), m)
    _plans[key] = (m, n, k, _kind(A), _KIND[B.dtype], kid, p1, p2, p3,
                   lib.mlk_gemm_workspace_bytes(n, m, int(p1), int(p3)) if p3 > 1 else 0, lib.mlk_gemm_counter_bytes(),
                   _is_fp8(A) and A_Scale is not None, tuple(C.shape), lib.mlk_gemm_layout_a)
    return C


def gemm_layoutA_wapper(A, B, m, n, k, alpha=1, beta=0, kernelParam1=1, kernelParam2=1, kernelParam3=1, kernelId=1,
                        bias=None):
    """csrc/gemm_layout_A.cu:684-750 with explicit launch parameters."""
    return _gemm_call(A, None, B, m, n, k, alpha, beta, bias, _B_ROWMAJOR, _C_ROWMAJOR, kernelId, kernelParam1,
                      kernelParam2, kernelParam3, "gemm_layoutA")


def _check_gemm_common(A, B):
    _check(A.is_cuda, "A must be a CUDA tensor")
    _check(B.is_cuda, "B must be a CUDA tensor")
    _check(A.is_contiguous(), "A must be contiguous")
    _check(B.is_contiguous(), "B must be contiguous")


def gemm_layoutA(A, B, alpha=1, beta=0, bias=None):
    """C[n, m] = alpha * B[n, k] . A^T (+ bias); A layout-A, B and C row-major
    (csrc/gemm_layout_A.cu:752-787)."""
    return _gemm_eager("gemm_layoutA", "layoutA_gemm", lambda: _gemm_layoutA_checked(A, B, alpha, beta, bias), A, None, B, alpha, beta, bias,
                       _B_ROWMAJOR, _C_ROWMAJOR)


def _gemm_layoutA_checked(A, B, alpha=1, beta=0, bias=None):
    """Every argument check of the reference's host launcher, the table lookup, the launch."""
    _check_gemm_common(A, B)
    m, a_k = _layout_a_dims(A)
    _check(B.dim() == 2, "B must be a 2D tensor")
    n, b_k = B.size(0), B.size(1)
    _check(a_k == b_k, "A and B must have the same k")
    k = a_k
    _check(m % 128 == 0, "GEMM m % 128 == 0, currently, will be revised soon")
    _check(k % 128 == 0, "GEMM k % 128 must be 0")
    kid, p1, p2, p3 = _gemm_guard(arg_selector.selector("layoutA_gemm").get_args((m, n, k)), m)
    return gemm_layoutA_wapper(A, B, m, n, k, alpha, beta, p1, p2, p3, kid, bias)


def gemm_layoutA_soft_fp8_wapper(A, A_Scale, B, m, n, k, alpha=1, beta=0, kernelParam1=1, kernelParam2=1,
                                 kernelParam3=1, kernelId=1, bias=None):
    """csrc/gemm_layout_A_soft_fp8.cu:749-823 with explicit launch parameters."""
    _check(_is_fp8(A), "A must hold one e4m3 byte per element")
    return _gemm_call(A, A_Scale, B, m, n, k, alpha, beta, bias, _B_ROWMAJOR, _C_ROWMAJOR, kernelId, kernelParam1,
                      kernelParam2, kernelParam3, "gemm_layoutA_soft_fp8")


def gemm_layoutA_soft_fp8(A, A_Scale, B, alpha=1, beta=0, bias=None):
    """Soft-FP8 weights (e4m3 bytes in layout-A + fp32 scale per 128x128 block), bf16
    activations (csrc/gemm_layout_A_soft_fp8.cu:825-862)."""
    return _gemm_eager("gemm_layoutA_soft_fp8", "layoutA_soft_fp8_gemm", lambda: _gemm_layoutA_soft_fp8_checked(A, A_Scale, B, alpha, beta, bias), A, A_Scale, B, alpha,
                       beta, bias, _B_ROWMAJOR, _C_ROWMAJOR)


def _gemm_layoutA_soft_fp8_checked(A, A_Scale, B, alpha=1, beta=0, bias=None):
    """Every argument check of the reference's host launcher, the table lookup, the launch."""
    _check_gemm_common(A, B)
    m, a_k = _layout_a_dims(A)
    _check(B.dim() == 2, "B must be a 2D tensor")
    n, b_k = B.size(0), B.size(1)
    _check(a_k == b_k, "A and B must have the same k")
    k = a_k
    _check(m % 128 == 0, "GEMM m % 128 == 0, currently, will be revised soon")
    _check(k % 128 == 0, "GEMM k % 128 must be 0")
    _check(B.dtype == torch.bfloat16, "soft-FP8 weights need bf16 activations")
    kid, p1, p2, p3 = _gemm_guard(arg_selector.selector("layoutA_soft_fp8_gemm").get_args((m, n, k)), m)
    return gemm_layoutA_soft_fp8_wapper(A, A_Scale, B, m, n, k, alpha, beta, p1, p2, p3, kid, bias)


def gemm_layoutA_linear(A, B, alpha=1, beta=0, scale_matrix=None, bias=None):
    """Route on the presence of a scale matrix (csrc/gemm_layoutA_linear.cu:9-18)."""
    if scale_matrix is not None:
        return gemm_layoutA_soft_fp8(A, scale_matrix, B, alpha, beta, bias)
    return gemm_layoutA(A, B, alpha, beta, bias)


def _native_b_dims(B):
    _check(B.dim() == 5, "B must be a 5D tensor")
    _check(B.size(2) == 4, "B.shape[2] must be 4")
    _check(B.size(3) == 16, "B.shape[3] must be 16")
    _check(B.size(4) == 8, "B.shape[4] must be 8")
    return B.size(1) * 16, B.size(0) * 32


def gemm_layoutAB_ContinuousC_wapper(A, B, m, n, k, alpha=1, beta=0, kernelParam1=1, kernelParam2=1, kernelParam3=1,
                                     kernelId=1, bias=None):
    """csrc/gemm_layout_ab_continuous_c.cu with explicit launch parameters."""
    return _gemm_call(A, None, B, m, n, k, alpha, beta, bias, _B_NATIVE, _C_ROWMAJOR, kernelId, kernelParam1,
                      kernelParam2, kernelParam3, "gemm_layoutAB_ContinuousC")


def gemm_layoutAB_ContinuousC(A, B, alpha=1, beta=0, bias=None):
    """A layout-A, B layout-B, C row-major [n, m] (csrc/gemm_layout_ab_continuous_c.cu:1051-1093)."""
    return _gemm_eager("gemm_layoutAB_ContinuousC", "continuous_gemm", lambda: _gemm_layoutAB_ContinuousC_checked(A, B, alpha, beta, bias), A, None, B, alpha, beta, bias,
                       _B_NATIVE, _C_ROWMAJOR)


def _gemm_layoutAB_ContinuousC_checked(A, B, alpha=1, beta=0, bias=None):
    """Every argument check of the reference's host launcher, the table lookup, the launch."""
    _check_gemm_common(A, B)
    m, a_k = _layout_a_dims(A)
    n, b_k = _native_b_dims(B)
    _check(a_k == b_k, "A and B must have the same k")
    k = a_k
    _check(m % 128 == 0, "GEMM m % 128 == 0, currently, will be revised soon")
    _check(k % 128 == 0, "GEMM k % 128 must be 0")
    kid, p1, p2, p3 = _gemm_guard(arg_selector.selector("continuous_gemm").get_args((m, n, k)), m)
    return gemm_layoutAB_ContinuousC_wapper(A, B, m, n, k, alpha, beta, p1, p2, p3, kid, bias)


def gemm_layoutABC_wapper(A, B, m, n, k, alpha=1, beta=0, kernelParam1=1, kernelParam2=1, kernelParam3=1,
                          kernelId=1, bias=None):
    """csrc/gemm_layout_abc.cu with explicit launch parameters."""
    return _gemm_call(A, None, B, m, n, k, alpha, beta, bias, _B_NATIVE, _C_NATIVE, kernelId, kernelParam1,
                      kernelParam2, kernelParam3, "gemm_layoutABC")


def gemm_layoutABC(A, B, alpha=1, beta=0, bias=None):
    """A layout-A, B layout-B, C layout-C [m/32, n/16, 4, 16, 8], ready to be the B of the
    next product (csrc/gemm_layout_abc.cu:754-791)."""
    return _gemm_eager("gemm_layoutABC", "layout_gemm", lambda: _gemm_layoutABC_checked(A, B, alpha, beta, bias), A, None, B, alpha, beta, bias,
                       _B_NATIVE, _C_NATIVE)


def _gemm_layoutABC_checked(A, B, alpha=1, beta=0, bias=None):
    """Every argument check of the reference's host launcher, the table lookup, the launch."""
    _check_gemm_common(A, B)
    m, a_k = _layout_a_dims(A)
    n, b_k = _native_b_dims(B)
    _check(a_k == b_k, "A and B must have the same k")
    k = a_k
    _check(m % 128 == 0, "GEMM m % 128 == 0, currently, will be revised soon")
    _check(k % 128 == 0, "GEMM k % 128 must be 0")
    kid, p1, p2, p3 = _gemm_guard(arg_selector.selector("layout_gemm").get_args((m, n, k)), m)
    return gemm_layoutABC_wapper(A, B, m, n, k, alpha, beta, p1, p2, p3, kid, bias)


# ----------------------------------------------------------------------- MoE
def fused_routing_gate(gating_output, score_fun, batch_size, hidden_size, n_groups, topK_groups, experts_ids,
                       selected_experts_weights, topK, load_balance_bias=None, renormalize=False):
    """Router: writes `experts_ids` (int32 [T, K]) and `selected_experts_weights` ([T, K]) in place and
    returns None (csrc/moe_kernels/fused_gating.cu:5-67).  `renormalize` is an extension: the reference
    leaves the division to its Python caller (muxi_moe_planC.py:69-70)."""
    _check(gating_output.dtype == selected_experts_weights.dtype,
           "Mismatched dtypes: gating_output and selected_experts_weights.")
    if load_balance_bias is not None:
        _check(load_balance_bias.dtype == gating_output.dtype,
               "Mismatched dtypes: load_balance_bias and gating_output.")
    _check(gating_output.dtype in _KIND, "Invalid dtype for gating_output: must be kFloat16 or kBFloat16.")
    _check(experts_ids.dtype == torch.int32, "Invalid dtype for experts_ids: must be kInt32.")
    _check(experts_ids.device == selected_experts_weights.device,
           "Device mismatch: experts_ids and selected_experts_weights.")
    _check(gating_output.is_cuda and gating_output.is_contiguous(), "gating_output must be a contiguous CUDA tensor")
    n_experts = gating_output.size(-1)
    _check(int(batch_size) * n_experts == gating_output.numel(), "batch_size does not match gating_output")
    _check(1 <= n_experts <= 256, "the router supports at most 256 experts")
    _check(n_groups >= 1 and n_experts % n_groups == 0, "n_groups must divide the number of experts")
    _check(1 <= topK_groups <= n_groups, "topK_groups must be in 1..n_groups")
    _check(1 <= topK <= min(32, n_experts), "topK must be in 1..min(32, experts)")
    _check(experts_ids.numel() >= batch_size * topK and selected_experts_weights.numel() >= batch_size * topK,
           "output tensors are too small")
    _lib.check(_lib.load().mlk_fused_routing_gate(_ptr(gating_output), _KIND[gating_output.dtype], int(score_fun),
                                                  int(batch_size), n_experts, int(n_groups), int(topK_groups),
                                                  int(topK), _ptr(load_balance_bias), int(bool(renormalize)),
                                                  _ptr(experts_ids), _ptr(selected_experts_weights), _stream()),
               "fused_routing_gate")
    return None


def batched_routed_activation_indexed_to_expert_block_indexed(batchSize, expertCount, topK, microBatchSize,
                                                              expertsIds, dev_sorted_token_ids, dev_cumsum_buffer,
                                                              dev_padded_num_experts, dev_experts_ids,
                                                              experts_map=None):
    """Token -> expert-block permutation (csrc/moe_kernels/fused_experts_compute.cu:6-48)."""
    _check(expertsIds.dtype == torch.int32, "expertsIds must be of type torch::kInt32.")
    for t, name in ((dev_sorted_token_ids, "dev_sorted_token_ids"), (dev_cumsum_buffer, "dev_cumsum_buffer"),
                    (dev_padded_num_experts, "dev_padded_num_experts"), (dev_experts_ids, "dev_experts_ids")):
        _check(expertsIds.device == t.device, "expertsIds must be on the same device as %s." % name)
        _check(t.dtype == torch.int32, "%s must be int32" % name)
    _check(microBatchSize == 16, "microBatchSize must be 16")
    _check(1 <= expertCount <= 1024, "expertCount must be in 1..1024")
    n_pairs = int(batchSize) * int(topK)
    _check(expertsIds.numel() >= n_pairs, "expertsIds is too small")
    padded = n_pairs + expertCount * (microBatchSize - 1)
    _check(dev_sorted_token_ids.numel() >= padded, "dev_sorted_token_ids is too small")
    _check(dev_cumsum_buffer.numel() >= expertCount + 1, "dev_cumsum_buffer is too small")
    _check(dev_experts_ids.numel() >= (padded + microBatchSize - 1) // microBatchSize, "dev_experts_ids is too small")
    if experts_map is not None:
        _check(experts_map.dtype == torch.int32, "experts_map must be int32")
    _lib.check(_lib.load().mlk_moe_align_tokens(_ptr(expertsIds), n_pairs, int(expertCount), int(microBatchSize),
                                                _ptr(experts_map), _ptr(dev_sorted_token_ids),
                                                _ptr(dev_cumsum_buffer), _ptr(dev_padded_num_experts),
                                                _ptr(dev_experts_ids), _stream()), "moe_align_tokens")
    return None


def _moe_workspace(device, nbytes, stream=None):
    return _moe_pool.get(device, _stream() if stream is None else stream, nbytes)


def fused_experts_compute(experts_weights_matrix1, experts_weights_matrix2, activations, batch_size, expert_count,
                          dynamic_experts_per_act, topk_ids, actived_experts_weights, sorted_token_ids, cumsum_buffer,
                          padded_num_experts, experts_ids, C, y, *args, **kwargs):
    """Both overloads of the reference's `fused_experts_compute` (ffi.cu:112-143):

    16-bit weights: (..., APerWarp=2, splitK=3, tile_m_2=128, tile_n_2=16, tile_k_2=128, block_dim_x_gemm=256,
                     microBatchSize=16, experts_map=None)
    soft-FP8:       (..., w1_scale, w2_scale, block_shape, soft_fp8=False, microBatchSize=16, experts_map=None)

    The overload is chosen as pybind does, from the type of the first extra argument.  Runs the alignment,
    the grouped gate/up GeMM with SiLU*up, the grouped down GeMM and the weighted sum into `y`.  `C` (the
    reference's intermediate buffer) is accepted and left untouched: the intermediate lives in a cached
    workspace in a layout the second GeMM can stream.  The MetaX tile parameters are accepted and ignored."""
    w1, w2, x = experts_weights_matrix1, experts_weights_matrix2, activations
    fp8 = (len(args) > 0 and isinstance(args[0], torch.Tensor)) or "w1_scale" in kwargs
    if fp8:
        names = ["w1_scale", "w2_scale", "block_shape", "soft_fp8", "microBatchSize", "experts_map"]
        defaults = {"soft_fp8": False, "microBatchSize": 16, "experts_map": None}
    else:
        names = ["APerWarp", "splitK", "tile_m_2", "tile_n_2", "tile_k_2", "block_dim_x_gemm", "microBatchSize",
                 "experts_map"]
        defaults = {"APerWarp": 2, "splitK": 3, "tile_m_2": 128, "tile_n_2": 16, "tile_k_2": 128,
                    "block_dim_x_gemm": 256, "microBatchSize": 16, "experts_map": None}
    _check(len(args) <= len(names), "fused_experts_compute: too many positional arguments")
    opts = dict(defaults)
    for name, val in zip(names, args):
        opts[name] = val
    for name, val in kwargs.items():
        _check(name in names and name not in names[:len(args)], "fused_experts_compute: unexpected argument %s" % name)
        opts[name] = val
    for name in names:
        _check(name in opts, "fused_experts_compute: missing argument %s" % name)

    _check(w1.dtype == w2.dtype, "experts_weights_matrix1 and experts_weights_matrix2 must have the same dtype.")
    _check(topk_ids.dtype == torch.int32, "expertsIds must be of type torch::kInt32.")
    _check(x.dtype == actived_experts_weights.dtype, "activations and activedExpertsWeights must have the same dtype.")
    _check(x.dtype == y.dtype, "activations and y must have the same dtype.")
    _check(x.dtype in _KIND, "activations must be fp16 or bf16")
    for t in (w1, w2, x, topk_ids, actived_experts_weights, sorted_token_ids, cumsum_buffer, padded_num_experts,
              experts_ids, y):
        _check(t.is_cuda and t.is_contiguous(), "all tensors must be contiguous CUDA tensors")
    w1_scale = w2_scale = None
    if fp8:
        _check(w1.element_size() == 1, "experts weights must be float8_e4m3fn bytes for the soft-FP8 overload.")
        w1_scale, w2_scale = opts["w1_scale"], opts["w2_scale"]
        _check(w1_scale.dtype == torch.float32 and w2_scale.dtype == torch.float32, "scales must be float32.")
        _check(w1_scale.device == w2_scale.device, "w1_scale and w2_scale must be on the same device.")
        block_shape = list(opts["block_shape"])
        _check(len(block_shape) == 2, "block_shape must have size 2.")
        _check(block_shape[0] == 128 and block_shape[1] == 128, "block_shape must be (128, 128) for float8_e4m3fn.")
        _check(bool(opts["soft_fp8"]), "soft_fp8 must be true for float8_e4m3fn.")
        _check(x.dtype == torch.bfloat16, "Weight date type and activation date type mismatch")
        w_kind = _FP8_KIND
    else:
        _check(w1.dtype == x.dtype, "Weight date type and activation date type mismatch")
        w_kind = _KIND[w1.dtype]
    _check(opts["microBatchSize"] == 16, "microBatchSize must be 16")
    # per-expert slabs: either the flattened [E, 2I, H] view the reference's tests pass or [E, 2I/16, H/8, 16, 8]
    if w1.dim() == 5:
        e1, m1, k1 = w1.shape[0], w1.shape[1] * 16, w1.shape[2] * 8
        e2, m2, k2 = w2.shape[0], w2.shape[1] * 16, w2.shape[2] * 8
    else:
        _check(w1.dim() == 3 and w2.dim() == 3, "expert weights must be [E, rows, cols]")
        e1, m1, k1 = w1.shape
        e2, m2, k2 = w2.shape
    _check(e1 == e2 == expert_count, "expert count mismatch")
    _check(k1 == m2 and m1 == 2 * k2, "w1 must be [E, 2I, H] and w2 [E, H, I]")
    hidden, inter = k1, k2
    _check(hidden % 128 == 0 and inter % 128 == 0, "hidden and intermediate sizes must be multiples of 128")
    T, K = int(batch_size), int(dynamic_experts_per_act)
    _check(x.numel() == T * hidden and y.numel() == T * hidden, "activations / y must be [batch, hidden]")
    if fp8:
        _check(tuple(w1_scale.shape) == (e1, m1 // 128, k1 // 128) and w1_scale.is_contiguous(),
               "w1_scale must be [E, 2I/128, H/128]")
        _check(tuple(w2_scale.shape) == (e2, m2 // 128, k2 // 128) and w2_scale.is_contiguous(),
               "w2_scale must be [E, H/128, I/128]")
    experts_map = opts["experts_map"]
    if experts_map is not None:
        _check(experts_map.dtype == torch.int32 and experts_map.is_cuda, "experts_map must be an int32 CUDA tensor")
    # the reference fills the caller's alignment buffers as a side effect of this call
    batched_routed_activation_indexed_to_expert_block_indexed(T, e1, K, 16, topk_ids, sorted_token_ids, cumsum_buffer,
                                                              padded_num_experts, experts_ids, experts_map)
    experts_compute_raw(w1, w2, x, T, e1, K, hidden, inter, w_kind, topk_ids, actived_experts_weights, experts_map,
                        w1_scale, w2_scale, y)
    return None


def experts_compute_raw(w1, w2, x, T, E, K, hidden, inter, w_kind, topk_ids, topk_weights, experts_map, w1_scale,
                        w2_scale, y):
    """Thin call of the C entry point (alignment + both grouped GeMMs + weighted sum); no checks."""
    lib = _lib.load()
    ws = _moe_workspace(x.device, lib.mlk_moe_workspace_bytes(T, E, K, hidden, inter))
    _lib.check(lib.mlk_fused_experts_compute(_ptr(w1), _ptr(w2), _ptr(x), T, E, K, hidden, inter, w_kind,
                                             _KIND[x.dtype], _ptr(topk_ids), _ptr(topk_weights), _ptr(experts_map),
                                             _ptr(w1_scale), _ptr(w2_scale), _ptr(y), _ptr(ws), ws.numel(),
                                             _stream()), "fused_experts_compute")


def fused_moe_raw(w1, w2, x, logits, T, E, K, hidden, inter, w_kind, score_fun, n_groups, topk_groups, bias,
                  renormalize, experts_map, w1_scale, w2_scale, topk_ids, topk_weights, y):
    """Thin call of the whole-layer entry point (router + alignment + both grouped GeMMs + weighted sum); no
    checks.  `topk_ids` / `topk_weights` receive the routing."""
    lib = _lib.load()
    ws = _moe_workspace(x.device, lib.mlk_moe_workspace_bytes(T, E, K, hidden, inter))
    _lib.check(lib.mlk_fused_moe(_ptr(w1), _ptr(w2), _ptr(x), _ptr(logits), T, logits.size(-1), E, K, hidden, inter,
                                 w_kind, _KIND[x.dtype], score_fun, n_groups, topk_groups, _ptr(bias),
                                 int(bool(renormalize)), _ptr(experts_map), _ptr(w1_scale), _ptr(w2_scale),
                                 _ptr(topk_ids), _ptr(topk_weights), _ptr(y), _ptr(ws), ws.numel(), _stream()),
               "fused_moe")


# ------------------------------------------------- names outside the hot path
def _out_of_scope(name, why):
    def fn(*args, **kwargs):
        raise NotImplementedError("%s is outside the weight-stationary hot path: %s" % (name, why))
    fn.__name__ = name
    return fn


gemmEx = _out_of_scope("gemmEx", "it wraps the vendor BLAS of the reference (csrc/gemm_ex.cu); use torch.matmul")
muxi_hgemm = _out_of_scope("muxi_hgemm", "large-tile prefill GEMM (csrc/muxi_hgemm.cu); use torch.matmul / hipBLASLt")
muxi_hgemm_layout = _out_of_scope("muxi_hgemm_layout", "large-tile prefill GEMM (csrc/muxi_hgemm_layout.cu)")
muxi_hgemm_layoutA = _out_of_scope("muxi_hgemm_layoutA", "large-tile prefill GEMM (csrc/muxi_hgemm_layoutA.cu)")
muxi_hgemm_layoutC = _out_of_scope("muxi_hgemm_layoutC", "large-tile prefill GEMM (csrc/muxi_hgemm_layoutC.cu)")
routing_gate = _out_of_scope("routing_gate", "legacy split MoE (csrc/moe_kernels/routing_gate.cu); use fused_routing_gate")
experts_compute = _out_of_scope("experts_compute",
                                "legacy split MoE (csrc/moe_kernels/experts_compute.cu); use fused_experts_compute")

__all__ = [
    "layoutB", "reLayoutC", "gemm_layoutABC", "gemm_layoutA_linear", "gemm_layoutA", "gemm_layoutA_soft_fp8",
    "gemm_layoutAB_ContinuousC", "gemmEx", "muxi_hgemm", "muxi_hgemm_layout", "muxi_hgemm_layoutA",
    "muxi_hgemm_layoutC", "gemv_layoutA", "gemm_layoutABC_wapper", "gemm_layoutA_wapper",
    "gemm_layoutA_soft_fp8_wapper", "gemm_layoutAB_ContinuousC_wapper", "gemv_layoutA_wapper", "fp8_weight_repack",
    "routing_gate", "experts_compute", "fused_routing_gate",
    "batched_routed_activation_indexed_to_expert_block_indexed", "fused_experts_compute",
    "pack_layout_a", "unpack_layout_a", "experts_compute_raw", "release_workspaces", "workspace_bytes_held",
    "fused_moe_raw",
]
