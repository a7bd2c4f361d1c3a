"""GPU: the entry point that allocates nothing (`mlk_gemm_layout_a_noalloc`, K-split scratch in a static device
array) against `mlk_gemm_layout_a` with a caller-owned workspace, through the C ABI.  Same kernels, same fold
order: the outputs must be equal bit for bit, on two calls in a row, the second with a smaller input."""
import pytest
import torch

from oracle import gemm as ogemm
from helpers import randn, pack_a, assert_close

pytestmark = pytest.mark.gpu


def _lib():
    from muxi_native_layout_kernels_amd import _lib as binding
    return binding.load()


def _both(lib, w, b, kernel_id, p1, p2, p3, alpha=1.0, bias=None):
    """(no-alloc output, workspace-argument output) for C = alpha * b . w^T + bias on the current stream."""
    n, k = w.shape
    m = b.shape[0]
    kind = {torch.float16: 0, torch.bfloat16: 1}[w.dtype]
    a = pack_a(w).cuda()
    bd = b.cuda()
    biasd = None if bias is None else bias.cuda()
    st = torch.cuda.current_stream().cuda_stream
    c0 = torch.full((m, n), float("nan"), dtype=w.dtype, device="cuda")
    c1 = torch.full((m, n), float("nan"), dtype=w.dtype, device="cuda")
    need = lib.mlk_gemm_workspace_bytes(m, n, p1, p3)
    ws = torch.empty(max(need, 1), dtype=torch.uint8, device="cuda")
    ws[:lib.mlk_gemm_counter_bytes()].zero_()
    bp = 0 if biasd is None else biasd.data_ptr()
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    rc = lib.mlk_gemm_layout_a_noalloc(a.data_ptr(), bd.data_ptr(), c0.data_ptr(), m, n, k, kind, kind, 0, 0, alpha, bp,
                                       None, kernel_id, p1, p2, p3, st)
    assert rc == 0, lib.mlk_last_error()
    assert torch.cuda.memory_allocated() == before
    rc = lib.mlk_gemm_layout_a(a.data_ptr(), bd.data_ptr(), c1.data_ptr(), m, n, k, kind, kind, 0, 0, alpha, bp, None,
                               kernel_id, p1, p2, p3, ws.data_ptr(), ws.numel(), st)
    assert rc == 0, lib.mlk_last_error()
    torch.cuda.synchronize()
    return c0, c1


def test_noalloc_equals_workspace_variant_on_two_calls_in_a_row(mlk):
    lib = _lib()
    assert lib.mlk_gemm_noalloc_scratch_bytes() == 16 << 20
    # first call: 48 tokens, K split four ways across workgroups
    w = randn((4096, 4096), torch.float16, 0.02, 1)
    b = randn((48, 4096), torch.float16, 1.0, 2)
    c0, c1 = _both(lib, w, b, 1, 2, 4, 4)
    assert torch.equal(c0, c1)
    assert_close(c0, ogemm.linear_expected(w, b), 1e-2, 1e-2, "no-alloc, first call")
    # second call right after it: smaller matrix, fewer tokens, fewer splits, bias and alpha
    w2 = randn((1024, 2048), torch.bfloat16, 0.02, 3)
    b2 = randn((16, 2048), torch.bfloat16, 1.0, 4)
    bias = randn((1, 1024), torch.bfloat16, 1.0, 5)
    c0, c1 = _both(lib, w2, b2, 1, 1, 2, 2, alpha=0.5, bias=bias)
    assert torch.equal(c0, c1)
    assert_close(c0, ogemm.linear_expected(w2, b2, 0.5, bias), 1e-2, 1e-2, "no-alloc, second call")
    # and the first shape again: what the smaller call left in the scratch does not matter
    c0b, _ = _both(lib, w, b, 1, 2, 4, 4)
    assert_close(c0b, ogemm.linear_expected(w, b), 1e-2, 1e-2, "no-alloc, third call")


@pytest.mark.parametrize("kernel_id,p1,p2,p3,m", [(2, 1, 1, 2, 64), (3, 2, 1, 2, 160), (1, 4, 2, 1, 8), (12, 2, 4, 3, 5)])
def test_noalloc_other_kernels(mlk, kernel_id, p1, p2, p3, m):
    lib = _lib()
    w = randn((2048, 2048), torch.bfloat16, 0.02, 10 + kernel_id)
    b = randn((m, 2048), torch.bfloat16, 1.0, 20 + kernel_id)
    c0, c1 = _both(lib, w, b, kernel_id, p1, p2, p3)
    assert torch.equal(c0, c1)
    assert_close(c0, ogemm.linear_expected(w, b), 1e-2, 1e-2, "no-alloc kernel %d" % kernel_id)


def test_noalloc_rejects_what_exceeds_the_built_in_scratch(mlk):
    lib = _lib()
    assert lib.mlk_gemm_workspace_bytes(64, 28672, 1, 8) > lib.mlk_gemm_noalloc_scratch_bytes()
    x = torch.zeros(16, dtype=torch.uint8, device="cuda")     # never dereferenced: the size check comes first
    rc = lib.mlk_gemm_layout_a_noalloc(x.data_ptr(), x.data_ptr(), x.data_ptr(), 64, 28672, 8192, 1, 1, 0, 0, 1.0, None,
                                       None, 1, 1, 4, 8, torch.cuda.current_stream().cuda_stream)
    assert rc == -3 and b"16 MiB" in lib.mlk_last_error()


def test_noalloc_recorded_into_a_graph_and_replayed(mlk):
    """The call recorded into a HIP graph with a K split across workgroups (so the built-in scratch is in use),
    replayed twice with eager work and synchronizations in between: every replay must give the workspace
    variant's bits, and the replays must leave the arrival counters clean for the eager call that follows."""
    lib = _lib()
    w = randn((2048, 4096), torch.bfloat16, 0.02, 31)
    b = randn((32, 4096), torch.bfloat16, 1.0, 32)
    n, k, m = 2048, 4096, 32
    a, bd = pack_a(w).cuda(), b.cuda()
    _, want = _both(lib, w, b, 1, 2, 4, 4)
    out = torch.zeros((m, n), dtype=torch.bfloat16, device="cuda")
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    torch.cuda.synchronize()
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            rc = lib.mlk_gemm_layout_a_noalloc(a.data_ptr(), bd.data_ptr(), out.data_ptr(), m, n, k, 1, 1, 0, 0, 1.0, None,
                                               None, 1, 2, 4, 4, torch.cuda.current_stream().cuda_stream)
            assert rc == 0, lib.mlk_last_error()
        for _ in range(2):
            out.zero_()
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(out, want)
            # eager work of the program between the replays
            c0, c1 = _both(lib, w, b, 1, 2, 4, 4)
            assert torch.equal(c0, c1) and torch.equal(c0, want)
