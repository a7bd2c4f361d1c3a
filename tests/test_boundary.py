"""CPU: the C-ABI library loads, exports every function include/mlk.h declares, the ctypes table
matches the header, and the host layer rejects bad arguments before touching the GPU."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "mlk.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mlk_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    names = _declared()
    for must in ("mlk_gemv_layout_a", "mlk_gemm_layout_a", "mlk_layout_b", "mlk_re_layout_c", "mlk_fp8_weight_repack",
                 "mlk_pack_layout_a", "mlk_unpack_layout_a", "mlk_fused_routing_gate", "mlk_moe_align_tokens",
                 "mlk_fused_experts_compute", "mlk_last_error", "mlk_version"):
        assert must in names


def test_library_exports_every_declared_symbol():
    from muxi_native_layout_kernels_amd import _lib
    assert os.path.exists(_lib.LIB_PATH), "build the library first: python -m muxi_native_layout_kernels_amd.build"
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for name in _declared():
        assert hasattr(lib, name), "libmlk.so does not export %s" % name


def test_ctypes_table_covers_the_header():
    from muxi_native_layout_kernels_amd import _lib
    assert sorted(_lib.SIGNATURES) == _declared()
    header = re.sub(r"/\*.*?\*/", "", open(os.path.join(ROOT, "include", "mlk.h")).read(), flags=re.S)
    for name, (_, argtypes) in _lib.SIGNATURES.items():
        m = re.search(r"\b%s\s*\(([^;]*?)\)\s*;" % name, header, flags=re.S)
        assert m, name
        params = m.group(1).strip()
        n = 0 if params in ("void", "") else params.count(",") + 1
        assert n == len(argtypes), "%s: header has %d parameters, ctypes table %d" % (name, n, len(argtypes))


def test_version_and_error_text_without_a_gpu():
    from muxi_native_layout_kernels_amd import _lib
    lib = _lib.load()
    assert lib.mlk_version() >= 1
    # argument validation happens before any HIP call, so it can be exercised on the CPU
    rc = lib.mlk_layout_b(None, None, 8, 32, None)
    assert rc == -1 and b"multiple of 16" in lib.mlk_last_error()
    rc = lib.mlk_gemv_layout_a(None, None, None, 1, 100, 32, 1, 1, 1.0, None, None, 256, 1, 1, 1, None)
    assert rc == -1 and b"m % 16" in lib.mlk_last_error()
    rc = lib.mlk_gemm_layout_a(None, None, None, 16, 128, 128, 1, 1, 0, 0, 1.0, None, None, 1, 3, 1, 1, None, 0, None)
    assert rc == -1 and b"p1" in lib.mlk_last_error()
    rc = lib.mlk_fused_routing_gate(None, 1, 0, 4, 300, 1, 1, 2, None, 0, None, None, None)
    assert rc == -1 and b"256" in lib.mlk_last_error()
    # empty problems succeed without pointers
    assert lib.mlk_layout_b(None, None, 0, 32, None) == 0
    assert lib.mlk_gemm_workspace_bytes(16, 4096, 1, 1) == 0
    assert lib.mlk_gemm_workspace_bytes(16, 4096, 1, 4) > 4 * 256 * 1024


def test_host_layer_rejects_bad_arguments_on_cpu():
    import muxi_layout_kernels as mlk
    a = torch.zeros(8, 16, 16, 8, dtype=torch.bfloat16)
    b = torch.zeros(16, 128, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="CUDA"):
        mlk.gemm_layoutA(a, b)
    with pytest.raises(RuntimeError, match="CUDA"):
        mlk.gemv_layoutA(a, b[:1])
    with pytest.raises(RuntimeError, match="CUDA"):
        mlk.layoutB(b)
    with pytest.raises(NotImplementedError):
        mlk.gemmEx(a, b)
    with pytest.raises(NotImplementedError):
        mlk.muxi_hgemm_layoutA(a, b)


def test_reference_names_are_all_present():
    import muxi_layout_kernels as mlk
    names = ["layoutB", "reLayoutC", "gemm_layoutABC", "gemm_layoutA_linear", "gemm_layoutA", "gemm_layoutA_soft_fp8",
             "gemm_layoutAB_ContinuousC", "gemmEx", "muxi_hgemm", "muxi_hgemm_layout", "muxi_hgemm_layoutA",
             "muxi_hgemm_layoutC", "gemv_layoutA", "gemm_layoutABC_wapper", "gemm_layoutA_wapper",
             "gemm_layoutA_soft_fp8_wapper", "gemm_layoutAB_ContinuousC_wapper", "gemv_layoutA_wapper",
             "fp8_weight_repack", "routing_gate", "experts_compute", "fused_routing_gate",
             "batched_routed_activation_indexed_to_expert_block_indexed", "fused_experts_compute"]
    assert len(names) == 24
    for n in names:
        assert callable(getattr(mlk, n)), n
    import inspect
    sig = inspect.signature(mlk.gemv_layoutA_wapper)
    assert list(sig.parameters) == ["A", "B", "m", "k", "alpha", "beta", "blockDimX", "kernelId", "kernelParam1",
                                    "kernelParam2", "scale_matrix", "bias"]
    assert sig.parameters["blockDimX"].default == 256
    sig = inspect.signature(mlk.gemm_layoutA_wapper)
    assert list(sig.parameters) == ["A", "B", "m", "n", "k", "alpha", "beta", "kernelParam1", "kernelParam2",
                                    "kernelParam3", "kernelId", "bias"]
    from muxi_layout_kernels.muxi_moe_planC import fused_moe
    sig = inspect.signature(fused_moe)
    assert list(sig.parameters)[:6] == ["hidden_states", "w1", "w2", "gating_output", "topk", "renormalize"]
    assert sig.parameters["splitK"].default == 3 and sig.parameters["score_func"].default == "softmax"
    from muxi_layout_kernels.utils import fused_moe as torch_moe, scale_tensor  # noqa: F401


def test_utils_scale_tensor_matches_block_loop():
    from muxi_layout_kernels.utils import scale_tensor
    w = torch.arange(300 * 260, dtype=torch.float32).reshape(300, 260).to(torch.bfloat16)
    s = torch.arange(9, dtype=torch.float32).reshape(3, 3) + 1
    got = scale_tensor(w, s)
    want = w.clone()
    for i in range(0, 300, 128):
        for j in range(0, 260, 128):
            want[i:i + 128, j:j + 128] *= s[i // 128, j // 128]
    assert torch.equal(got, want)
