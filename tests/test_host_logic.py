"""CPU: host-side logic of the operator mirror that needs no GPU - argument parsing of the overloaded
`fused_experts_compute`, `fused_moe` argument errors, launch-parameter guards, workspace sizing."""
import pytest
import torch

from muxi_native_layout_kernels_amd import ops, arg_selector, _lib
from muxi_native_layout_kernels_amd.moe_planC import fused_moe


def test_gemm_guard_accepts_both_kernels_and_rejects_bad_rows():
    assert ops._gemm_guard((1, 4, 4, 1), 11008) == (1, 4, 4, 1)
    assert ops._gemm_guard((2, 2, 1, 2), 11008) == (2, 2, 1, 2)
    assert ops._gemm_guard((14, 4, 2, 1), 11008) == (14, 4, 2, 1)    # kernel 1 with an explicit ring depth
    assert ops._gemm_guard((13, 4, 2, 1), 11008) == (1, 1, 4, 1)
    assert ops._gemm_guard((4, 1, 2, 1), 11008) == (4, 1, 2, 1)      # one workgroup per CU
    assert ops._gemm_guard((18, 8, 4, 1), 28672) == (18, 8, 4, 1)    # eight row groups per wave
    assert ops._gemm_guard((3, 1, 1, 2), 11008) == (3, 1, 1, 2)      # panel kernel
    assert ops._gemm_guard((3, 2, 4, 2), 272) == (3, 2, 4, 2)        # its row groups per wave need not divide N/16
    assert ops._gemm_guard((5, 1, 1, 1), 11008) == (1, 1, 4, 1)      # unknown kernel id
    assert ops._gemm_guard((1, 3, 4, 1), 11008) == (1, 1, 4, 1)      # row groups per wave not in {1,2,4}
    assert ops._gemm_guard((1, 4, 4, 1), 16 * 6) == (1, 1, 4, 1)     # 6 row groups are not a multiple of 4
    assert ops._gemm_guard((1, 1, 5, 1), 4096) == (1, 1, 4, 1)       # waves per workgroup not a power of two


def test_default_heuristics_are_valid_launch_parameters():
    for n, k in ((16, 32), (4096, 4096), (152064, 3584)):
        block, kid, p1, p2 = arg_selector._gemv_default(n, k)
        assert kid == 1 and 64 <= block <= 1024 and block % 64 == 0 and p1 == 1 and p2 in (1, 2, 4, 6, 8)
    for n, m, k in ((128, 1, 128), (11008, 64, 4096), (4096, 16, 14336)):
        kid, p1, p2, p3 = arg_selector._gemm_default(n, m, k)
        assert ops._gemm_guard((kid, p1, p2, p3), n) == (kid, p1, p2, p3)


def test_fused_moe_argument_errors_before_any_gpu_work():
    h = torch.zeros(2, 128, dtype=torch.bfloat16)
    g = torch.zeros(2, 8, dtype=torch.bfloat16)
    w1 = torch.zeros(8, 256, 128, dtype=torch.bfloat16)
    w2 = torch.zeros(8, 128, 128, dtype=torch.bfloat16)
    with pytest.raises(ValueError, match="num_expert_group must be 1"):
        fused_moe(h, w1, w2, g, 2, True, use_grouped_topk=False, num_expert_group=2)
    with pytest.raises(ValueError, match="Unsupported scoring function"):
        fused_moe(h, w1, w2, g, 2, True, score_func="tanh")
    with pytest.raises(AssertionError, match="Number of tokens mismatch"):
        fused_moe(h, w1, w2, g[:1], 2, True)
    with pytest.raises(RuntimeError, match="CUDA"):
        fused_moe(h, w1, w2, g, 2, True)


def test_fused_experts_compute_overload_resolution_errors():
    t = torch.zeros(1)
    args = [t] * 3 + [1, 8, 2] + [t] * 8
    with pytest.raises(RuntimeError, match="too many positional"):
        ops.fused_experts_compute(*args, 2, 3, 128, 16, 128, 256, 16, None, 99)
    with pytest.raises(RuntimeError, match="unexpected argument"):
        ops.fused_experts_compute(*args, bogus=1)
    with pytest.raises(RuntimeError, match="unexpected argument"):
        ops.fused_experts_compute(*args, 2, APerWarp=4)      # given twice


def test_workspace_sizes_from_the_library():
    lib = _lib.load()
    small = lib.mlk_moe_workspace_bytes(1, 8, 2, 4096, 14336)
    big = lib.mlk_moe_workspace_bytes(256, 8, 2, 4096, 14336)
    huge = lib.mlk_moe_workspace_bytes(4096, 8, 2, 4096, 14336)
    assert 0 < small < big == huge          # tokens are processed in passes of 256
    assert lib.mlk_gemm_counter_bytes() == 65536


def test_beta_must_be_zero():
    with pytest.raises(RuntimeError, match="beta"):
        ops._check_beta(0.5)
    ops._check_beta(0)


def test_panel_kernel_default_shape():
    """Unscanned row-major shapes: the panel kernel above 64 tokens; 128-row panels while there
    are few of them, and as many K slices as keep panels x slices within the CU count."""
    from muxi_native_layout_kernels_amd import arg_selector as sel
    assert sel.panel_shape(11008, 128, 4096) == (2, 2)         # 43 panels of 256 rows -> 86 of 128 rows
    assert sel.panel_shape(11008, 256, 4096) == (2, 1)         # 86 -> 172
    assert sel.panel_shape(11008, 512, 4096) == (4, 1)         # 172 panels
    assert sel.panel_shape(8192, 128, 8192) == (2, 4)          # 32 -> 64
    assert sel.panel_shape(8192, 512, 8192) == (4, 2)          # 128 panels
    assert sel.panel_shape(28672, 128, 8192) == (4, 2)         # 112 panels
    assert sel.panel_shape(1024, 128, 1024) == (2, 2)          # 8 windows: at least four per slice
    assert sel.panel_shape(1024, 128, 384) == (2, 1)
    assert sel._gemm_default_rowmajor(11008, 512, 4096) == (3, 4, 4, 1)
    assert sel._gemm_default_rowmajor(11008, 72, 4096) == (3, 2, 4, 2)
    assert sel._gemm_default_rowmajor(11008, 64, 4096)[0] == 1      # the narrow kernels up to 64 tokens
    assert sel._gemm_default_rowmajor(11008, 512, 4096 + 64)[0] == 2  # K is no multiple of 128
    assert sel._gemm_default(11008, 512, 4096)[0] == 2              # native operands never get the panel kernel
