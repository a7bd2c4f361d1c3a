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
    assert ops._gemm_guard((5, 4, 1, 2), 11008) == (5, 4, 1, 2)      # panel kernel, last round sliced
    assert ops._gemm_guard((5, 2, 4, 3), 272) == (5, 2, 4, 3)
    assert ops._gemm_guard((6, 1, 1, 1), 11008) == (1, 1, 4, 1)      # unknown kernel id
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


def test_workspace_pool_never_frees_what_it_handed_out():
    """A larger request gets a new buffer; the earlier one stays owned (a captured graph may still use its
    address).  Streams do not share buffers, repeated requests on one stream do."""
    pool = ops.WorkspacePool(1024, zero_prefix=True)
    cpu = torch.device("cpu")
    a = pool.get(cpu, 0, 1000, 64)
    ptr_a = a.data_ptr()
    assert a.numel() >= 1024 and not a[:64].any()
    assert pool.get(cpu, 0, 512, 64) is a                     # fits: same buffer
    b = pool.get(cpu, 0, 1 << 16, 64)
    assert b is not a and b.numel() >= 1 << 16 and not b[:64].any()
    assert pool.get(cpu, 0, 1000, 64) is b                    # new calls use the larger one
    c = pool.get(cpu, 7, 1000, 64)                            # another stream: its own buffer
    assert c is not a and c is not b
    owned = {t.data_ptr() for t in pool.owned()}
    assert {ptr_a, b.data_ptr(), c.data_ptr()} <= owned
    a.fill_(3)                                                # still valid memory of ours
    assert int(a[5]) == 3
    # growth is geometric, so a slowly growing series of shapes retires few buffers
    for n in range(1 << 16, 1 << 18, 4096):
        pool.get(cpu, 0, n, 64)
    assert len(pool.owned()) <= 8


def test_workspace_pool_release():
    """release() drops the retired buffers (and the live ones unless asked not to) and says how much that was;
    the next request simply gets a new buffer."""
    pool = ops.WorkspacePool(1024)
    cpu = torch.device("cpu")
    a = pool.get(cpu, 0, 1000)
    b = pool.get(cpu, 0, 1 << 16)                             # retires a
    assert pool.held_bytes() == a.numel() + b.numel()
    assert pool.release(retired_only=True) == a.numel() and pool.held_bytes() == b.numel()
    assert pool.get(cpu, 0, 100) is b                         # the live buffer is still the one in use
    assert pool.release() == b.numel() and pool.held_bytes() == 0
    c = pool.get(cpu, 0, 100)
    assert c is not b and c.numel() >= 1024


def test_moe_workspace_follows_the_plan():
    """The fp32 buffer of the K-sliced down projections is sized for the slices the plan uses (not for the most
    the kernels could take), a call of several passes covers its shorter last pass, and the query grows with the
    token count within a pass."""
    lib = _lib.load()
    E, K, H, I = 256, 8, 7168, 2048
    sizes = [lib.mlk_moe_workspace_bytes(t, E, K, H, I) for t in (1, 16, 64, 256)]
    assert sizes == sorted(sizes)
    # 256 tokens: 2048 pairs; eight slices of fp32 rows would be 470 MB, the plan uses far fewer
    slices = max(_plan(256, E, K, H, I, kind)["down_slices"] for kind in (1, 2))
    assert sizes[-1] < 2048 * H * 4 * (slices + 1) + (64 << 20)
    for n in (257, 300, 500, 511, 1024):
        last = n % 256
        need = lib.mlk_moe_workspace_bytes(n, E, K, H, I)
        assert need >= lib.mlk_moe_workspace_bytes(256, E, K, H, I)
        if last:
            assert need >= lib.mlk_moe_workspace_bytes(last, E, K, H, I)


def test_routing_buffers_are_kept_for_every_shape_and_stream():
    from muxi_native_layout_kernels_amd import moe_planC
    cpu = torch.device("cpu")
    first = moe_planC._routing_buffers(3, 2, torch.bfloat16, cpu, stream=0)
    ptr = first[0].data_ptr()
    for t in range(4, 140):                                   # many other shapes must not evict it
        moe_planC._routing_buffers(t, 2, torch.bfloat16, cpu, stream=0)
    again = moe_planC._routing_buffers(3, 2, torch.bfloat16, cpu, stream=0)
    assert again[0].data_ptr() == ptr and again[1] is first[1]
    other = moe_planC._routing_buffers(3, 2, torch.bfloat16, cpu, stream=5)
    assert other[0].data_ptr() != ptr


def _plan(T, E, K, H, I, kind):
    import ctypes
    out = (ctypes.c_int32 * 8)()
    rc = _lib.load().mlk_moe_plan(T, E, K, H, I, kind, ctypes.addressof(out))
    assert rc == 0
    return dict(path=out[0], cb=out[1], max_tasks=out[2], down_r=out[3], down_slices=out[4], down_wk=out[5],
                down_lds=out[6], static_lds=out[7])


@pytest.mark.parametrize("kind", [1, 2])
@pytest.mark.parametrize("E,K,H,I", [(256, 8, 7168, 256), (256, 8, 256, 128), (128, 8, 2048, 768), (8, 2, 4096, 14336),
                                     (64, 6, 1024, 512)])
def test_moe_plan_fits_the_workgroup_lds_for_every_token_count(E, K, H, I, kind):
    """Every pass of 1..256 tokens (also the remainder passes of longer inputs) must get a down-projection
    shape whose LDS fits the 64 KiB a workgroup gets by default, with at least four waves whenever more
    than one row group per wave was chosen."""
    for T in range(1, 257):
        p = _plan(T, E, K, H, I, kind)
        assert p["path"] in (0, 1, 2, 3, 4) and p["cb"] in (1, 2, 3, 4, 6, 8)
        if p["path"] in (1, 2):
            assert p["down_lds"] + p["static_lds"] <= 64 * 1024, (T, p)
            assert p["down_wk"] >= 1 and p["down_lds"] == p["down_wk"] * p["down_r"] * p["cb"] * 1024 + T * 16 * p["down_r"] * 4
            if p["down_r"] > 1:
                assert p["down_wk"] >= 4 and p["cb"] == 1 and p["down_slices"] == p["down_r"], (T, p)
                assert (H // 16) % p["down_r"] == 0 and (I // 32) % p["down_r"] == 0
        if p["path"] == 3:
            assert p["cb"] >= 2 and (I // 32) % (p["down_slices"] * (2 if p["cb"] > 4 else 4)) == 0
        if p["path"] == 4:          # panel kernels: output rows in tiles of 256, at least four k windows per slice
            assert kind == 2 and p["cb"] >= 5 and H % 256 == 0 and 1 <= p["down_slices"] <= 8
            assert p["down_slices"] == 1 or (I // 128) // p["down_slices"] >= 4
            assert p["down_wk"] in (1, 2)       # workgroups per CU the down kernel is built for
            if p["down_wk"] == 2:               # two per CU only where the expected grid fills them (256 CUs assumed)
                assert (H // 256) * min(E, T * K) * p["down_slices"] >= 512, (T, p)
        assert p["path"] != 0 or T == 1


def test_moe_plan_known_cases():
    # soft-FP8, 256 experts, top-8 (the DeepSeek configuration): 4 row groups per wave while the output tile
    # fits, 2 from 172 tokens up (the tile of 4 row groups would leave fewer than four waves)
    assert _plan(16, 256, 8, 7168, 256, 2)["down_r"] == 4
    assert _plan(171, 256, 8, 7168, 256, 2)["down_r"] == 4
    assert _plan(172, 256, 8, 7168, 256, 2)["down_r"] == 2
    assert _plan(244, 256, 8, 7168, 256, 2)["down_r"] == 2
    assert _plan(244, 256, 8, 7168, 256, 2)["path"] == 2
    # Mixtral shape: one token -> GeMV kernels; 16 tokens -> in-kernel alignment; 64 and 256 -> row-shared kernels
    assert _plan(1, 8, 2, 4096, 14336, 1)["path"] == 0
    assert _plan(16, 8, 2, 4096, 14336, 1)["path"] == 1
    assert _plan(64, 8, 2, 4096, 14336, 1)["path"] == 3
    assert _plan(256, 8, 2, 4096, 14336, 1)["path"] == 3
    # soft-FP8 with more than 64 tokens per pass over an expert: panel kernels, if the output rows tile in 256
    assert _plan(64, 8, 2, 4096, 14336, 2)["path"] == 3
    assert _plan(256, 8, 2, 4096, 14336, 2)["path"] == 4
    # its down projection: 16 row tiles x 8 experts x 4 K slices = two workgroups on each of 256 CUs
    mixtral = _plan(256, 8, 2, 4096, 14336, 2)
    assert (mixtral["down_slices"], mixtral["down_wk"]) == (4, 2)
    # a grid that cannot reach two per CU keeps one per CU: 4 row tiles x 8 experts x 8 slices = 256
    small = _plan(256, 8, 2, 1024, 14336, 2)
    assert small["path"] == 4 and small["down_wk"] == 1
    assert _plan(256, 8, 2, 4096 + 128, 14336, 2)["path"] == 3
    # 500 tokens run as 256 + 244: the plan of the first pass is what the query reports
    assert _plan(500, 256, 8, 7168, 256, 2) == _plan(256, 256, 8, 7168, 256, 2)
