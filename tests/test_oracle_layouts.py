"""CPU: pins the oracle's layout / repack / soft-FP8 statements."""
import numpy as np
import pytest
import torch

from oracle import layouts, softfp8


def _rand_bits(shape, seed, dtype=np.uint16):
    rng = np.random.default_rng(seed)
    return rng.integers(0, np.iinfo(dtype).max, size=shape, dtype=dtype, endpoint=True)


@pytest.mark.parametrize("n,k", [(16, 8), (32, 64), (48, 96)])
def test_layout_a_closed_form_equals_index_loop(n, k):
    w = _rand_bits((n, k), 1)
    assert np.array_equal(layouts.pack_layout_a(w), layouts.pack_layout_a_loop(w))
    assert np.array_equal(layouts.unpack_layout_a(layouts.pack_layout_a(w)), w)


def test_layout_a_matches_torch_view_permute():
    # the expression the reference's scripts use (gemv_benchmark.py:47-48)
    w = torch.arange(64 * 64, dtype=torch.int16).reshape(64, 64)
    ref = w.view(64 // 16, 16, 64 // 8, 8).permute(0, 2, 1, 3).contiguous().numpy()
    assert np.array_equal(layouts.pack_layout_a(w.numpy()), ref)


@pytest.mark.parametrize("m,k", [(16, 32), (32, 64), (48, 128)])
def test_layout_b_closed_form_equals_index_loop(m, k):
    b = _rand_bits((m, k), 2)
    assert np.array_equal(layouts.pack_layout_b(b), layouts.pack_layout_b_loop(b))
    assert np.array_equal(layouts.unpack_layout_b(layouts.pack_layout_b(b)), b)


def test_layout_b_and_c_match_torch_view_permute():
    # transposeB_bench.py:10-11 and gemm_benchmark.py:74-76
    n, k = 32, 64
    b = torch.arange(n * k, dtype=torch.int16).reshape(n, k)
    ref = b.view(n // 16, 16, k // 32, 4, 8).permute(2, 0, 3, 1, 4).contiguous()
    assert np.array_equal(layouts.pack_layout_b(b.numpy()), ref.numpy())
    back = ref.view(k // 32, n // 16, 4, 16, 8).permute(1, 3, 0, 2, 4).contiguous().view(n, k)
    assert np.array_equal(layouts.unpack_layout_c(ref.numpy()), back.numpy())


def test_layout_roundtrip_keeps_nan_payloads():
    w = np.full((16, 32), 0x7FC1, dtype=np.uint16)
    w[3, 5] = 0xFFFF
    assert np.array_equal(layouts.unpack_layout_a(layouts.pack_layout_a(w)), w)
    assert np.array_equal(layouts.unpack_layout_c(layouts.pack_layout_b(w)), w)


def test_fp8_repack_closed_form_loop_involution():
    w = np.arange(256 * 256, dtype=np.uint32).astype(np.uint8).reshape(256, 256)
    r = layouts.fp8_weight_repack(w)
    assert np.array_equal(r, layouts.fp8_weight_repack_loop(w))
    assert np.array_equal(layouts.fp8_weight_repack(r), w)
    assert list(r.reshape(-1)[:8]) == [0, 2, 1, 3, 4, 6, 5, 7]


def test_softfp8_table_matches_library_decode():
    codes = np.arange(256, dtype=np.uint8)
    lib = torch.from_numpy(codes).view(torch.float8_e4m3fn).float().numpy()
    dec = softfp8.decode_e4m3(codes)
    for c in range(256):
        if c in (0x7F, 0xFF):
            assert dec[c] == (480.0 if c == 0x7F else -480.0)
        else:
            assert dec[c] == lib[c] and np.signbit(dec[c]) == np.signbit(lib[c])


def test_softfp8_scaled_truncates():
    codes = np.arange(256, dtype=np.uint8)
    for scale in (1.0, 0.5, 0.0123, 3.7):
        got = softfp8.dequant_bf16_bits(codes, np.float32(scale))
        val = softfp8.decode_e4m3(codes).astype(np.float32) * np.float32(scale)
        want = (val.astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
        assert np.array_equal(got, want)
        # truncation never rounds away from zero
        assert np.all(np.abs(softfp8.bf16_bits_to_f32(got)) <= np.abs(val))
    # scale 1: every e4m3 value is a bf16 value
    assert np.array_equal(softfp8.bf16_bits_to_f32(softfp8.dequant_bf16_bits(codes, np.float32(1.0))),
                          softfp8.decode_e4m3(codes))


def test_expand_block_scale():
    s = np.arange(6, dtype=np.float32).reshape(2, 3)
    full = softfp8.expand_block_scale(s, 200, 300)
    assert full.shape == (200, 300)
    assert full[127, 127] == 0 and full[128, 0] == 3 and full[199, 299] == 5 and full[0, 256] == 2
