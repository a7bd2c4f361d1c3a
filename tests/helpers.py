"""Shared helpers for the parity tests: seeded inputs, packing through the oracle."""
import numpy as np
import torch

from oracle import layouts


def gen(seed):
    g = torch.Generator()
    g.manual_seed(seed)
    return g


def randn(shape, dtype, std, seed):
    return (torch.randn(shape, generator=gen(seed), dtype=torch.float32) * std).to(dtype)


def bits(t):
    """torch 16-bit tensor -> numpy int16 view (bit patterns)."""
    return t.contiguous().view(torch.int16).numpy()


def pack_a(w):
    """CPU torch [N, K] (16-bit or uint8) -> layout-A tensor through the oracle."""
    if w.element_size() == 1:
        return torch.from_numpy(layouts.pack_layout_a(w.view(torch.uint8).numpy()))
    return torch.from_numpy(layouts.pack_layout_a(bits(w))).view(w.dtype)


def pack_b(b):
    return torch.from_numpy(layouts.pack_layout_b(bits(b))).view(b.dtype)


def fp8_codes(shape, seed, std=16.0):
    """e4m3 bytes from N(0,1)*std clipped to +-448 (finite codes only)."""
    w = (torch.randn(shape, generator=gen(seed)) * std).clamp_(-448.0, 448.0)
    return w.to(torch.float8_e4m3fn).view(torch.uint8)


def assert_close(got, want64, rtol=1e-2, atol=1e-2, what=""):
    """got: torch tensor (any float dtype, any device); want64: float64 ndarray."""
    g = got.detach().cpu().to(torch.float64).numpy()
    err = np.abs(g - want64)
    tol = atol + rtol * np.abs(want64)
    bad = err > tol
    assert not bad.any(), "%s: %d / %d outside rtol=%g atol=%g, max err %g at %s" % (
        what, bad.sum(), bad.size, rtol, atol, err.max(), np.unravel_index(err.argmax(), err.shape))
