"""GPU parity: relayout kernels against the oracle, bit-exact, through the C ABI."""
import numpy as np
import pytest
import torch

from oracle import layouts
from helpers import bits

pytestmark = pytest.mark.gpu


def _bits16(shape, seed):
    rng = np.random.default_rng(seed)
    return torch.from_numpy(rng.integers(-32768, 32767, size=shape, dtype=np.int16, endpoint=True))


@pytest.mark.parametrize("n,k", [(16, 32), (128, 256), (4096, 4096), (11008, 4096)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_pack_unpack_layout_a(mlk, n, k, dtype):
    w = _bits16((n, k), n + k).view(dtype)
    nat = mlk.pack_layout_a(w.cuda())
    assert nat.shape == (n // 16, k // 8, 16, 8)
    assert np.array_equal(bits(nat.cpu()), layouts.pack_layout_a(bits(w)))
    assert torch.equal(mlk.unpack_layout_a(nat).view(torch.int16).cpu(), w.view(torch.int16))


def test_pack_layout_a_bytes_and_batch(mlk):
    rng = np.random.default_rng(5)
    w = torch.from_numpy(rng.integers(0, 255, size=(3, 64, 128), dtype=np.uint8, endpoint=True))
    nat = mlk.pack_layout_a(w.cuda()).cpu().numpy()
    for e in range(3):
        assert np.array_equal(nat[e], layouts.pack_layout_a(w[e].numpy()))
    assert torch.equal(mlk.unpack_layout_a(torch.from_numpy(nat).cuda()).cpu(), w)


@pytest.mark.parametrize("m,k", [(16, 32), (32, 8192), (64, 4096), (256, 4096), (2048, 256)])
def test_layout_b(mlk, m, k):
    b = _bits16((m, k), m * 7 + k).view(torch.bfloat16)
    nat = mlk.layoutB(b.cuda())
    assert nat.shape == (k // 32, m // 16, 4, 16, 8)
    assert np.array_equal(bits(nat.cpu()), layouts.pack_layout_b(bits(b)))
    # layout-C is layout-B with k := m, so reLayoutC inverts layoutB
    assert torch.equal(mlk.reLayoutC(nat).view(torch.int16).cpu(), b.view(torch.int16))


@pytest.mark.parametrize("m,n", [(16, 32), (32, 8192), (1712, 128)])  # 1712/16 = 107 > 104 token groups
def test_re_layout_c(mlk, m, n):
    c = _bits16((m, n), m + n).view(torch.float16)
    c_nat = torch.from_numpy(layouts.pack_layout_c(bits(c))).view(torch.float16)
    out = mlk.reLayoutC(c_nat.cuda())
    assert out.shape == (m, n)
    assert torch.equal(out.view(torch.int16).cpu(), c.view(torch.int16))


@pytest.mark.parametrize("shape", [(256, 256), (100, 36), (3, 512, 256), (28672, 8192)])
def test_fp8_weight_repack(mlk, shape):
    rng = np.random.default_rng(11)
    w = torch.from_numpy(rng.integers(0, 255, size=shape, dtype=np.uint8, endpoint=True))
    out = mlk.fp8_weight_repack(w.cuda())
    assert np.array_equal(out.cpu().numpy(), layouts.fp8_weight_repack(w.numpy()))
    assert torch.equal(mlk.fp8_weight_repack(out).cpu(), w)  # involution


def test_fp8_weight_repack_tails_and_unaligned_views(mlk):
    """Sizes that are not multiples of 16 bytes (the last one to three dwords take the dword kernel) and views
    whose first byte is 4 or 8 bytes into an allocation (no 16-byte alignment: the dword kernel takes it all)."""
    rng = np.random.default_rng(12)
    for nbytes in (4, 12, 20, 4 * 1027, 16 * 513 + 8):
        for lead in (0, 4, 8):
            whole = torch.from_numpy(rng.integers(0, 255, size=lead + nbytes, dtype=np.uint8, endpoint=True)).cuda()
            w = whole[lead:]
            assert w.data_ptr() % 16 == lead
            out = mlk.fp8_weight_repack(w)
            assert np.array_equal(out.cpu().numpy(), layouts.fp8_weight_repack(w.cpu().numpy())), (nbytes, lead)


def test_relayout_errors(mlk):
    with pytest.raises(RuntimeError, match="multiple of 16"):
        mlk.layoutB(torch.zeros(8, 32, dtype=torch.bfloat16, device="cuda"))
    with pytest.raises(RuntimeError, match="multiple of 32"):
        mlk.layoutB(torch.zeros(16, 48, dtype=torch.bfloat16, device="cuda"))
    with pytest.raises(RuntimeError, match="CUDA"):
        mlk.layoutB(torch.zeros(16, 32, dtype=torch.bfloat16))
    empty = mlk.layoutB(torch.zeros(0, 32, dtype=torch.bfloat16, device="cuda"))
    assert empty.shape == (1, 0, 4, 16, 8)


def test_stream_read_probe(mlk):
    """The measurement aid reads a buffer and writes nothing; it must accept any divisor grid."""
    from muxi_native_layout_kernels_amd import _lib
    lib = _lib.load()
    buf = torch.randint(0, 255, (8 << 20,), dtype=torch.uint8, device="cuda")
    keep = buf.clone()
    st = torch.cuda.current_stream().cuda_stream
    for block, wgs in ((256, 1024), (1024, 64), (64, 8192)):
        assert lib.mlk_stream_read(buf.data_ptr(), buf.numel(), block, wgs, None, st) == 0
    torch.cuda.synchronize()
    assert torch.equal(buf, keep)
    assert lib.mlk_stream_read(buf.data_ptr(), buf.numel(), 256, 1000, None, st) == -1   # 8192 tiles % 1000 != 0


def test_mfma_probe(mlk):
    """The matrix-core yardstick runs, writes nothing, and refuses null operands."""
    from muxi_native_layout_kernels_amd import _lib
    lib = _lib.load()
    a = torch.randn((64 * 1024,), device="cuda").to(torch.bfloat16)
    b = torch.randn((64 * 1024,), device="cuda").to(torch.bfloat16)
    keep = (a.clone(), b.clone())
    st = torch.cuda.current_stream().cuda_stream
    assert lib.mlk_mfma_probe(a.data_ptr(), b.data_ptr(), 10, 8, None, st) == 0
    torch.cuda.synchronize()
    assert torch.equal(a, keep[0]) and torch.equal(b, keep[1])
    assert lib.mlk_mfma_probe(None, b.data_ptr(), 10, 8, None, st) == -1
