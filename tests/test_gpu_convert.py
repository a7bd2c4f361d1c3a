"""Checkpoint conversion through the HIP packing kernel: bit-equal to the oracle's packing, and the
converted file feeds `fused_moe` / `gemm_layoutA_linear` directly."""
import pytest
import torch
from safetensors.torch import save_file

from helpers import randn, fp8_codes, pack_a, assert_close
from oracle import moe as omoe, router as orouter

pytestmark = pytest.mark.gpu


def _experts(tmp_path, E, H, I, dtype, fp8):
    tensors = {}
    for e in range(E):
        for i, (proj, shape) in enumerate((("w1", (I, H)), ("w3", (I, H)), ("w2", (H, I)))):
            base = "model.layers.0.block_sparse_moe.experts.%d.%s" % (e, proj)
            if fp8:
                tensors[base + ".weight"] = fp8_codes(shape, 31 * e + i, std=1.0).view(torch.float8_e4m3fn)
                g = torch.Generator().manual_seed(977 * e + i)
                tensors[base + ".weight_scale_inv"] = torch.rand((shape[0] // 128, shape[1] // 128), generator=g) * 0.03 + 0.005
            else:
                tensors[base + ".weight"] = randn(shape, dtype, 0.02, 31 * e + i)
    tensors["model.layers.0.self_attn.o_proj.weight"] = randn((H, H), dtype, 0.02, 5)
    tensors["model.norm.weight"] = randn((H,), dtype, 1.0, 6)
    path = str(tmp_path / "in.safetensors")
    save_file(tensors, path)
    return path, tensors


@pytest.mark.parametrize("fp8", [False, True])
def test_converted_file_feeds_fused_moe(mlk, tmp_path, fp8):
    from muxi_native_layout_kernels_amd import convert as cv
    from muxi_native_layout_kernels_amd.moe_planC import fused_moe
    E, K, H, I, T, dtype = 4, 2, 256, 384, 9, torch.bfloat16
    src, tensors = _experts(tmp_path, E, H, I, dtype, fp8)
    dst = str(tmp_path / "packed.safetensors")
    cv.convert(src, dst, preset="mixtral")                   # device packing
    ck = cv.PackedCheckpoint(dst)
    pre = "model.layers.0.block_sparse_moe.experts"
    w1, w2 = ck.tensor(pre + ".w1"), ck.tensor(pre + ".w2")

    def raw(t):
        return t.view(torch.uint8) if fp8 else t
    for e in range(E):
        gate, up, down = (tensors["%s.%d.%s.weight" % (pre, e, p)] for p in ("w1", "w3", "w2"))
        assert torch.equal(raw(w1[e]).cpu(), pack_a(raw(torch.cat([gate, up], 0))))
        assert torch.equal(raw(w2[e]).cpu(), pack_a(raw(down)))
        assert torch.equal(raw(ck.logical(pre + ".w2")[e]).cpu(), raw(down))      # un-packing restores the input
    o = "model.layers.0.self_attn.o_proj.weight"
    assert torch.equal(ck.tensor(o).cpu(), pack_a(tensors[o])) and torch.equal(ck.logical(o).cpu(), tensors[o])
    assert torch.equal(ck.tensor("model.norm.weight").cpu(), tensors["model.norm.weight"])

    x = randn((T, H), dtype, 1.0, 70)
    logits = randn((T, E), dtype, 1.0, 71)
    kw = {}
    w1u = torch.stack([torch.cat([tensors["%s.%d.w1.weight" % (pre, e)], tensors["%s.%d.w3.weight" % (pre, e)]], 0)
                       for e in range(E)])
    w2u = torch.stack([tensors["%s.%d.w2.weight" % (pre, e)] for e in range(E)])
    if fp8:
        s1, s2 = ck.scale(pre + ".w1"), ck.scale(pre + ".w2")
        kw = dict(w1_scale=s1, w2_scale=s2, block_shape=[128, 128], soft_fp8=True)
        w1u = omoe.dequant_experts(w1u.view(torch.uint8).numpy(), s1.cpu().numpy())
        w2u = omoe.dequant_experts(w2u.view(torch.uint8).numpy(), s2.cpu().numpy())
    y = fused_moe(x.cuda(), w1, w2, logits.cuda(), K, True, **kw)
    ids, wts = orouter.route(logits, 0, 1, 1, K, None)
    want = omoe.moe_expected(x, w1u, w2u, ids, orouter.renormalize(wts), round_h_to=dtype)
    assert_close(y, want, 1e-2, 1e-2, "fused_moe on a converted checkpoint")


def test_converted_projection_feeds_linear(mlk, tmp_path):
    from muxi_native_layout_kernels_amd import convert as cv
    w = randn((512, 256), torch.float16, 0.05, 1)
    src, dst = str(tmp_path / "in.safetensors"), str(tmp_path / "out.safetensors")
    save_file({"proj.weight": w, "proj.bias": randn((512,), torch.float16, 1.0, 2)}, src)
    cv.convert(src, dst, preset="linear")
    ck = cv.PackedCheckpoint(dst)
    x = randn((5, 256), torch.float16, 1.0, 3)
    y = mlk.gemm_layoutA_linear(ck.tensor("proj.weight"), x.cuda(), bias=ck.tensor("proj.bias").view(1, -1))
    want = x.double().numpy() @ w.double().numpy().T + ck.tensor("proj.bias").double().cpu().numpy()
    assert_close(y, want, 1e-2, 1e-2, "linear on a converted projection")


def test_cli_converts_a_sharded_checkpoint(mlk, tmp_path, capsys):
    """The command line end to end: two input shards, the deepseek preset, device packing, the result re-opened."""
    from muxi_native_layout_kernels_amd import convert as cv
    E, H, I = 2, 256, 128
    shard_a, shard_b = {}, {}
    for e in range(E):
        for i, (proj, shape) in enumerate((("gate_proj", (I, H)), ("up_proj", (I, H)), ("down_proj", (H, I)))):
            base = "model.layers.1.mlp.experts.%d.%s" % (e, proj)
            (shard_a if e == 0 else shard_b)[base + ".weight"] = randn(shape, torch.bfloat16, 0.02, 10 * e + i)
    shard_b["model.layers.1.mlp.gate.weight"] = randn((E, H), torch.bfloat16, 0.1, 77)
    pa, pb, dst = str(tmp_path / "a.safetensors"), str(tmp_path / "b.safetensors"), str(tmp_path / "out.safetensors")
    save_file(shard_a, pa)
    save_file(shard_b, pb)
    cv.main(["--preset", "deepseek", pa, pb, dst])
    assert "wrote" in capsys.readouterr().out
    ck = cv.PackedCheckpoint(dst)
    w1 = ck.tensor("model.layers.1.mlp.experts.w1")
    assert tuple(w1.shape) == (E, 2 * I // 16, H // 8, 16, 8)
    gate1 = shard_b["model.layers.1.mlp.experts.1.gate_proj.weight"]
    up1 = shard_b["model.layers.1.mlp.experts.1.up_proj.weight"]
    assert torch.equal(w1[1].cpu(), pack_a(torch.cat([gate1, up1], 0)))
    assert ck.info("model.layers.1.mlp.gate.weight")["layout"] == "plain"
