"""Host logic of the checkpoint converter: plan, container format, error paths.

The packing step is injected (the oracle's numpy packer) so these tests run without a GPU;
tests/test_gpu_convert.py runs the same conversion through the HIP kernel.
"""
import json
import struct

import numpy as np
import pytest
import torch
from safetensors import safe_open
from safetensors.torch import load_file, save_file

from helpers import randn, fp8_codes, pack_a
from muxi_native_layout_kernels_amd import convert as cv


def oracle_pack(t):
    if t.dtype == torch.float8_e4m3fn:
        return pack_a(t.view(torch.uint8))
    return pack_a(t)


def reference_expression(w):
    """The packing loop of the reference's scripts (benchmark_and_test/test_muxi_moe.py:74-81)."""
    n, k = w.shape
    return w.view(n // 16, 16, k // 8, 8).permute(0, 2, 1, 3).contiguous()


def mixtral_like(tmp_path, E=3, H=64, I=96, dtype=torch.bfloat16, layers=2):
    tensors = {}
    seed = 10
    for L in range(layers):
        pre = "model.layers.%d" % L
        for e in range(E):
            for proj, shape in (("w1", (I, H)), ("w3", (I, H)), ("w2", (H, I))):
                tensors["%s.block_sparse_moe.experts.%d.%s.weight" % (pre, e, proj)] = randn(shape, dtype, 0.1, seed)
                seed += 1
        tensors[pre + ".block_sparse_moe.gate.weight"] = randn((E, H), dtype, 0.1, seed)
        tensors[pre + ".self_attn.q_proj.weight"] = randn((H, H), dtype, 0.1, seed + 1)
        tensors[pre + ".input_layernorm.weight"] = randn((H,), dtype, 0.1, seed + 2)
        seed += 3
    tensors["model.embed_tokens.weight"] = randn((160, H), dtype, 0.1, seed)
    path = str(tmp_path / "in.safetensors")
    save_file(tensors, path)
    return path, tensors


def test_mixtral_plan_and_bytes(tmp_path):
    src, tensors = mixtral_like(tmp_path)
    dst = str(tmp_path / "out.safetensors")
    layout = cv.convert(src, dst, preset="mixtral", pack=oracle_pack)
    out = load_file(dst)                      # any safetensors reader opens the result
    E, H, I = 3, 64, 96
    for L in range(2):
        pre = "model.layers.%d.block_sparse_moe" % L
        w1, w2 = out[pre + ".experts.w1"], out[pre + ".experts.w2"]
        assert tuple(w1.shape) == (E, 2 * I // 16, H // 8, 16, 8) and tuple(w2.shape) == (E, H // 16, I // 8, 16, 8)
        for e in range(E):
            gate = tensors["%s.experts.%d.w1.weight" % (pre, e)]
            up = tensors["%s.experts.%d.w3.weight" % (pre, e)]
            down = tensors["%s.experts.%d.w2.weight" % (pre, e)]
            assert torch.equal(w1[e], reference_expression(torch.cat([gate, up], 0)))
            assert torch.equal(w2[e], reference_expression(down))
        assert layout[pre + ".experts.w1"]["logical_shape"] == [E, 2 * I, H]
        assert layout[pre + ".experts.w1"]["sources"][:2] == [pre + ".experts.0.w1.weight", pre + ".experts.0.w3.weight"]
        # the router, the norm and the embedding table go through untouched; the attention projection is packed
        assert torch.equal(out[pre + ".gate.weight"], tensors[pre + ".gate.weight"])
        q = "model.layers.%d.self_attn.q_proj.weight" % L
        assert torch.equal(out[q], reference_expression(tensors[q])) and layout[q]["layout"] == "A"
        n = "model.layers.%d.input_layernorm.weight" % L
        assert torch.equal(out[n], tensors[n]) and layout[n]["layout"] == "plain"
    assert torch.equal(out["model.embed_tokens.weight"], tensors["model.embed_tokens.weight"])
    # nothing of the input is dropped or duplicated
    named = [s for info in layout.values() for s in info["sources"]]
    assert sorted(named) == sorted(tensors)


def test_header_is_self_describing(tmp_path):
    src, _ = mixtral_like(tmp_path, layers=1)
    dst = str(tmp_path / "out.safetensors")
    cv.convert(src, dst, preset="mixtral", pack=oracle_pack)
    with open(dst, "rb") as f:
        (n,) = struct.unpack("<Q", f.read(8))
        assert n % 8 == 0
        header = json.loads(f.read(n))
    meta = header["__metadata__"]
    assert meta["format"] == cv.FORMAT and meta["preset"] == "mixtral"
    table = json.loads(meta["mlk_layout"])
    end = 0
    for name, info in header.items():
        if name == "__metadata__":
            continue
        assert info["data_offsets"][0] == end           # dense, in table order
        end = info["data_offsets"][1]
        assert name in table
    ck = cv.PackedCheckpoint(dst, device="cpu")
    assert ck.names() == list(table)
    assert ck.info("model.layers.0.block_sparse_moe.experts.w2")["layout"] == "A"
    assert ck.scale("model.layers.0.block_sparse_moe.experts.w2") is None


def test_deepseek_fp8_scales(tmp_path):
    E, H, I = 2, 256, 128
    tensors = {}
    for e in range(E):
        for i, (proj, shape) in enumerate((("gate_proj", (I, H)), ("up_proj", (I, H)), ("down_proj", (H, I)))):
            base = "model.layers.3.mlp.experts.%d.%s" % (e, proj)
            tensors[base + ".weight"] = fp8_codes(shape, 50 + 3 * e + i).view(torch.float8_e4m3fn)
            tensors[base + ".weight_scale_inv"] = torch.rand(
                ((shape[0] + 127) // 128, (shape[1] + 127) // 128), generator=torch.Generator().manual_seed(e * 3 + i)) + 0.5
    tensors["model.layers.3.mlp.gate.weight"] = randn((E, H), torch.bfloat16, 0.1, 1)
    tensors["model.layers.3.mlp.gate.e_score_correction_bias"] = randn((E,), torch.float32, 0.1, 2)
    tensors["model.layers.3.mlp.shared_experts.up_proj.weight"] = fp8_codes((I, H), 99).view(torch.float8_e4m3fn)
    tensors["model.layers.3.mlp.shared_experts.up_proj.weight_scale_inv"] = torch.ones(1, 2)
    src, dst = str(tmp_path / "in.safetensors"), str(tmp_path / "out.safetensors")
    save_file(tensors, src)
    cv.convert(src, dst, preset="deepseek", pack=oracle_pack)
    ck = cv.PackedCheckpoint(dst, device="cpu")
    pre = "model.layers.3.mlp.experts"
    w1, s1, s2 = ck.tensor(pre + ".w1"), ck.scale(pre + ".w1"), ck.scale(pre + ".w2")
    assert w1.dtype == torch.float8_e4m3fn and tuple(w1.shape) == (E, 2 * I // 16, H // 8, 16, 8)
    assert tuple(s1.shape) == (E, 2, 2) and tuple(s2.shape) == (E, 2, 1)
    for e in range(E):
        gate = tensors["model.layers.3.mlp.experts.%d.gate_proj.weight" % e].view(torch.uint8)
        up = tensors["model.layers.3.mlp.experts.%d.up_proj.weight" % e].view(torch.uint8)
        assert torch.equal(w1[e].view(torch.uint8), reference_expression(torch.cat([gate, up], 0)))
        assert torch.equal(s1[e], torch.cat([tensors["model.layers.3.mlp.experts.%d.gate_proj.weight_scale_inv" % e],
                                             tensors["model.layers.3.mlp.experts.%d.up_proj.weight_scale_inv" % e]], 0))
        assert torch.equal(s2[e], tensors["model.layers.3.mlp.experts.%d.down_proj.weight_scale_inv" % e])
    shared = "model.layers.3.mlp.shared_experts.up_proj.weight"
    assert ck.info(shared)["layout"] == "A" and ck.info(shared)["scale"] == shared + "_scale_inv"
    assert torch.equal(ck.scale(shared), torch.ones(1, 2))
    assert ck.info("model.layers.3.mlp.gate.weight")["layout"] == "plain"


def test_linear_preset_and_keep_plain(tmp_path):
    t = {"a.weight": randn((32, 64), torch.float16, 1, 1), "b.weight": randn((24, 64), torch.float16, 1, 2),
         "c.weight": randn((32, 64), torch.float32, 1, 3), "lm_head.weight": randn((48, 32), torch.float16, 1, 4),
         "tok_embeddings.weight": randn((32, 32), torch.float16, 1, 5), "d.bias": randn((32,), torch.float16, 1, 6)}
    src, dst = str(tmp_path / "in.safetensors"), str(tmp_path / "out.safetensors")
    save_file(t, src)
    layout = cv.convert([src], dst, preset="linear", keep_plain=[r"^lm_head"], pack=oracle_pack)
    kinds = {k: v["layout"] for k, v in layout.items()}
    assert kinds == {"a.weight": "A", "b.weight": "plain", "c.weight": "plain", "lm_head.weight": "plain",
                     "tok_embeddings.weight": "plain", "d.bias": "plain"}     # 24 rows do not tile, fp32 is not a weight type
    out = load_file(dst)
    assert torch.equal(out["a.weight"], reference_expression(t["a.weight"]))
    assert torch.equal(out["b.weight"], t["b.weight"])


def test_sharded_input(tmp_path):
    a = {"x.q_proj.weight": randn((16, 32), torch.bfloat16, 1, 1)}
    b = {"y.q_proj.weight": randn((32, 32), torch.bfloat16, 1, 2)}
    pa, pb, dst = str(tmp_path / "a.safetensors"), str(tmp_path / "b.safetensors"), str(tmp_path / "o.safetensors")
    save_file(a, pa)
    save_file(b, pb)
    cv.convert([pa, pb], dst, preset="mixtral", pack=oracle_pack)
    out = load_file(dst)
    assert torch.equal(out["y.q_proj.weight"], reference_expression(b["y.q_proj.weight"]))
    save_file(a, pb)
    with pytest.raises(ValueError, match="more than one input"):
        cv.convert([pa, pb], dst, preset="mixtral", pack=oracle_pack)


def test_plan_errors(tmp_path):
    src, tensors = mixtral_like(tmp_path, layers=1)
    dst = str(tmp_path / "out.safetensors")
    broken = dict(tensors)
    del broken["model.layers.0.block_sparse_moe.experts.1.w3.weight"]
    save_file(broken, src)
    with pytest.raises(ValueError, match="up weights do not cover"):
        cv.convert(src, dst, preset="mixtral", pack=oracle_pack)
    broken = dict(tensors)
    broken["model.layers.0.block_sparse_moe.experts.2.w2.weight"] = randn((64, 80), torch.bfloat16, 1, 1)
    save_file(broken, src)
    with pytest.raises(ValueError, match="expert 2 down"):
        cv.convert(src, dst, preset="mixtral", pack=oracle_pack)
    odd = {"m.block_sparse_moe.experts.0.%s.weight" % p: randn(s, torch.bfloat16, 1, 1)
           for p, s in (("w1", (40, 64)), ("w3", (40, 64)), ("w2", (64, 40)))}
    save_file(odd, src)
    with pytest.raises(ValueError, match="do not tile"):
        cv.convert(src, dst, preset="mixtral", pack=oracle_pack)


def test_reader_rejects_other_files(tmp_path):
    p = str(tmp_path / "plain.safetensors")
    save_file({"a": torch.zeros(4)}, p)
    with pytest.raises(ValueError, match="not a mlk-layout-A"):
        cv.PackedCheckpoint(p, device="cpu")


def test_packing_needs_the_gpu(tmp_path):
    if torch.cuda.is_available():
        pytest.skip("a device is present")
    src, _ = mixtral_like(tmp_path, layers=1)
    with pytest.raises(RuntimeError, match="no HIP device"):
        cv.convert(src, str(tmp_path / "o.safetensors"), preset="mixtral")


def test_cli_dry_run(tmp_path, capsys):
    src, _ = mixtral_like(tmp_path, layers=1)
    cv.main(["--preset", "mixtral", "--dry-run", src, str(tmp_path / "never.safetensors")])
    printed = capsys.readouterr().out
    assert "model.layers.0.block_sparse_moe.experts.w1" in printed and "<- 6 tensor(s)" in printed
    assert not (tmp_path / "never.safetensors").exists()
