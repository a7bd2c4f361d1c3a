"""Offline weight conversion: safetensors checkpoint -> packed layout-A file.

The reference has no converter: every script packs its weights with an ad-hoc
`view(N//16, 16, K//8, 8).permute(0, 2, 1, 3)` loop, per expert for the MoE
(benchmark_and_test/test_muxi_moe.py:73-81, gemv_benchmark.py:47-48).  This tool
does that once, on the GPU, for a whole checkpoint:

  * 2-D projection weights `[N, K]` -> layout-A `[N/16, K/8, 16, 8]`;
  * per-expert gate / up / down matrices -> the two stacked operands of
    `fused_moe`: `w1 [E, 2I/16, H/8, 16, 8]` (gate rows first, then up rows, the
    order `silu_and_mul` expects, csrc/moe_kernels/silu_and_mul.h:61-98) and
    `w2 [E, H/16, I/8, 16, 8]`;
  * soft-FP8 weights keep their bytes (layout-A is a permutation of 8-element
    granules, whatever the element size) and their fp32 block scales
    `[ceil(N/128), ceil(K/128)]` travel beside them, stacked the same way;
  * everything else is copied through unchanged.

The output is itself a safetensors file, so any safetensors reader can open it;
what makes it self-describing is the `__metadata__` entry `mlk_layout`, a JSON
object  name -> {"layout": "A" | "plain", "logical_shape": [...], "sources":
[...], "scale": name | null}.  Tensors are streamed one source matrix at a time
(read, pack on the device, write), so host memory holds one matrix, not the
checkpoint.

    python -m muxi_native_layout_kernels_amd.convert --preset mixtral in.safetensors out.safetensors
"""
import argparse
import json
import re
import struct
from collections import OrderedDict

import torch

FORMAT = "mlk-layout-A/1"

# gate / up / down names of one expert, by checkpoint family
PRESETS = {
    # model.layers.L.block_sparse_moe.experts.E.w1|w3|w2.weight  (w1 = gate, w3 = up, w2 = down)
    "mixtral": dict(
        experts=r"^(?P<prefix>.*\.block_sparse_moe)\.experts\.(?P<expert>\d+)\.(?P<proj>w1|w2|w3)\.(?P<what>weight|weight_scale_inv)$",
        roles={"w1": "gate", "w3": "up", "w2": "down"},
        linear=r"^.*\.(q_proj|k_proj|v_proj|o_proj)\.(?P<what>weight|weight_scale_inv)$"),
    # model.layers.L.mlp.experts.E.gate_proj|up_proj|down_proj.weight (+ .weight_scale_inv for fp8 blocks)
    "deepseek": dict(
        experts=r"^(?P<prefix>.*\.mlp)\.experts\.(?P<expert>\d+)\.(?P<proj>gate_proj|up_proj|down_proj)\.(?P<what>weight|weight_scale_inv)$",
        roles={"gate_proj": "gate", "up_proj": "up", "down_proj": "down"},
        linear=r"^.*\.(q_proj|q_a_proj|q_b_proj|kv_a_proj_with_mqa|kv_b_proj|k_proj|v_proj|o_proj|gate_proj|up_proj|down_proj)\.(?P<what>weight|weight_scale_inv)$"),
    # no experts: every 2-D "*.weight" that tiles is a projection, embedding tables aside
    "linear": dict(experts=None, roles={}, linear=r"^(?!.*embed).*\.(?P<what>weight|weight_scale_inv)$"),
}

_ST_DTYPE = {"F16": torch.float16, "BF16": torch.bfloat16, "F32": torch.float32, "F64": torch.float64,
             "I64": torch.int64, "I32": torch.int32, "I16": torch.int16, "I8": torch.int8, "U8": torch.uint8,
             "BOOL": torch.bool, "F8_E4M3": torch.float8_e4m3fn, "F8_E5M2": torch.float8_e5m2}
_ST_NAME = {v: k for k, v in _ST_DTYPE.items()}
_PACKABLE = ("F16", "BF16", "F8_E4M3", "U8")


def _elem_size(st_dtype):
    return torch.empty(0, dtype=_ST_DTYPE[st_dtype]).element_size()


class _Source:
    """One tensor of the input: where it lives and what it looks like (no data read)."""

    def __init__(self, path, name, st_dtype, shape):
        self.path, self.name, self.dtype, self.shape = path, name, st_dtype, tuple(shape)


def _read_header(path):
    with open(path, "rb") as f:
        (n,) = struct.unpack("<Q", f.read(8))
        return json.loads(f.read(n))


def scan_sources(paths):
    out = OrderedDict()
    for path in paths:
        for name, info in _read_header(path).items():
            if name == "__metadata__":
                continue
            if name in out:
                raise ValueError("tensor %r appears in more than one input file" % name)
            out[name] = _Source(path, name, info["dtype"], info["shape"])
    return out


class _Entry:
    """One tensor of the output: its pieces in file order.  A piece is (source, pack?)."""

    def __init__(self, name, st_dtype, shape, layout, logical_shape, pieces, scale=None):
        self.name, self.dtype, self.shape, self.layout = name, st_dtype, tuple(shape), layout
        self.logical_shape, self.pieces, self.scale = tuple(logical_shape), pieces, scale

    @property
    def nbytes(self):
        n = _elem_size(self.dtype)
        for d in self.shape:
            n *= d
        return n


def _tiles(shape):
    return len(shape) == 2 and shape[0] % 16 == 0 and shape[1] % 32 == 0


def build_plan(sources, preset="linear", keep_plain=()):
    """Decide what every output tensor is made of.  `sources`: name -> _Source.  Returns a list of _Entry."""
    rules = PRESETS[preset] if isinstance(preset, str) else preset
    experts_re = re.compile(rules["experts"]) if rules.get("experts") else None
    linear_re = re.compile(rules["linear"]) if rules.get("linear") else None
    keep_plain = [re.compile(p) for p in keep_plain]
    used = set()
    entries = []

    # ---- experts: prefix -> role -> what -> {expert id: source}
    groups = OrderedDict()
    if experts_re:
        for name, src in sources.items():
            m = experts_re.match(name)
            if not m:
                continue
            role = rules["roles"][m.group("proj")]
            groups.setdefault(m.group("prefix"), {}).setdefault(role, {}).setdefault(m.group("what"), {})[
                int(m.group("expert"))] = src
    for prefix, roles in groups.items():
        for role in ("gate", "up", "down"):
            if role not in roles or "weight" not in roles[role]:
                raise ValueError("%s: experts have no %s weights" % (prefix, role))
        n_exp = len(roles["gate"]["weight"])
        for role in ("gate", "up", "down"):
            ids = sorted(roles[role]["weight"])
            if ids != list(range(n_exp)):
                raise ValueError("%s: %s weights do not cover experts 0..%d" % (prefix, role, n_exp - 1))
        g0, d0 = roles["gate"]["weight"][0], roles["down"]["weight"][0]
        inter, hidden = g0.shape
        if d0.shape != (hidden, inter):
            raise ValueError("%s: down projection is %s, expected %s" % (prefix, d0.shape, (hidden, inter)))
        if g0.dtype not in _PACKABLE:
            raise ValueError("%s: expert weights of type %s cannot be packed" % (prefix, g0.dtype))
        if inter % 16 or hidden % 32 or hidden % 16 or inter % 32:
            raise ValueError("%s: expert matrices %dx%d do not tile (16 rows x 32 columns)" % (prefix, inter, hidden))
        w1_pieces, w2_pieces = [], []
        for e in range(n_exp):
            for role in ("gate", "up"):
                s = roles[role]["weight"][e]
                if s.shape != (inter, hidden) or s.dtype != g0.dtype:
                    raise ValueError("%s: expert %d %s is %s %s" % (prefix, e, role, s.dtype, s.shape))
                w1_pieces.append((s, True))
                used.add(s.name)
            s = roles["down"]["weight"][e]
            if s.shape != (hidden, inter) or s.dtype != g0.dtype:
                raise ValueError("%s: expert %d down is %s %s" % (prefix, e, s.dtype, s.shape))
            w2_pieces.append((s, True))
            used.add(s.name)
        scaled = "weight_scale_inv" in roles["gate"]
        s1_name = prefix + ".experts.w1_scale" if scaled else None
        s2_name = prefix + ".experts.w2_scale" if scaled else None
        entries.append(_Entry(prefix + ".experts.w1", g0.dtype, (n_exp, 2 * inter // 16, hidden // 8, 16, 8), "A",
                              (n_exp, 2 * inter, hidden), w1_pieces, s1_name))
        entries.append(_Entry(prefix + ".experts.w2", g0.dtype, (n_exp, hidden // 16, inter // 8, 16, 8), "A",
                              (n_exp, hidden, inter), w2_pieces, s2_name))
        if scaled:
            # block scales [ceil(rows/128), ceil(cols/128)]; gate rows then up rows only concatenate cleanly when
            # the gate matrix ends on a block boundary
            if inter % 128:
                raise ValueError("%s: block-scaled experts need the intermediate size to be a multiple of 128" % prefix)
            sr, sc = (inter + 127) // 128, (hidden + 127) // 128
            p1, p2 = [], []
            for e in range(n_exp):
                for role in ("gate", "up"):
                    s = roles[role]["weight_scale_inv"].get(e)
                    if s is None or s.shape != (sr, sc) or s.dtype != "F32":
                        raise ValueError("%s: expert %d %s scale missing or not fp32 %s" % (prefix, e, role, (sr, sc)))
                    p1.append((s, False))
                    used.add(s.name)
                s = roles["down"]["weight_scale_inv"].get(e)
                if s is None or s.shape != (sc, sr) or s.dtype != "F32":
                    raise ValueError("%s: expert %d down scale missing or not fp32 %s" % (prefix, e, (sc, sr)))
                p2.append((s, False))
                used.add(s.name)
            entries.append(_Entry(s1_name, "F32", (n_exp, 2 * sr, sc), "plain", (n_exp, 2 * sr, sc), p1))
            entries.append(_Entry(s2_name, "F32", (n_exp, sc, sr), "plain", (n_exp, sc, sr), p2))

    # ---- projections and the rest, in input order
    for name, src in sources.items():
        if name in used:
            continue
        m = linear_re.match(name) if linear_re else None
        plain = any(p.match(name) for p in keep_plain)
        if m and not plain and m.group("what") == "weight" and src.dtype in _PACKABLE and _tiles(src.shape):
            n, k = src.shape
            scale = name + "_scale_inv" if (name + "_scale_inv") in sources else None
            entries.append(_Entry(name, src.dtype, (n // 16, k // 8, 16, 8), "A", (n, k), [(src, True)], scale))
        else:
            entries.append(_Entry(name, src.dtype, src.shape, "plain", src.shape, [(src, False)]))
    return entries


def _device_pack(t):
    """[N, K] host tensor -> layout-A bytes, through the HIP kernel."""
    from . import ops
    if not torch.cuda.is_available():
        raise RuntimeError("convert: packing runs on the GPU and no HIP device is visible")
    dev = t.cuda()
    if dev.dtype in (torch.float8_e4m3fn, torch.float8_e5m2):
        dev = dev.view(torch.uint8)
    return ops.pack_layout_a(dev).cpu()


def _raw_bytes(t):
    t = t.contiguous()
    return t.view(torch.uint8).numpy().tobytes() if t.numel() else b""


def write_packed(entries, dst_path, pack=None, extra_metadata=None):
    """Stream `entries` into a safetensors file at `dst_path`.  `pack`: [N, K] host tensor -> packed host tensor."""
    from safetensors import safe_open
    pack = pack or _device_pack
    header = OrderedDict()
    layout = OrderedDict()
    offset = 0
    for e in entries:
        header[e.name] = {"dtype": e.dtype, "shape": list(e.shape), "data_offsets": [offset, offset + e.nbytes]}
        layout[e.name] = {"layout": e.layout, "logical_shape": list(e.logical_shape),
                          "sources": [s.name for s, _ in e.pieces], "scale": e.scale}
        offset += e.nbytes
    meta = {"format": FORMAT, "mlk_layout": json.dumps(layout)}
    meta.update(extra_metadata or {})
    header["__metadata__"] = meta
    blob = json.dumps(header, separators=(",", ":")).encode()
    blob += b" " * (-len(blob) % 8)
    handles = {}
    try:
        with open(dst_path, "wb") as out:
            out.write(struct.pack("<Q", len(blob)))
            out.write(blob)
            for e in entries:
                written = 0
                for src, do_pack in e.pieces:
                    f = handles.get(src.path)
                    if f is None:
                        f = handles[src.path] = safe_open(src.path, framework="pt", device="cpu")
                    t = f.get_tensor(src.name)
                    if do_pack:
                        t = pack(t)
                    data = _raw_bytes(t)
                    out.write(data)
                    written += len(data)
                if written != e.nbytes:
                    raise RuntimeError("%s: wrote %d bytes, header says %d" % (e.name, written, e.nbytes))
    finally:
        handles.clear()
    return layout


def convert(src_paths, dst_path, preset="linear", keep_plain=(), pack=None):
    """Convert the checkpoint made of `src_paths` into one packed file.  Returns the layout table written."""
    if isinstance(src_paths, str):
        src_paths = [src_paths]
    entries = build_plan(scan_sources(src_paths), preset, keep_plain)
    return write_packed(entries, dst_path, pack, {"preset": preset if isinstance(preset, str) else "custom"})


class PackedCheckpoint:
    """Reader of a converted file.  `tensor(name)` returns the tensor as stored (layout-A tensors come back
    5-D / 4-D, ready for `gemm_layoutA*` / `gemv_layoutA` / `fused_moe`); `scale(name)` its block scales or None."""

    def __init__(self, path, device="cuda"):
        from safetensors import safe_open
        self.path, self.device = path, device
        self._f = safe_open(path, framework="pt", device="cpu")
        meta = self._f.metadata() or {}
        if meta.get("format") != FORMAT:
            raise ValueError("%s is not a %s file (format = %r)" % (path, FORMAT, meta.get("format")))
        self.layout = json.loads(meta["mlk_layout"])
        names = set(self._f.keys())
        for name, info in self.layout.items():
            if name not in names:
                raise ValueError("%s: layout table names %r, which the file does not hold" % (path, name))
            if info["scale"] is not None and info["scale"] not in names:
                raise ValueError("%s: %r refers to missing scale tensor %r" % (path, name, info["scale"]))

    def names(self):
        return list(self.layout)

    def info(self, name):
        return self.layout[name]

    def tensor(self, name):
        return self._f.get_tensor(name).to(self.device)

    def scale(self, name):
        s = self.layout[name]["scale"]
        return None if s is None else self.tensor(s)

    def logical(self, name):
        """The tensor in its original row-major shape (un-packed on the device)."""
        from . import ops
        t = self.tensor(name)
        if self.layout[name]["layout"] != "A":
            return t
        if t.dtype in (torch.float8_e4m3fn, torch.float8_e5m2):
            return ops.unpack_layout_a(t.view(torch.uint8)).view(t.dtype)
        return ops.unpack_layout_a(t)


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--preset", choices=sorted(PRESETS), default="linear")
    ap.add_argument("--keep-plain", action="append", default=[],
                    help="regular expression of tensor names to copy through un-packed (repeatable)")
    ap.add_argument("--dry-run", action="store_true", help="print the plan and write nothing")
    ap.add_argument("inputs", nargs="+", help="input .safetensors shards, then the output file")
    args = ap.parse_args(argv)
    if len(args.inputs) < 2:
        ap.error("need at least one input and the output file")
    *srcs, dst = args.inputs
    entries = build_plan(scan_sources(srcs), args.preset, args.keep_plain)
    for e in entries:
        print("%-7s %-8s %-28s %s  <- %d tensor(s)" % (e.layout, e.dtype, list(e.shape), e.name, len(e.pieces)))
    if not args.dry_run:
        write_packed(entries, dst, None, {"preset": args.preset})
        print("wrote", dst)


if __name__ == "__main__":
    main()
