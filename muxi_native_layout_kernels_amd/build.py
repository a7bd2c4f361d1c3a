"""Build the C-ABI shared library `libmlk.so` for gfx950 with hipcc, in-tree.

`python -m muxi_native_layout_kernels_amd.build` compiles every `csrc/*.hip`
into one object each (in parallel) and links `muxi_native_layout_kernels_amd/libmlk.so`;
`python -m muxi_native_layout_kernels_amd.build mlk_moe mlk_gemv` recompiles only the named sources.
hipcc cross-compiles, so no GPU is needed to build.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OUT = os.path.join(HERE, "libmlk.so")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

FLAGS = [
    "--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17", "-Wall", "-Wno-unused-function",
    # packed fp32 VALU forms are switched off for all device code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def sources():
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


def _compile(src):
    obj = os.path.join(HERE, "build", os.path.basename(src)[:-4] + ".o")
    os.makedirs(os.path.dirname(obj), exist_ok=True)
    cmd = [HIPCC, *FLAGS, "-c", src, "-o", obj]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in proc.stderr.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, err))
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build(verbose=True, only=None):
    """Compile every source and link.  `only` (names of sources without the extension) recompiles just those and
    links them with the objects a previous full build left in build/: for work on one kernel file."""
    srcs = sources()
    todo = srcs if not only else [s for s in srcs if os.path.basename(s)[:-4] in only]
    with ThreadPoolExecutor(max_workers=min(8, max(1, len(todo)))) as pool:
        list(pool.map(_compile, todo))
    objs = [os.path.join(HERE, "build", os.path.basename(s)[:-4] + ".o") for s in srcs]
    missing = [o for o in objs if not os.path.exists(o)]
    if missing:
        raise RuntimeError("no object for %s: run a full build first" % ", ".join(missing))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", OUT]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError("link failed:\n" + proc.stderr)
    if verbose:
        print("built", OUT)
    return OUT


if __name__ == "__main__":
    build(only=set(sys.argv[1:]) or None)
