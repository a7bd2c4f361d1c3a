"""csv-driven launch-parameter dispatch for gfx950.

Host-side mirror of the reference's seven selectors (csrc/arg_selector.cu:14-540,
csrc/arg_selector.h:9-125).  Same file names, same column layout and the same
parse rules: the first line is a header, cells are integers separated by ',',
rows with the wrong number of cells are reported and skipped, a later row with
the same key replaces an earlier one.  A shape that is not in its table gets a
one-time warning and a fallback that is remembered for the rest of the process
(arg_selector.cu:63-72, :207-224).  The tables are immutable after loading; the
miss memo is kept under a lock.  Where the reference falls back to fixed
arguments, a GEMM shape whose table holds the same weight shape at other token
counts borrows the row of the nearest scanned count in the same kernel range
(up to 64 tokens, or above), and only a weight shape that was never scanned
gets arguments from a rule of thumb.

What the columns select on gfx950 (the rows are produced by the scripts in
`kernel_args_scan/`):

  GeMV tables   m,k -> BLOCK_DIM_X, KernelId, KernelParam1, KernelParam2
                BLOCK_DIM_X  threads per workgroup (64..1024)
                KernelId     1 = streaming GeMV, one workgroup per KernelParam1 row groups
                             2 = the same stream from KernelParam1 workgroups per CU, each walking a
                                 contiguous range of row groups in one uninterrupted stream per wave
                             3 = kernel 2 with the products of soft-FP8 weights on the matrix cores
                KernelParam1 row groups (16 rows) per workgroup (kernel 1) / workgroups per CU (2, 3)
                KernelParam2 16-byte loads kept in flight per wave
  GEMM tables   m,n,k -> kernelId, kernelParam1, kernelParam2, kernelParam3
                kernelId     1 = wave-tiled MFMA kernel (waves of a workgroup split K)
                             2 = row-shared tile kernel (4 waves share the activations of
                                 each k window through LDS; kernelParam2 is not used)
                             3 = panel kernel for more than 64 tokens (128 or 256 weight
                                 rows x 128 tokens per workgroup, 32x32x16 MFMA, any number of
                                 tokens in one launch; row-major operands, K % 128 == 0;
                                 kernelParam1 = 2: panels of 128 rows, 4: of 256 rows,
                                 kernelParam2 = 1: panels of 128 tokens, 2: of 256 tokens,
                                 other values: chosen from the shape)
                             4 = kernel 1 with one workgroup per CU and the row groups dealt out
                                 evenly, two to four per workgroup (16-bit weights; up to eight with soft-FP8 weights; soft-FP8 weights or
                                 layout-B activations from 17 tokens on with kernelParam2 = 4 or 8; row-major
                                 operands, up to 64 tokens, N/16 above the CU count; from 33 tokens on,
                                 and from 17 tokens on with kernelParam2 = 8, the activations of a k
                                 window are shared through LDS by up to eight waves; kernelParam1
                                 and kernelParam3 are not used; otherwise the same as 1)
                             5 = kernel 3 with the K slices (kernelParam3) applied only to the panels left
                                 over after whole rounds of one panel per CU
                             12, 14, 16, 18 = kernel 1 with 2, 4, 6, 8 k tiles in flight per
                                 wave (up to 16 tokens, row-major activations and output;
                                 otherwise the same as 1)
                kernelParam1 row groups per wave (1, 2, 4, 8)
                kernelParam2 waves per workgroup splitting K (1..16)
                kernelParam3 K splits across workgroups
"""
import os
import sys
import threading

_HERE = os.path.dirname(os.path.abspath(__file__))

GEMM_FALLBACK = (1, 1, 1, 1)
GEMV_FALLBACK = (256, 1, 1, 1)


class _Selector:
    def __init__(self, filename, key_cells, fallback, label, heuristic=None, neighbours=False):
        self.filename = filename
        self.key_cells = key_cells
        self.fallback = fallback
        self.label = label
        self.heuristic = heuristic
        self.neighbours = neighbours        # GEMM tables: a miss may borrow the row of a nearby token count
        self._by_shape = None
        self._table = None
        self._memo = {}
        self._lock = threading.Lock()

    def path(self):
        return os.path.join(_HERE, self.filename)

    def _load(self):
        table = {}
        try:
            with open(self.path(), "r") as f:
                lines = f.read().splitlines()
        except OSError:
            sys.stderr.write("Error opening file: %s\n" % self.path())
            sys.stderr.write("All %s shape will fallback to default args\n" % self.label)
            lines = []
        for line in lines[1:]:
            if not line.strip():
                continue
            try:
                cells = [int(c) for c in line.split(",")]
            except ValueError:
                sys.stderr.write("Invalid line: %s\n" % line)
                continue
            if len(cells) != self.key_cells + 4:
                sys.stderr.write("Invalid line: %s\n" % line)
                continue
            table[tuple(cells[:self.key_cells])] = tuple(cells[self.key_cells:])
        return table

    def table(self):
        if self._table is None:
            with self._lock:
                if self._table is None:
                    self._table = self._load()
        return self._table

    def _neighbour(self, key):
        """Row of the same weight shape (rows, K) at the nearest scanned token count, or None.  The tables hold a
        few token counts per shape; the launch parameters change slowly between them, and every kernel takes any
        token count of its range (up to 64 tokens the narrow kernels, above 64 the panel kernel), so the next
        scanned count upwards in the same range is borrowed, else the next one downwards."""
        if self._by_shape is None:
            by_shape = {}
            for (rows, tokens, k), args in self.table().items():
                by_shape.setdefault((rows, k), []).append((tokens, args))
            for rows_of in by_shape.values():
                rows_of.sort()
            self._by_shape = by_shape
        rows, tokens, k = key
        narrow = tokens <= 64
        same = [(t, a) for t, a in self._by_shape.get((rows, k), ()) if (t <= 64) == narrow]
        above = [(t, a) for t, a in same if t >= tokens]
        if above:
            return above[0]
        return same[-1] if same else None

    def get_args(self, key):
        key = tuple(int(v) for v in key)
        hit = self.table().get(key)
        if hit is not None:
            return hit
        with self._lock:
            memo = self._memo.get(key)
            if memo is not None:
                return memo
            near = self._neighbour(key) if self.neighbours else None
            if near is not None:
                args = near[1]
                sys.stderr.write(" Warning: No matching arguments found for %s shape: %s. Borrowing the args of %d "
                                 "tokens: %s\n" % (self.label, ", ".join(str(v) for v in key), near[0],
                                                   ",".join(str(v) for v in args)))
                self._memo[key] = args
                return args
            args = self.heuristic(*key) if self.heuristic is not None else self.fallback
            sys.stderr.write(" Warning: No matching arguments found for %s shape: %s. Fallback args to %s\n" %
                             (self.label, ", ".join(str(v) for v in key), ",".join(str(v) for v in args)))
            self._memo[key] = args
            return args


def _gemv_default(n, k):
    """Fallback for a GeMV shape that was never scanned: one row group per
    workgroup, enough waves that the grid holds >= 8 waves per CU, 4 loads in flight."""
    groups = max(1, n // 16)
    waves = 4
    while waves < 16 and groups * waves < 256 * 8:
        waves *= 2
    return (waves * 64, 1, 1, 4)


def _gemm_default(n, m, k):
    """Fallback for a GEMM shape that was never scanned."""
    groups = max(1, n // 16)
    if m > 64 and groups % 4 == 0 and (k // 32) % 2 == 0:
        # more than 64 tokens: the row-shared kernel takes 128 tokens per pass over the weights
        return (2, 2 if groups % 8 == 0 else 1, 1, 2 if (k // 32) % 4 == 0 else 1)
    r = 1 if m > 32 else 2
    if groups % r:
        r = 1
    waves = 1
    while waves < 16 and (groups // r) * waves < 256 * 8:
        waves *= 2
    return (1, r, waves, 1)


def panel_shape(n, m, k, cus=256):
    """(row groups per wave, K slices) for kernel id 3.  A panel is 256 weight rows x 128 tokens; while there are
    at most three eighths as many of them as CUs, 128-row panels (two row groups per wave) put twice as many CUs
    to work.  K slices: as many (4, 2 or 1) as keep every workgroup on a CU of its own, with at least four
    128-wide k windows per slice."""
    panels = ((n + 255) // 256) * ((m + 127) // 128)
    rg = 4
    if panels * 8 <= cus * 3:
        rg, panels = 2, ((n + 127) // 128) * ((m + 127) // 128)
    for sk in (4, 2):
        if panels * sk <= cus and (k // 128) // sk >= 4:
            return rg, sk
    return rg, 1


def _gemm_default_rowmajor(n, m, k):
    """Row-major activations and output: above 64 tokens the panel kernel (id 3) takes over (measured ahead of
    the row-shared kernel from 72 tokens on; panel width left to the library)."""
    if m > 64 and k % 128 == 0:
        rg, sk = panel_shape(n, m, k)
        return (3, rg, 4, sk)
    return _gemm_default(n, m, k)


_SELECTORS = {
    # reference getters: csrc/arg_selector.cu:84-87 (layout gemm), :158-161 (continuous C),
    # :236-239 (gemv fp16), :312-315 (layoutA gemm), :389-392 (layoutA soft fp8), :464-467 (soft-fp8 gemv),
    # :537-540 (bf16 gemv)
    "layout_gemm": _Selector("layout_gemm_dispatch_arg.csv", 3, GEMM_FALLBACK, "layout GEMM", _gemm_default, True),
    "continuous_gemm": _Selector("continuous_gemm_dispatch_arg.csv", 3, GEMM_FALLBACK, "ContinuousC GEMM",
                                 _gemm_default, True),
    "layoutA_gemm": _Selector("layoutA_gemm_dispatch_arg.csv", 3, GEMM_FALLBACK, "layoutA GEMM",
                              _gemm_default_rowmajor, True),
    "layoutA_soft_fp8_gemm": _Selector("layoutA_Soft_Fp8_gemm_dispatch_arg.csv", 3, GEMM_FALLBACK,
                                       "layoutA soft-FP8 GEMM", _gemm_default_rowmajor, True),
    "gemv_fp16": _Selector("layout_gemv_dispatch_arg.csv", 2, GEMV_FALLBACK, "GEMV", _gemv_default),
    "gemv_bf16": _Selector("layout_gemv_bf16_dispatch_arg.csv", 2, GEMV_FALLBACK, "bf16 GEMV", _gemv_default),
    "gemv_soft_fp8": _Selector("layout_gemv_soft_fp8_dispatch_arg.csv", 2, GEMV_FALLBACK, "soft-FP8 GEMV",
                               _gemv_default),
}


def selector(name):
    return _SELECTORS[name]


def gemv_guard(args, n, k):
    """Guard rails applied after the GeMV lookup (csrc/gemv_layout_a.cu:132-143): a row
    that asks for more row groups per workgroup than divide N/16, or more than
    the wave count allows, is replaced by the plain configuration."""
    block, kid, p1, p2 = args
    if block % 64 or not 64 <= block <= 1024 or p2 not in (1, 2, 4, 6, 8):
        return (256, 1, 1, 4)
    if kid == 1 and p1 >= 1 and (n // 16) % p1 == 0 and (block // 64) % p1 == 0:
        return args
    if kid in (2, 3) and 1 <= p1 <= 16 and p2 != 1:       # p1 = workgroups per CU
        return args
    return (256, 1, 1, 4)


def parse_table_text(text, key_cells):
    """Parse csv text with the selector's rules (used by the scan scripts and the tests)."""
    table = {}
    for line in text.splitlines()[1:]:
        if not line.strip():
            continue
        try:
            cells = [int(c) for c in line.split(",")]
        except ValueError:
            continue
        if len(cells) != key_cells + 4:
            continue
        table[tuple(cells[:key_cells])] = tuple(cells[key_cells:])
    return table
