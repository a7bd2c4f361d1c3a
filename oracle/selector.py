"""csv dispatch tables, restated on the CPU.

TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).

Parse rules of csrc/arg_selector.cu:14-50 (GEMM tables, 7 integer cells,
key = first three) and :170-205 (GeMV tables, 6 cells, key = first two): the
first line is a header and is skipped, cells are split on ',', every cell is
converted with an integer parse, a row with the wrong number of cells is
reported and skipped, and a later row with the same key replaces an earlier one.
A missing key falls back to (1,1,1,1) for GEMM (:63-72) and (256,1,1,1) for GeMV
(:207-224).  GeMV guard rails after the lookup: csrc/gemv_layout_a.cu:132-143.

Pinned by known-answer rows taken from the reference's shipped tables (kept as a
small data fixture under tests/golden/).
"""

GEMM_FALLBACK = (1, 1, 1, 1)
GEMV_FALLBACK = (256, 1, 1, 1)


def parse_table(text, key_cells):
    table = {}
    lines = text.splitlines()
    for line in lines[1:]:
        if line == "":
            continue
        cells = [int(c) for c in line.split(",")]
        if len(cells) != key_cells + 4:
            continue
        table[tuple(cells[:key_cells])] = tuple(cells[key_cells:])
    return table


def lookup(table, key, fallback):
    return table.get(tuple(key), fallback)


def gemv_guard(args, n_rows, k):
    block, kid, p1, p2 = args
    if kid == 1 and n_rows % (16 * p1) != 0:
        return GEMV_FALLBACK
    if kid == 2 and k > 8192:
        return GEMV_FALLBACK
    return args
