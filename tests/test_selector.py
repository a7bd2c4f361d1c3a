"""CPU: csv dispatch tables - parse rules, fallbacks, guard rails, shipped tables."""
import os

import pytest

from oracle import selector as osel
from muxi_native_layout_kernels_amd import arg_selector

GOLD = os.path.join(os.path.dirname(__file__), "golden")


def test_excerpt_known_answers_oracle_and_product_agree():
    text = open(os.path.join(GOLD, "gemv_bf16_excerpt.csv")).read()
    want = osel.parse_table(text, 2)
    got = arg_selector.parse_table_text(text, 2)
    assert got == want
    # three rows share the key (4096, 4096); the last one wins (reference table line 45)
    assert got[(4096, 4096)] == (256, 1, 1, 3)
    # the 5-cell row is skipped
    assert (1024, 4096) not in got
    assert got[(19008, 5120)] == (256, 1, 1, 8)


def _golden_rows():
    """(table file, line number in the reference's table, cells) of every known-answer row."""
    out = []
    for line in open(os.path.join(GOLD, "selector_rows.csv")).read().splitlines():
        if line.startswith("#"):
            continue
        fname, lineno, row = line.split(",", 2)
        out.append((fname, int(lineno), [int(c) for c in row.strip('"').split(",")]))
    return out


def test_known_answer_rows_through_a_multi_row_table(tmp_path):
    """The reference-held rows are looked up through whole tables built around them: a header, decoy rows
    with other keys before and after, an earlier duplicate of the key with other values (the later row
    must win) and a row with too few cells (skipped).  Oracle and product must both return the
    reference's answer."""
    for nkey, fallback in ((2, arg_selector.GEMV_FALLBACK), (3, arg_selector.GEMM_FALLBACK)):
        rows = [cells for fname, _, cells in _golden_rows() if len(cells) == nkey + 4]
        assert rows
        lines = ["header"]
        for i, cells in enumerate(rows):
            key, val = cells[:nkey], cells[nkey:]
            decoy_key = [key[0] + 16 * (i + 1)] + key[1:]
            lines.append(",".join(map(str, decoy_key + [7, 7, 7, 7])))
            lines.append(",".join(map(str, key + [v + 1 for v in val])))          # earlier duplicate, loses
            lines.append(",".join(map(str, key[:nkey] + val[:2])))                 # wrong cell count, skipped
            lines.append(",".join(map(str, cells)))                                # the reference's row, wins
            lines.append(",".join(map(str, [key[0] + 32 * (i + 1)] + key[1:] + [9, 9, 9, 9])))
        text = "\n".join(lines) + "\n"
        want_table = osel.parse_table(text, nkey)
        path = tmp_path / ("table%d.csv" % nkey)
        path.write_text(text)
        sel = arg_selector._Selector(str(path), nkey, fallback, "golden")
        sel.path = lambda path=path: str(path)
        for cells in rows:
            key, val = tuple(cells[:nkey]), tuple(cells[nkey:])
            assert osel.lookup(want_table, key, fallback) == val
            assert sel.get_args(key) == val
        miss = tuple([5] * nkey)
        assert osel.lookup(want_table, miss, fallback) == fallback


def test_fallbacks_and_guards_oracle():
    assert osel.lookup({}, (1, 2, 3), osel.GEMM_FALLBACK) == (1, 1, 1, 1)
    assert osel.lookup({}, (1, 2), osel.GEMV_FALLBACK) == (256, 1, 1, 1)
    assert osel.gemv_guard((256, 1, 3, 1), 4096, 4096) == (256, 1, 1, 1)   # 256 row groups % 3 != 0
    assert osel.gemv_guard((256, 2, 16, 0), 4096, 16384) == (256, 1, 1, 1)  # kernel 2 needs k <= 8192
    assert osel.gemv_guard((128, 1, 2, 1), 4096, 4096) == (128, 1, 2, 1)


def test_product_selector_miss_is_memoised_and_warns_once(capsys, tmp_path, monkeypatch):
    sel = arg_selector._Selector("does_not_exist.csv", 3, arg_selector.GEMM_FALLBACK, "test GEMM")
    a = sel.get_args((128, 16, 128))
    b = sel.get_args((128, 16, 128))
    err = capsys.readouterr().err
    assert a == b == (1, 1, 1, 1)
    assert err.count("No matching arguments") == 1
    assert "Error opening file" in err


def test_product_selector_reads_table(tmp_path):
    p = tmp_path / "t.csv"
    p.write_text("m,n,k,kernelId,kernelParam1,kernelParam2,kernelParam3\n128,16,256,1,2,4,1\nbad,row\n128,16,256,1,4,8,1\n")
    sel = arg_selector._Selector(str(p), 3, arg_selector.GEMM_FALLBACK, "tmp")
    sel.path = lambda: str(p)
    assert sel.get_args((128, 16, 256)) == (1, 4, 8, 1)


def test_gemm_miss_borrows_the_nearest_scanned_token_count(capsys, tmp_path):
    """A GEMM key whose weight shape is in the table at other token counts takes the next scanned count upwards in
    the same kernel range (up to 64 tokens / above), else the next one downwards; an unknown weight shape takes the
    rule of thumb.  GeMV selectors never borrow."""
    p = tmp_path / "t.csv"
    p.write_text("m,n,k,kernelId,kernelParam1,kernelParam2,kernelParam3\n"
                 "4096,8,4096,14,1,4,1\n4096,32,4096,4,1,8,1\n4096,64,4096,2,2,1,1\n"
                 "4096,256,4096,3,4,1,2\n4096,1024,4096,3,4,2,1\n8192,16,1024,1,2,2,1\n")
    sel = arg_selector._Selector(str(p), 3, arg_selector.GEMM_FALLBACK, "tmp", lambda n, m, k: (9, 9, 9, 9), True)
    sel.path = lambda: str(p)
    assert sel.get_args((4096, 32, 4096)) == (4, 1, 8, 1)        # a hit stays a hit
    assert sel.get_args((4096, 1, 4096)) == (14, 1, 4, 1)        # up to the 8-token row
    assert sel.get_args((4096, 24, 4096)) == (4, 1, 8, 1)
    assert sel.get_args((4096, 33, 4096)) == (2, 2, 1, 1)
    assert sel.get_args((4096, 100, 4096)) == (3, 4, 1, 2)       # above 64 tokens only the rows above 64 count
    assert sel.get_args((4096, 512, 4096)) == (3, 4, 2, 1)
    assert sel.get_args((4096, 4096, 4096)) == (3, 4, 2, 1)      # nothing above: the largest scanned count
    assert sel.get_args((8192, 48, 1024)) == (1, 2, 2, 1)        # nothing above in the range: downwards
    assert sel.get_args((8192, 128, 1024)) == (9, 9, 9, 9)       # no row above 64 tokens for this shape
    assert sel.get_args((1024, 16, 1024)) == (9, 9, 9, 9)        # weight shape never scanned
    err = capsys.readouterr().err
    assert err.count("Borrowing the args of") == 7 and err.count("Fallback args to") == 2
    plain = arg_selector._Selector(str(p), 3, arg_selector.GEMM_FALLBACK, "tmp")
    plain.path = lambda: str(p)
    assert plain.get_args((4096, 24, 4096)) == (1, 1, 1, 1)
    for name in ("gemv_fp16", "gemv_bf16", "gemv_soft_fp8"):
        assert not arg_selector.selector(name).neighbours
    for name in ("layout_gemm", "continuous_gemm", "layoutA_gemm", "layoutA_soft_fp8_gemm"):
        assert arg_selector.selector(name).neighbours


def test_gemv_guard_product():
    assert arg_selector.gemv_guard((512, 1, 2, 4), 4096, 4096) == (512, 1, 2, 4)
    assert arg_selector.gemv_guard((512, 1, 3, 4), 4096, 4096) == (256, 1, 1, 4)
    assert arg_selector.gemv_guard((100, 1, 1, 4), 4096, 4096) == (256, 1, 1, 4)


@pytest.mark.parametrize("name", ["layout_gemm", "continuous_gemm", "layoutA_gemm", "layoutA_soft_fp8_gemm",
                                  "gemv_fp16", "gemv_bf16", "gemv_soft_fp8"])
def test_shipped_tables_parse(name):
    sel = arg_selector.selector(name)
    assert os.path.exists(sel.path()), "every selector ships its table"
    table = sel.table()
    text = open(sel.path()).read()
    assert table == osel.parse_table(text, sel.key_cells)
    for key, val in table.items():
        assert len(key) == sel.key_cells and len(val) == 4
