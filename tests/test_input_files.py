"""Input files of the hot path: Matrix Market ingestion (upstream data_prepare.py:34-66 in one step), the
.mtx.coo text the upstream program reads (struct.cc:92-175) and the binary cache.  CPU only."""
import numpy as np
import pytest

import cases
import alphasparse_amd as A
from alphasparse_amd import _capi as K


def _coo(m):
    d = m.dump()
    return (d["coo_row_index_cache"].astype(np.int64), d["coo_col_index_cache"].astype(np.int64),
            np.asarray(d["coo_value_cache"], np.float64))


def _data_prepare(text, keep_values):
    """What upstream's data_prepare.py writes for a general Matrix Market file: '%' lines dropped, the first
    remaining line is the size line, entries sorted as (row, col, val) tuples; val forced to 1 upstream."""
    lines = [ln for ln in text.splitlines() if ln and ln[0] != "%"]
    rows, cols = (int(t) for t in lines[0].split()[:2])
    data = sorted((int(a), int(b), float(c[0]) if keep_values and c else 1.0) for a, b, *c in (ln.split() for ln in lines[1:]))
    r, c, v = (np.array(x) for x in zip(*data))
    return rows, cols, r - 1, c - 1, v.astype(np.float64)


GENERAL = """%%MatrixMarket matrix coordinate real general
% a comment
%another
4 5 7
3 1 2.5
1 2 -1e-3
4 5 7
1 1 4.0
2 3 1.25E+2
3 4 -8
2 1 0.5
"""


@pytest.mark.parametrize("keep", [True, False])
def test_mtx_general_matches_data_prepare(tmp_path, keep):
    p = tmp_path / "g.mtx"
    p.write_text(GENERAL)
    m = A.Matrix.from_mtx_file(p, K.DOUBLE, keep_values=keep)
    rows, cols, r, c, v = _data_prepare(GENERAL, keep)
    info = m.info()
    assert (info["rows"], info["cols"], info["nnz"]) == (rows, cols, len(r))
    gr, gc, gv = _coo(m)
    assert np.array_equal(gr, r) and np.array_equal(gc, c) and np.array_equal(gv, v)
    assert m.check_sorted() and not m.has_empty_row()


def test_mtx_symmetric_skew_and_pattern(tmp_path):
    sym = "%%MatrixMarket matrix coordinate real symmetric\n3 3 4\n1 1 2\n2 1 -1\n3 2 5\n3 3 1\n"
    p = tmp_path / "s.mtx"
    p.write_text(sym)
    r, c, v = _coo(A.Matrix.from_mtx_file(p, K.DOUBLE))
    dense = np.zeros((3, 3))
    dense[r, c] = v
    assert np.array_equal(dense, [[2, -1, 0], [-1, 0, 5], [0, 5, 1]]) and len(r) == 6
    skew = "%%MatrixMarket matrix coordinate real skew-symmetric\n3 3 2\n2 1 -1\n3 1 4\n"
    p.write_text(skew)
    r, c, v = _coo(A.Matrix.from_mtx_file(p, K.DOUBLE))
    dense = np.zeros((3, 3))
    dense[r, c] = v
    assert np.array_equal(dense, [[0, 1, -4], [-1, 0, 0], [4, 0, 0]])
    pat = "%%MatrixMarket matrix coordinate pattern general\n2 3 3\n2 3\n1 1\n2 1\n"
    p.write_text(pat)
    m = A.Matrix.from_mtx_file(p, K.FLOAT)
    r, c, v = _coo(m)
    assert r.tolist() == [0, 1, 1] and c.tolist() == [0, 0, 2] and v.tolist() == [1, 1, 1]


def test_mtx_float_values_are_rounded_like_stof(tmp_path):
    p = tmp_path / "f.mtx"
    p.write_text("%%MatrixMarket matrix coordinate real general\n1 2 2\n1 1 0.1\n1 2 1e-40\n")
    _, _, v32 = _coo(A.Matrix.from_mtx_file(p, K.FLOAT))
    _, _, v64 = _coo(A.Matrix.from_mtx_file(p, K.DOUBLE))
    assert v32[0] == float(np.float32(0.1)) and v32[1] == float(np.float32(1e-40)) and v64.tolist() == [0.1, 1e-40]


def test_mtx_errors_and_empty_rows(tmp_path):
    p = tmp_path / "e.mtx"
    p.write_text("%%MatrixMarket matrix coordinate real general\n3 3 2\n1 1 1\n3 3 1\n")
    m = A.Matrix.from_mtx_file(p, K.FLOAT)
    assert m.has_empty_row() and m.check_sorted()          # upstream's script stops here ("has empty line")
    for bad in ("%%MatrixMarket matrix array real general\n2 2\n1\n2\n3\n4\n",
                "%%MatrixMarket matrix coordinate complex general\n2 2 1\n1 1 1 0\n",
                "%%MatrixMarket matrix coordinate real general\n2 2 1\n3 1 1\n",
                "%%MatrixMarket matrix coordinate real general\n2 2 1\n1 1\n",
                "%%MatrixMarket matrix coordinate real general\n2 2 0\n"):
        p.write_text(bad)
        with pytest.raises(A.AlphaSparseError):
            A.Matrix.from_mtx_file(p, K.FLOAT)
    with pytest.raises(A.AlphaSparseError):
        A.Matrix.from_mtx_file(tmp_path / "missing.mtx", K.FLOAT)


@pytest.mark.parametrize("vdt,npd", [(K.FLOAT, np.float32), (K.DOUBLE, np.float64)])
def test_binary_cache_round_trip(tmp_path, vdt, npd):
    rows, cols, r, c, v, _ = cases._steps([3, 1, 4, 1, 5, 9, 2, 6, 1, 1], 70000, 5)
    v = np.asarray(v, np.float64) * np.pi
    m = A.Matrix.from_coo(rows, cols, r, c, v, vdt)
    path = tmp_path / "m.bin"
    m.write_binary_file(path)
    assert path.stat().st_size == 64 + len(r) * (8 + np.dtype(npd).itemsize)
    m2 = A.Matrix.from_binary_file(path)
    a, b = _coo(m), _coo(m2)
    assert all(np.array_equal(x, y) for x, y in zip(a, b))
    i, j = m.info(), m2.info()
    assert (i["rows"], i["cols"], i["nnz"]) == (j["rows"], j["cols"], j["nnz"])
    # the same matrix through the three file formats
    coo = tmp_path / "m.mtx.coo"
    m.write_coo_file(coo)
    c3 = _coo(A.Matrix.from_coo_file(coo, vdt))
    assert all(np.array_equal(x, y) for x, y in zip(a, c3))
    mtx = tmp_path / "m.mtx"
    mtx.write_text("%%MatrixMarket matrix coordinate real general\n" + coo.read_text())
    c4 = _coo(A.Matrix.from_mtx_file(mtx, vdt))
    assert all(np.array_equal(x, y) for x, y in zip(a, c4))


def test_binary_cache_rejects_damaged_files(tmp_path):
    rows, cols, r, c, v, _ = cases._steps([2, 3, 1], 9, 6)
    m = A.Matrix.from_coo(rows, cols, r, c, np.asarray(v, np.float64), K.FLOAT)
    path = tmp_path / "m.bin"
    m.write_binary_file(path)
    raw = path.read_bytes()
    for damaged in (raw[:-1], raw + b"\0", b"NOTACOO\0" + raw[8:], raw[:36] + b"\x07" + raw[37:]):
        path.write_bytes(damaged)
        with pytest.raises(A.AlphaSparseError):
            A.Matrix.from_binary_file(path)
    # an index beyond the matrix
    bad = bytearray(raw)
    bad[64:68] = (1000).to_bytes(4, "little")
    path.write_bytes(bytes(bad))
    with pytest.raises(A.AlphaSparseError):
        A.Matrix.from_binary_file(path)


# ---- the .mtx.coo reader against a literal file and against the reference's own reader ------------------------------
# 1-based indices, rows non-decreasing, header with and without the element count, values in the spellings stof /
# stod accept, a blank line and a line that starts with white space (both skipped by the reference, struct.cc:121).
COO_TEXT = """4 6 7
1 1 4.0
1 6 -1
2 3 1.25E+2

3 1 0.1
 9 9 9
3 4 -8e-3
4 2 1e-40
4 6 16777217
"""
COO_KNOWN = dict(rows=4, cols=6, row=[0, 0, 1, 2, 2, 3, 3], col=[0, 5, 2, 0, 3, 1, 5],
                 val=[4.0, -1.0, 125.0, 0.1, -8e-3, 1e-40, 16777217.0])


@pytest.mark.parametrize("vdt,npd", [(K.FLOAT, np.float32), (K.DOUBLE, np.float64)], ids=["fp32", "fp64"])
@pytest.mark.parametrize("header", ["4 6 7", "4 6"], ids=["with_nnz", "without_nnz"])
def test_coo_file_known_answer(tmp_path, vdt, npd, header):
    p = tmp_path / "k.mtx.coo"
    p.write_text(COO_TEXT.replace("4 6 7", header, 1))
    m = A.Matrix.from_coo_file(p, vdt)
    info = m.info()
    assert (info["rows"], info["cols"], info["nnz"]) == (COO_KNOWN["rows"], COO_KNOWN["cols"], 7)
    r, c, v = _coo(m)
    assert r.tolist() == COO_KNOWN["row"] and c.tolist() == COO_KNOWN["col"]
    # every value rounded once, from the decimal text to the value type (stof / stod): 0.1 and 16777217 differ
    # between float and double, 1e-40 is a float denormal
    want = np.array([npd(t) for t in ("4.0", "-1", "1.25E+2", "0.1", "-8e-3", "1e-40", "16777217")]).astype(np.float64)
    assert np.array_equal(v, want)
    assert m.check_sorted() and not m.has_empty_row()


def _ref_read(path, vdt):
    import ctypes as C
    import ref_lib
    L = ref_lib.lib()
    L.ref_read_coo_file.restype = C.c_int64
    L.ref_read_coo_file.argtypes = [C.c_char_p, C.c_int, K.u64p, K.u64p, K.f64p, C.c_uint64, K.u64p]
    hdr = np.zeros(2, np.uint64)
    n = L.ref_read_coo_file(str(path).encode(), vdt, None, None, None, 0, hdr.ctypes.data_as(K.u64p))
    r, c, v = np.zeros(n, np.uint64), np.zeros(n, np.uint64), np.zeros(n, np.float64)
    L.ref_read_coo_file(str(path).encode(), vdt, r.ctypes.data_as(K.u64p), c.ctypes.data_as(K.u64p), v.ctypes.data_as(K.f64p), n,
                        hdr.ctypes.data_as(K.u64p))
    return int(hdr[0]) + 1, int(hdr[1]) + 1, r.astype(np.int64), c.astype(np.int64), v


def _needs_reference():
    import ref_lib
    if not ref_lib.available():
        pytest.skip("oracle/_ref/libasref.so is not built (make -C oracle ref, needs the reference sources)")


@pytest.mark.parametrize("where", ["cpu", pytest.param("gpu_box", marks=pytest.mark.gpu)])
@pytest.mark.parametrize("vdt", [K.FLOAT, K.DOUBLE], ids=["fp32", "fp64"])
def test_coo_file_reader_matches_the_reference_reader(tmp_path, vdt, where):
    """as_matrix_from_coo_file against get_matrix_index_and_val_from_file (struct.cc:92-175) compiled from the
    reference's own source: the literal file with and without the element count, and generated files whose values
    are written with 9 and 17 significant digits, in plain and in exponent spelling."""
    _needs_reference()
    # (the reference's stof throws on a value that is no normal float, and the exception ends the process: the
    # denormal of the literal file is only given to the fp64 reader, and generated values stay within float range)
    literal = COO_TEXT if vdt == K.DOUBLE else COO_TEXT.replace("1e-40", "1e-30")
    texts = [literal, literal.replace("4 6 7", "4 6", 1)]
    rng = np.random.default_rng(11)
    for seed, fmt in ((1, "%.9g"), (2, "%.17g"), (3, "%e"), (4, "%.3f")):
        rows, cols, r, c, _, _ = cases._steps([3, 1, 40, 1, 5, 9, 2, 6, 1, 1] * 7, 900, seed)
        vals = rng.standard_normal(len(r)) * 10.0 ** rng.integers(-25, 25, len(r))
        lines = ["%d %d %d" % (rows, cols, len(r))] + ["%d %d %s" % (a + 1, b + 1, fmt % x) for a, b, x in zip(r, c, vals)]
        texts.append("\n".join(lines) + ("\n" if seed % 2 else ""))          # with and without a final newline
    for i, text in enumerate(texts):
        p = tmp_path / ("m%d.mtx.coo" % i)
        p.write_text(text)
        m = A.Matrix.from_coo_file(p, vdt)
        info = m.info()
        r, c, v = _coo(m)
        ref_rows, ref_cols, rr, rc, rv = _ref_read(p, vdt)
        assert (info["rows"], info["cols"], info["nnz"]) == (ref_rows, ref_cols, len(rr)), i
        assert np.array_equal(r, rr) and np.array_equal(c, rc), i
        assert np.array_equal(v.view(np.uint64), rv.view(np.uint64)), i      # bit for bit


@pytest.mark.parametrize("bad,why", [
    ("3 3 2\n1 1 1\n0 2 1\n", "row index 0"), ("3 3 2\n1 0 1\n2 2 1\n", "column index 0"),
    ("3 3 2\n1 1 1\n4 2 1\n", "row beyond the header"), ("3 3 2\n1 4 1\n2 2 1\n", "column beyond the header"),
    ("3 3 2\n1 1 1\n2 2\n", "no value"), ("3 3 2\n1 1 1\nx 2 1\n", "row does not parse"),
    ("3 3 2\n1 1 1\n2 y 1\n", "column does not parse"), ("3 3 2\n1 1 1\n2 2 z\n", "value does not parse"),
    ("3 3 2\n2 1 1\n1 2 1\n", "rows decrease"), ("0 3 1\n1 1 1\n", "no rows"), ("3 3 0\n", "no entries"), ("", "empty file"),
    ("3 3 2\n1 1 1\n-2 2 1\n", "negative row")], ids=lambda t: t.replace(" ", "_") if " " in t and "\n" not in t else None)
def test_coo_file_rejects_bad_entries(tmp_path, bad, why):
    """An entry outside the matrix would address x or y out of bounds on the device: the reader stops instead
    (the reference takes whatever atol makes of the line: struct.cc:140-141)."""
    p = tmp_path / "bad.mtx.coo"
    p.write_text(bad)
    with pytest.raises(A.AlphaSparseError):
        A.Matrix.from_coo_file(p, K.FLOAT)


def test_from_coo_arrays_rejects_entries_outside_the_matrix():
    with pytest.raises(A.AlphaSparseError):
        A.Matrix.from_coo(3, 3, [0, 3], [0, 1], np.ones(2), K.FLOAT)
    with pytest.raises(A.AlphaSparseError):
        A.Matrix.from_coo(3, 3, [0, 1], [0, 3], np.ones(2), K.FLOAT)
