"""Matrices and operator-graph cases shared by the golden-fixture generator and the parity tests."""
import numpy as np

from alphasparse_amd import _capi as K
from alphasparse_amd import skeletons as SK
from alphasparse_amd import synthetic as S

def _steps(lens, cols, seed):
    """Rows with prescribed lengths, uniform distinct columns, values U[-1,1] (float32)."""
    rng = np.random.default_rng(seed)
    lens = np.asarray(lens, dtype=np.int64)
    row = np.repeat(np.arange(len(lens), dtype=np.int64), lens)
    col = S._distinct_cols(row, cols, rng)
    val = rng.uniform(-1.0, 1.0, len(row))
    return S._finish(len(lens), cols, row, col, val, "uniform", rng, np.float32)


MATRICES = {
    # name: (generator, value dtype)
    "uni40": (lambda: S.uniform_rows(128, 40, seed=3), K.FLOAT),
    "uni8": (lambda: S.uniform_rows(96, 8, seed=4), K.FLOAT),
    "lap": (lambda: S.laplacian_5pt(12, seed=5), K.FLOAT),
    "pl": (lambda: S.power_law(160, max_len=100, mean_len=8.0, seed=7), K.FLOAT),
    "pl_long": (lambda: _steps([100, 250, 400] * 5, 640, 8), K.FLOAT),
    "fem": (lambda: S.fem_blocks(30, 9, 12, seed=9), K.DOUBLE),
    "irr": (lambda: S.extreme_irregular(220, 3, 150, 219, seed=10), K.DOUBLE),
    "steps": (lambda: _steps([3] * 40 + [20] * 24 + [90] * 8, 128, 11), K.FLOAT),
    # benchmark configuration 1 at its stated shape: 4096 x 4096, exactly 8 elements per row, fp32
    "c1": (lambda: S.uniform_rows(), K.FLOAT),
}

D3 = [(K.DENSE_ROW_COARSE_SORT_FIXED, (1,)),
      (K.DENSE_ROW_DIV_ACC_TO_EXPONENTIAL_INCREASE_ROW_NNZ, (8, 64, 4, 0))]
D2 = [(K.DENSE_ROW_DIV_ACC_TO_EXPONENTIAL_INCREASE_ROW_NNZ, (8, 64, 4, 0))]
SORT = [(K.DENSE_ROW_COARSE_SORT_FIXED, (1,))]
COLDIV64 = [("node", K.DENSE_FIXED_COL_DIV, (64,))]
COLDIV50 = [("node", K.DENSE_FIXED_COL_DIV, (50,))]
FINE_SORT = [("node", K.DENSE_FINE_SORT, (), ())]
BAND_SORT = [("node", K.DENSE_FINE_SORT, (), (0, 37, 90, 150))]

# Division of an existing sub-block (node parameters: DENSE_ROW_DIV scalars = {sub-block, height of equal strips},
# DENSE_FIXED_COL_DIV scalars = {band width, sub-block}); the parent leaves the table, its parts go to the end
ROWSTRIPS_UNI = ("node", K.DENSE_ROW_DIV, (), (0, 48, 128))          # uni40: rows [0, 48) and [48, 128)
ROWSTRIPS_PL = ("node", K.DENSE_ROW_DIV, (), (0, 64, 160))           # pl: rows [0, 64) and [64, 160)
SUBDIV_COLS = [ROWSTRIPS_UNI, ("node", K.DENSE_FIXED_COL_DIV, (50, 0))]   # the first strip into bands of 50 columns
SUBDIV_ROWS = [ROWSTRIPS_UNI, ("node", K.DENSE_ROW_DIV, (0, 20), ())]     # the first strip into strips of 20 rows
SUBDIV_ROWS_PL = [ROWSTRIPS_PL, ("node", K.DENSE_ROW_DIV, (1, 30), ())]   # the second strip into strips of 30 rows

# (case id, matrix, dense strategies, skeleton applied to every sub-matrix, skeleton knobs)
FORMAT_CASES = [
    ("ell_uni", "uni8", [], "S5", {"wave": 32}),
    ("ell_lap", "lap", [], "S5", {"wave": 32}),
    ("ell_fem_sorted", "fem", SORT, "S5", {"wave": 32}),
    ("sell64_uni", "uni40", [], "S1", {"m": 64}),
    ("sell32_pl", "pl", [], "S1", {"m": 32}),
    ("sell64_pl_sorted", "pl", SORT, "S1", {"m": 64}),
    ("csr5_t5_pl", "pl", [], "S9", {"t": 5}),
    ("csr5_t3_uni", "uni40", [], "S9", {"t": 3}),
    ("csr5_t2_irr", "irr", [], "S9", {"t": 2}),
    ("wlbcol32_uni", "uni40", [], "S4", {"c": 32}),
    ("wlbcol32_fem_sorted", "fem", SORT, "S4", {"c": 32}),
    ("s6_uni", "uni40", [], "S6", {"m": 4, "len": 40, "c": 32}),
    ("s7_uni", "uni40", [], "S7", {"n": 512, "c": 32}),
    ("s7_pl_long", "pl_long", [], "S7", {"n": 700, "c": 64}),
    ("s6_fem", "fem", [], "S6", {"m": 2, "len": 27, "c": 8}),
    ("longrow128_pl_long", "pl_long", [], "S8", {"b": 128}),
    ("longrow256_pl_long_sorted", "pl_long", SORT, "S8", {"b": 256}),
    ("s2_uni", "uni40", [], "S2", {"m": 32, "len": 40, "s": 4}),
    ("s2_fem", "fem", [], "S2", {"m": 64, "len": 27, "s": 10}),
    ("s3_uni", "uni40", [], "S3", {"n": 512, "s": 7}),
    ("s3_pl_long", "pl_long", [], "S3", {"n": 700, "s": 13}),
    ("base_direct_pl", "pl", [], "B1", {"m": 48, "w": 8}),
    ("base_direct_fem_sorted", "fem", SORT, "B1", {"m": 30, "w": 6}),
    ("base_lds_uni", "uni40", [], "B2", {"n": 512, "w": 4, "s": 7}),
    ("base_lds_pl_long_sorted", "pl_long", SORT, "B2", {"n": 700, "w": 1, "s": 13}),
    ("d2_steps_ell", "steps", D2, "S5", {"wave": 32}),
    ("d3_pl_ell", "pl", D3, "S5", {"wave": 32}),
    ("d3_irr_csr5", "irr", D3, "S9", {"t": 3}),
    # DENSE_FIXED_COL_DIV: column bands, every band a sub-matrix over all rows
    ("coldiv64_uni_ell", "uni40", COLDIV64, "S5", {"wave": 32}),
    ("coldiv50_uni_sell", "uni40", COLDIV50, "S1", {"m": 32}),
    ("coldiv64_uni_csr5", "uni40", COLDIV64, "S9", {"t": 3}),
    ("coldiv50_uni_wlbcol", "uni40", COLDIV50, "S4", {"c": 8}),
    ("coldiv64_uni_longrow", "uni40", COLDIV64, "S8", {"b": 32}),
    ("coldiv64_uni_s2", "uni40", COLDIV64, "S2", {"m": 32, "len": 1, "s": 3}),
    # a sub-block of an already divided matrix divided again (fixed_len_col_div / fixed_len_row_div with a sub-block)
    ("subdiv_cols_uni_ell", "uni40", SUBDIV_COLS, "S5", {"wave": 32}),
    ("subdiv_cols_uni_csr5", "uni40", SUBDIV_COLS, "S9", {"t": 3}),
    ("subdiv_rows_uni_sell", "uni40", SUBDIV_ROWS, "S1", {"m": 32}),
    ("subdiv_rows_pl_csr5", "pl", SUBDIV_ROWS_PL, "S9", {"t": 3}),
    # total_dense_block_sort: all rows by length (stable), and inside bands of rows
    ("finesort_pl_sell", "pl", FINE_SORT, "S1", {"m": 32}),
    ("finesort_irr_ell", "irr", FINE_SORT, "S5", {"wave": 32}),
    ("bandsort_pl_csr5", "pl", BAND_SORT, "S9", {"t": 3}),
    ("bandsort_irr_longrow", "irr", BAND_SORT, "S8", {"b": 32}),
    # compressed_block_sort (op_manager.cc:4104): the rows inside all or some BLBs by falling length, right after the
    # BLB level is made; the permutation (y_write_index) goes through every template's row numbers
    ("blocksort_pl_sell32", "pl", [], "S1", {"m": 32, "block_sort": []}),
    ("blocksort_pl_s2", "pl", [], "S2", {"m": 32, "len": 1, "s": 3, "block_sort": [0, 2, 4]}),
    ("blocksort_pl_s3", "pl", [], "S3", {"n": 128, "s": 3, "block_sort": []}),
    ("blocksort_pl_s6", "pl", [], "S6", {"m": 4, "len": 1, "c": 8, "block_sort": []}),
    ("blocksort_pl_long_s7", "pl_long", [], "S7", {"n": 700, "c": 64, "block_sort": []}),
    ("blocksort_pl_base_direct", "pl", [], "B1", {"m": 40, "w": 8, "block_sort": []}),
    ("blocksort_pl_base_lds", "pl", [], "B2", {"n": 200, "w": 4, "s": 3, "block_sort": [1]}),
    # configuration 1 (4096 x 4096, 8 per row) through the ELL graph and through the SELL graph the search returns for it
    ("c1_ell", "c1", [], "S5", {"wave": 32}),
    ("c1_sell512", "c1", [], "S1", {"m": 512}),
]


# operator graphs without an upstream counterpart (no fixtures; checked through invariants and y parity)
EXTENSION_CASES = [
    ("xslice_pl_long", "pl_long", [], "X1", {"slice": 128}),
    ("xslice_pl_long_sorted", "pl_long", SORT, "X1", {"slice": 256}),
    ("xslice_fem", "fem", [], "X1", {"slice": 32}),
    ("xslice_irr_d3", "irr", D3, "X1", {"slice": 64}),
    ("tile_pl_long", "pl_long", [], "T1", {"slice": 128, "group": 8, "b": 64}),
    ("tile_pl_sorted", "pl", SORT, "T1", {"slice": 64, "group": 32, "b": 100}),
    ("tile_fem", "fem", [], "T1", {"slice": 32, "group": 16, "b": 256}),
    ("tile_irr_d3", "irr", D3, "T1", {"slice": 64, "group": 64, "b": 32}),
    ("tile_steps_d2", "steps", D2, "T1", {"slice": 4096, "group": 4096, "b": 8192}),
    ("tile_subdiv_rows_pl", "pl", SUBDIV_ROWS_PL, "T1", {"slice": 64, "group": 16, "b": 100}),
    ("tile_subdiv_cols_uni", "uni40", SUBDIV_COLS, "T1", {"slice": 32, "group": 16, "b": 64}),
    ("bin_pl_long", "pl_long", [], "T2", {"slice": 128, "group": 8, "b": 64}),
    ("bin_pl_sorted", "pl", SORT, "T2", {"slice": 64, "group": 32, "b": 100}),
    ("bin_fem", "fem", [], "T2", {"slice": 32, "group": 16, "b": 256}),
    ("bin_irr_d3", "irr", D3, "T2", {"slice": 64, "group": 64, "b": 32}),
    ("bin_steps_d2", "steps", D2, "T2", {"slice": 4096, "group": 200, "b": 8192}),
]


# long_short_row_decomposition: (fixture id, matrix name, low bounds of the row-length classes)
DECOMPOSITION_CASES = [
    ("decomp_pl", "pl", (0, 8, 64)),
    ("decomp_irr", "irr", (0, 2, 3, 100, 100000)),     # the last class has no row and is left out
]


def decomposition_dump(make_matrix, case):
    """{"part<i>/<key>": array} of the parts of one decomposition case (COO arrays and shape of every part)."""
    _, mname, bounds = case
    gen, vdt = MATRICES[mname]
    rows, cols, r, c, v, _ = gen()
    m = make_matrix(rows, cols, r, c, np.asarray(v, np.float64), vdt)
    flat = {}
    for i, part in enumerate(m.long_short_row_decomposition(bounds)):
        info = part.info()
        flat["part%d/shape" % i] = np.array([info["rows"], info["cols"], info["nnz"]], np.int64)
        flat["part%d/row" % i] = np.asarray(part.get_u64(-1, 103, 0)[0], np.int64)
        flat["part%d/col" % i] = np.asarray(part.get_u64(-1, 103, 1)[0], np.int64)
        flat["part%d/val" % i] = np.asarray(part.get_f64(-1, 3), np.float64)
    return flat


# Row and column padding of the whole matrix: (fixture id, matrix name, [(operator, arguments), ...]); the
# arguments of dense_col_level_padding are (every n-th row, elements added to it)
PADDING_CASES = [
    ("pad_rows_end", "pl", [("total_row_level_padding", (64, K.END_PADDING, 3))]),
    ("pad_rows_top", "pl", [("total_row_level_padding", (64, K.TOP_PADDING, 0))]),
    ("pad_rows_multiple_already", "uni40", [("total_row_level_padding", (32, K.END_PADDING, 0))]),
    ("pad_add_end3", "irr", [("total_row_level_padding_add", (37, 3, K.END_PADDING, 5))]),
    ("pad_add_top", "fem", [("total_row_level_padding_add", (5, 1, K.TOP_PADDING, 0))]),
    ("pad_direct_end0", "lap", [("total_row_level_padding_direct", (200, 0, K.END_PADDING, 0))]),
    ("pad_cols", "pl", [("dense_col_level_padding", (7, 3))]),
    ("pad_rows_then_cols", "irr", [("total_row_level_padding", (128, K.END_PADDING, 1)), ("dense_col_level_padding", (5, 2))]),
]


def padding_dump(make_matrix, case):
    """{"shape", "row", "col", "val"} of the matrix after the padding operators of one PADDING_CASE."""
    _, mname, steps = case
    gen, vdt = MATRICES[mname]
    rows, cols, r, c, v, _ = gen()
    m = make_matrix(rows, cols, r, c, np.asarray(v, np.float64), vdt)
    for name, args in steps:
        if name == "dense_col_level_padding":
            every, extra = args
            n_rows = m.info()["rows"]
            lens = np.bincount(np.asarray(m.get_u64(-1, 103, 0)[0], np.int64), minlength=n_rows)
            picked = np.arange(0, n_rows, every)
            m.dense_col_level_padding(picked, lens[picked] + extra)
        else:
            getattr(m, name)(*args)
    info = m.info()
    return {"shape": np.array([info["rows"], info["cols"], info["nnz"]], np.int64),
            "row": np.asarray(m.get_u64(-1, 103, 0)[0], np.int64),
            "col": np.asarray(m.get_u64(-1, 103, 1)[0], np.int64),
            "val": np.asarray(m.get_f64(-1, 3), np.float64)}


def build_case(make_matrix, case, wave):
    """Run one FORMAT_CASE on a matrix object (product Matrix or upstream RefMatrix).
    make_matrix(rows, cols, row, col, val, val_dtype) -> object with the MatrixAPI methods."""
    _, mname, dense, skel, kw = case
    gen, vdt = MATRICES[mname]
    rows, cols, r, c, v, x = gen()
    m = make_matrix(rows, cols, r, c, v.astype(np.float64), vdt)
    for step in dense:
        if step[0] == "node":      # ("node", node type, scalars[, list]): a dense node without a parameter strategy
            m.execute_node(step[1], -1, scalars=step[2], lst=step[3] if len(step) > 3 else ())
        else:
            m.execute_strategy(step[0], -1, step[1])
    m.execute_strategy(K.COMPRESS_NONE)
    kw = dict(kw)
    if skel == "S5":
        kw["wave"] = wave
    templates = None
    for sub in range(m.info()["n_sub"]):
        templates = SK.apply_skeleton(m, sub, skel, **kw)
    return m, templates


def flatten_dump(d, prefix=""):
    """dict from MatrixAPI.dump() / template_dump() -> {key: ndarray} suitable for np.savez."""
    out = {}
    for k, v in d.items():
        key = prefix + k
        if isinstance(v, dict):
            out.update(flatten_dump(v, key + "/"))
        elif isinstance(v, tuple):
            a = np.asarray(v[0])
            if a.dtype == np.uint64 and (len(a) == 0 or a.max() < 2 ** 32):
                a = a.astype(np.uint32)
            out[key + "|values"] = a
            out[key + "|meta"] = np.array([str(x) for x in v[1:]])
        elif isinstance(v, (int, np.integer)):
            out[key + "|scalar"] = np.array([v], dtype=np.int64)
        else:
            v = np.asarray(v)
            if v.dtype == np.float64 and np.array_equal(v.astype(np.float32).astype(np.float64), v):
                v = v.astype(np.float32)  # exact; halves the fixture size for fp32 matrices
            elif v.dtype == np.uint64 and (len(v) == 0 or v.max() < 2 ** 32):
                v = v.astype(np.uint32)
            out[key + "|values"] = v
    return out


def compare_flat(got, want, skip=()):
    """-> list of human-readable differences between two flattened dumps."""
    diffs = []
    for k in sorted(set(got) | set(want)):
        if any(s in k for s in skip):
            continue
        if k not in got or k not in want:
            diffs.append("%s: only in %s" % (k, "got" if k in got else "want"))
            continue
        a, b = np.asarray(got[k]), np.asarray(want[k])
        if a.dtype.kind in "ui" and b.dtype.kind in "ui":
            a, b = a.astype(np.uint64), b.astype(np.uint64)
        elif a.dtype.kind in "uif" and b.dtype.kind in "uif":
            a, b = a.astype(np.float64), b.astype(np.float64)
        if a.shape != b.shape or not np.array_equal(a, b):
            diffs.append("%s: got %s%s want %s%s" % (k, a.shape, a.ravel()[:8], b.shape, b.ravel()[:8]))
    return diffs
