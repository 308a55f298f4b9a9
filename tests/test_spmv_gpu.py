"""y = A x through the generated HIP kernels (called through the C ABI) against the CPU CSR oracle.

Acceptance: relative L2 error <= 1e-5 (fp32) / 1e-12 (fp64) AND, per row,
|y - y_ref| <= 64 * eps * sum|a_ij x_j|.  Formats are built at wave = 64."""
import ctypes as C

import numpy as np
import pytest

import cases
import spmv_oracle as O
import alphasparse_amd as A
from alphasparse_amd import _capi as K
from alphasparse_amd import skeletons as SK
from alphasparse_amd import synthetic as S

pytestmark = pytest.mark.gpu

NP = {K.FLOAT: np.float32, K.DOUBLE: np.float64}


def oracle_y(rows, r, c, v, x):
    return O.spmv_csr(O.coo_to_csr(rows, r), c.astype(np.uint32), v, x)


def assert_y(y, y_ref, mag, npd, what):
    rel, ratio, tol = O.check_y(y, y_ref, mag, npd)
    assert rel <= tol, "%s: relative L2 error %.3e > %.0e" % (what, rel, tol)
    assert ratio <= 1.0, "%s: a row exceeds its error bound (%.2f x)" % (what, ratio)


def run_case(gpu, gen, vdt, dense, skel, kw, launches=({},), templates_filter=None):
    rows, cols, r, c, v, x = gen
    npd = NP[vdt]
    v, x = v.astype(npd), x.astype(npd)
    y_ref, mag = oracle_y(rows, r, c, v, x)
    m = A.Matrix.from_coo(rows, cols, r, c, v.astype(np.float64), vdt, wave=64)
    for step in dense:
        if step[0] == "node":
            m.execute_node(step[1], -1, scalars=step[2], lst=step[3] if len(step) > 3 else ())
        else:
            m.execute_strategy(step[0], -1, step[1])
    m.execute_strategy(K.COMPRESS_NONE)
    n_sub = m.info()["n_sub"]
    for sub in range(n_sub):
        templates = SK.apply_skeleton(m, sub, skel, **kw)
    ran = 0
    for tp in templates:
        if templates_filter and tp not in templates_filter:
            continue
        assert all(A.template_is_supported(m, s, tp) for s in range(n_sub)), K.TEMPLATE_NAMES[tp]
        for launch in launches:
            b = A.Builder(m)
            for s in range(n_sub):
                b.set_template(s, tp)
                if launch:
                    b.set_launch(s, **launch)
            b.compile().upload(gpu)
            what = "%s %s %s %s" % (skel, kw, K.TEMPLATE_NAMES[tp], launch)
            print("case:", what, flush=True)
            assert_y(b.spmv(x), y_ref, mag, npd, what)
            assert_y(b.spmv(x), y_ref, mag, npd, what + " (second run: y must be re-zeroed)")
            # a y full of NaN before the call: the clear is launched exactly where the graph needs it, and a
            # graph without clear stores every row
            assert_y(b.spmv_device(x), y_ref, mag, npd, what + " (y = NaN before the call, clear: %s)" % b.clears_y())
            b.close()
            ran += 1
    assert ran > 0


def test_wave_reductions_dpp_matches_shuffle(gpu):
    """as_group_sum (DPP row operations) against the ds_bpermute shuffle version and numpy."""
    L = K.lib()
    L.as_selftest_group_sum.argtypes = [C.c_int, C.c_int, C.c_int, K.f64p, K.f64p, K.f64p]
    rng = np.random.default_rng(0)
    for is_double in (0, 1):
        for lanes in (1, 2, 4, 8, 16, 32, 64):
            vin = rng.integers(-9, 9, 64).astype(np.float64)
            a, b = np.zeros(64), np.zeros(64)
            assert L.as_selftest_group_sum(gpu, lanes, is_double, vin.ctypes.data_as(K.f64p), a.ctypes.data_as(K.f64p),
                                           b.ctypes.data_as(K.f64p)) == 0, L.as_last_error()
            want = vin.reshape(-1, lanes).sum(1)
            assert np.array_equal(a.reshape(-1, lanes)[:, -1], want)   # last lane of each group
            assert np.array_equal(b.reshape(-1, lanes)[:, 0], want)
            if lanes <= 16:
                assert np.array_equal(a.reshape(-1, lanes), np.repeat(want[:, None], lanes, 1))


def test_wave_segmented_sum(gpu):
    """as_wave_segmented_sum / as_is_segment_tail (DPP row shifts + row broadcasts) against numpy on key patterns
    whose runs start, end and cross the 16-lane rows in every way."""
    L = K.lib()
    u32p = C.POINTER(C.c_uint32)
    L.as_selftest_segmented_sum.argtypes = [C.c_int, C.c_int, u32p, K.f64p, K.f64p, K.f64p]
    rng = np.random.default_rng(1)
    patterns = [np.zeros(64), np.arange(64), np.arange(64) // 16, np.arange(64) // 3, (np.arange(64) + 5) // 16,
                np.r_[np.zeros(15), np.ones(49)], np.r_[np.zeros(17), np.ones(30), np.full(17, 2)],
                np.r_[np.zeros(31), np.ones(2), np.full(31, 7)], np.r_[np.arange(10), np.full(54, 10)]]
    patterns += [np.sort(rng.integers(0, k, 64)) for k in (2, 3, 5, 9, 20, 64, 65535) for _ in range(6)]
    for is_double in (0, 1):
        for key in patterns:
            key = np.ascontiguousarray(key, dtype=np.uint32)
            vin = rng.integers(-9, 9, 64).astype(np.float64)
            a, b = np.zeros(64), np.zeros(64)
            assert L.as_selftest_segmented_sum(gpu, is_double, key.ctypes.data_as(u32p), vin.ctypes.data_as(K.f64p),
                                               a.ctypes.data_as(K.f64p), b.ctypes.data_as(K.f64p)) == 0, L.as_last_error()
            want = np.array([vin[np.flatnonzero(key[:i + 1] == key[i])].sum() for i in range(64)])
            tail = np.r_[key[1:] != key[:-1], True].astype(np.float64)
            assert np.array_equal(a, want), (key, a, want)
            assert np.array_equal(b, tail), (key, b, tail)


MATS = {
    "uni40": lambda: S.uniform_rows(2048, 40, seed=3),
    "lap": lambda: S.laplacian_5pt(100),
    "pl": lambda: S.power_law(3000, max_len=900, mean_len=14.0, seed=7),
    "fem": lambda: S.fem_blocks(700, 27, 200),
    "irr": lambda: S.extreme_irregular(4000, 6, 2000, 3999, seed=9),
    "odd": lambda: cases._steps([100, 250, 400, 1500] * 40, 2043, 8),
}
D3 = [(K.DENSE_ROW_COARSE_SORT_FIXED, (1,)), (K.DENSE_ROW_DIV_ACC_TO_EXPONENTIAL_INCREASE_ROW_NNZ, (32, 2048, 4, 0))]
SORT = [(K.DENSE_ROW_COARSE_SORT_FIXED, (1,))]
COLDIV = lambda width: [("node", K.DENSE_FIXED_COL_DIV, (width,))]
FINE_SORT = lambda *bands: [("node", K.DENSE_FINE_SORT, (), bands)]
VEC = ({}, {"vec_width": 2}, {"vec_width": 4})
RED = ({}, {"thread_num_of_row_reduce": 4}, {"thread_num_of_row_reduce": 16}, {"thread_num_of_row_reduce": 64})

GPU_CASES = [
    ("lap", [], "S5", {}, VEC), ("uni40", [], "S5", {}, VEC), ("pl", SORT, "S5", {}, ({},)),
    ("lap", [], "S1", {"m": 64}, VEC), ("lap", [], "S1", {"m": 256}, VEC), ("pl", SORT, "S1", {"m": 128}, ({},)),
    ("lap", [], "S9", {"t": 3}, ({},)), ("pl", [], "S9", {"t": 5}, ({}, {"thread_num_in_block": 128})),
    ("pl", [], "S9", {"t": 2}, ({},)), ("irr", [], "S9", {"t": 4}, ({},)), ("uni40", [], "S9", {"t": 32}, ({},)),
    ("uni40", [], "S4", {"c": 16}, VEC), ("fem", [], "S4", {"c": 64}, VEC), ("pl", SORT, "S4", {"c": 32}, ({},)),
    ("uni40", [], "S6", {"m": 4, "len": 40, "c": 16}, RED), ("fem", [], "S6", {"m": 2, "len": 81, "c": 32}, RED),
    ("uni40", [], "S7", {"n": 512, "c": 16}, RED), ("pl", SORT, "S7", {"n": 896, "c": 64}, ({},)),
    ("fem", [], "S8", {"b": 128}, ({}, {"thread_num_in_block": 64}, {"thread_num_in_block": 1024})),
    ("irr", [], "S8", {"b": 1024}, ({},)), ("pl", [], "S8", {"b": 256}, ({},)), ("pl", SORT, "S8", {"b": 512}, ({},)),
    ("uni40", [], "S2", {"m": 64, "len": 40, "s": 4}, RED), ("fem", [], "S2", {"m": 32, "len": 81, "s": 10}, RED),
    ("uni40", [], "S3", {"n": 896, "s": 7}, RED), ("pl", SORT, "S3", {"n": 512, "s": 3}, ({},)),
    ("pl", D3, "S8", {"b": 128}, ({},)), ("pl", D3, "S1", {"m": 64}, ({},)), ("pl", D3, "S5", {}, ({},)),
    ("irr", D3, "S9", {"t": 3}, ({},)),
    # DENSE_FIXED_COL_DIV: column bands over all rows; every band's kernel reads x from its first column on and
    # accumulates y atomically (513 and 701 give bands whose first column is not a multiple of 4)
    ("uni40", COLDIV(700), "S5", {}, VEC), ("uni40", COLDIV(513), "S1", {"m": 64}, ({},)), ("uni40", COLDIV(1024), "S9", {"t": 4}, ({},)),
    ("uni40", COLDIV(701), "S8", {"b": 64}, ({},)), ("uni40", COLDIV(1024), "S4", {"c": 16}, ({},)),
    ("uni40", COLDIV(512), "S2", {"m": 64, "len": 1, "s": 4}, ({},)), ("uni40", COLDIV(700), "T1", {"slice": 256, "group": 128, "b": 512}, ({},)),
    ("uni40", COLDIV(513), "T1", {"slice": 128, "group": 512, "b": 512}, ({},)), ("fem", COLDIV(1000), "S1", {"m": 64}, ({},)),
    ("uni40", COLDIV(600), "B1", {"m": 64, "w": 16}, ({},)), ("uni40", COLDIV(600), "X1", {"slice": 128}, ({},)),
    # total_dense_block_sort over all rows and inside bands of rows: y goes back through the permutation
    ("pl", FINE_SORT(), "S1", {"m": 64}, ({},)), ("pl", FINE_SORT(0, 1000, 1001, 2500), "S5", {}, ({},)),
    ("irr", FINE_SORT(0, 17), "T1", {"slice": 1024, "group": 512, "b": 300}, ({},)), ("pl", FINE_SORT(0, 700), "T2", {"slice": 512, "group": 16, "b": 1024}, ({},)),
    # compressed_block_sort: rows inside the BLBs by falling length, y through y_write_index (direct stores, LDS
    # row sums and atomics alike); all BLBs or a few of them
    ("pl", [], "S1", {"m": 128, "block_sort": []}, VEC), ("irr", [], "S1", {"m": 64, "block_sort": [0, 3, 7]}, ({},)),
    ("pl", [], "S2", {"m": 64, "len": 1, "s": 4, "block_sort": []}, RED), ("pl", [], "S3", {"n": 512, "s": 3, "block_sort": []}, ({},)),
    ("pl", [], "S6", {"m": 4, "len": 1, "c": 16, "block_sort": []}, ({},)), ("pl", [], "S7", {"n": 896, "c": 64, "block_sort": [1, 2]}, ({},)),
    ("pl", [], "B1", {"m": 96, "w": 8, "block_sort": []}, ({},)), ("pl", [], "B2", {"n": 512, "w": 8, "s": 3, "block_sort": []}, ({},)),
    ("uni40", COLDIV(700), "S1", {"m": 64, "block_sort": []}, ({},)), ("pl", D3[1:], "S1", {"m": 64, "block_sort": []}, ({},)),
    # the two general templates (outside the white list)
    ("uni40", [], "B1", {"m": 64, "w": 16}, ({}, {"thread_num_in_block": 64}, {"thread_num_in_block": 1024})),
    ("pl", SORT, "B1", {"m": 96, "w": 8}, ({},)), ("pl", D3, "B1", {"m": 64, "w": 8}, ({},)), ("fem", [], "B1", {"m": 30, "w": 6}, ({},)),
    ("uni40", [], "B2", {"n": 512, "w": 4, "s": 7}, RED), ("pl", SORT, "B2", {"n": 512, "w": 8, "s": 3}, ({},)),
    ("fem", [], "B2", {"n": 1024, "w": 3, "s": 10}, RED),
    # x slice in LDS (no upstream counterpart); "odd" has a column count that is not a multiple of 4
    ("pl", [], "X1", {"slice": 512}, ({}, {"thread_num_in_block": 256})), ("pl", D3, "X1", {"slice": 1024}, ({},)),
    ("irr", SORT, "X1", {"slice": 1024}, ({},)), ("fem", [], "X1", {"slice": 128}, ({},)),
    ("odd", [], "X1", {"slice": 256}, ({}, {"thread_num_in_block": 64})), ("odd", [], "X1", {"slice": 16384}, ({},)),
    # 2-D tiles, x slice and row sums in LDS (no upstream counterpart): rows of every length, tiles smaller and
    # larger than a BLB, more and fewer rows than a row group, sort permutation, strips
    ("pl", [], "T1", {"slice": 512, "group": 256, "b": 1024}, ({}, {"thread_num_in_block": 256}, {"thread_num_in_block": 64})),
    ("pl", SORT, "T1", {"slice": 1024, "group": 4096, "b": 512}, ({},)), ("pl", D3, "T1", {"slice": 256, "group": 64, "b": 8192}, ({},)),
    ("irr", SORT, "T1", {"slice": 1024, "group": 512, "b": 300}, ({},)), ("fem", [], "T1", {"slice": 128, "group": 128, "b": 4096}, ({},)),
    ("odd", [], "T1", {"slice": 256, "group": 16, "b": 8192}, ({}, {"thread_num_in_block": 128})),
    ("odd", [], "T1", {"slice": 16384, "group": 4096, "b": 2048}, ({},)), ("lap", [], "T1", {"slice": 2048, "group": 2048, "b": 8192}, ({},)),
    ("uni40", [], "T1", {"slice": 16384, "group": 4096, "b": 8192}, ({},)),
    # the same tiles in two passes (products to scratch, row sums per row group)
    # (a row group needs rows x longest row LDS slots, so matrices with long rows get small groups here)
    ("pl", [], "T2", {"slice": 512, "group": 16, "b": 1024}, ({}, {"thread_num_in_block": 256}, {"thread_num_in_block": 64})),
    ("pl", SORT, "T2", {"slice": 1024, "group": 20, "b": 512}, ({},)), ("pl", D3, "T2", {"slice": 256, "group": 8, "b": 8192}, ({},)),
    ("irr", SORT, "T2", {"slice": 1024, "group": 4, "b": 300}, ({},)), ("fem", [], "T2", {"slice": 128, "group": 128, "b": 4096}, ({},)),
    ("odd", [], "T2", {"slice": 256, "group": 8, "b": 8192}, ({}, {"thread_num_in_block": 128})),
    ("odd", [], "T2", {"slice": 16384, "group": 13, "b": 2048}, ({},)), ("lap", [], "T2", {"slice": 2048, "group": 2048, "b": 8192}, ({},)),
    ("lap", SORT, "T2", {"slice": 16384, "group": 4095, "b": 8192}, ({},)), ("uni40", [], "T2", {"slice": 16384, "group": 511, "b": 8192}, ({},)),
    ("uni40", [], "T2", {"slice": 64, "group": 100, "b": 64}, ({},)),
    # row groups much larger than a summing group of the second pass; rows longer than the slot budget
    ("pl", SORT, "T2", {"slice": 1024, "group": 4096, "b": 512}, ({},)), ("pl", [], "T2", {"slice": 512, "group": 1000, "b": 1024}, ({},)),
    ("irr", SORT, "T2", {"slice": 1024, "group": 2048, "b": 300}, ({},)), ("lap", [], "T2", {"slice": 4096, "group": 10000, "b": 8192}, ({},)),
]


@pytest.mark.parametrize("vdt", [K.FLOAT, K.DOUBLE], ids=["fp32", "fp64"])
@pytest.mark.parametrize("mat,dense,skel,kw,launches", GPU_CASES,
                         ids=["%s-%s%s-%s" % (c[0], "D" if c[1] else "", c[2], "_".join("%s%s" % (k, "".join(map(str, v)) if isinstance(v, list) else v) for k, v in c[3].items())) for c in GPU_CASES])
def test_spmv_matches_cpu_csr(gpu, mat, dense, skel, kw, launches, vdt):
    run_case(gpu, MATS[mat](), vdt, dense, skel, kw, launches)


def _with_empty_rows(seed=5):
    """A power-law matrix in which about a third of the rows hold no element (also the first and the last row)."""
    rows, cols, r, c, v, x = S.power_law(3000, max_len=700, mean_len=10.0, seed=seed)
    rng = np.random.default_rng(seed)
    drop = rng.uniform(size=rows) < 0.35
    drop[[0, rows - 1]] = True
    keep = ~drop[np.asarray(r, np.int64)]
    return rows, cols, r[keep], c[keep], v[keep], x


@pytest.mark.parametrize("vdt", [K.FLOAT, K.DOUBLE], ids=["fp32", "fp64"])
@pytest.mark.parametrize("dense,skel,kw", [([], "S5", {}), (SORT, "S1", {"m": 64}), ([], "S9", {"t": 4}), (D3, "S8", {"b": 128}),
                                           (SORT, "T1", {"slice": 512, "group": 256, "b": 1024}), ([], "T1", {"slice": 1024, "group": 64, "b": 512}),
                                           (SORT, "T2", {"slice": 512, "group": 16, "b": 1024}), ([], "B2", {"n": 512, "w": 8, "s": 3}),
                                           (D3, "S2", {"m": 64, "len": 1, "s": 4})],
                         ids=lambda p: p if isinstance(p, str) else None)
def test_spmv_with_empty_rows_removed(gpu, dense, skel, kw, vdt):
    """remove_empty_rows as the first operator: every kernel family writes the rows that hold elements to their
    original places (through the compaction map, alone or under a sort) and leaves the others at zero."""
    rows, cols, r, c, v, x = _with_empty_rows()
    npd = NP[vdt]
    v, x = v.astype(npd), x.astype(npd)
    y_ref, mag = oracle_y(rows, r, c, v, x)
    assert (np.bincount(np.asarray(r, np.int64), minlength=rows) == 0).sum() > 900
    m = A.Matrix.from_coo(rows, cols, r, c, v.astype(np.float64), vdt, wave=64)
    m.remove_empty_rows()
    for s, p in dense:
        m.execute_strategy(s, -1, p)
    m.execute_strategy(K.COMPRESS_NONE)
    n_sub = m.info()["n_sub"]
    for sub in range(n_sub):
        templates = SK.apply_skeleton(m, sub, skel, **kw)
    for tp in templates:
        assert all(A.template_is_supported(m, s, tp) for s in range(n_sub)), K.TEMPLATE_NAMES[tp]
        b = A.Builder(m)
        for s in range(n_sub):
            b.set_template(s, tp)
        b.compile().upload(gpu)
        print("case: empty rows", skel, kw, K.TEMPLATE_NAMES[tp], flush=True)
        y = b.spmv(x)
        assert len(y) == rows
        assert_y(y, y_ref, mag, npd, "%s %s" % (skel, K.TEMPLATE_NAMES[tp]))
        assert_y(b.spmv(x), y_ref, mag, npd, "%s second run" % skel)
        assert b.clears_y()  # the rows that were removed are stored by no kernel
        assert_y(b.spmv_device(x), y_ref, mag, npd, "%s y = NaN before the call" % skel)
        b.close()


@pytest.mark.parametrize("vdt", [K.FLOAT, K.DOUBLE], ids=["fp32", "fp64"])
def test_long_short_row_decomposition_spmv(gpu, vdt):
    """A = A_short + A_long (long_short_row_decomposition), every part through its own graph and kernel after
    remove_empty_rows, no sort anywhere: the parts' y add up to A x (their rows are disjoint)."""
    rows, cols, r, c, v, x = S.extreme_irregular(4000, 6, 2000, 3999, seed=9)
    npd = NP[vdt]
    v, x = v.astype(npd), x.astype(npd)
    y_ref, mag = oracle_y(rows, r, c, v, x)
    m = A.Matrix.from_coo(rows, cols, r, c, v.astype(np.float64), vdt, wave=64)
    parts = m.long_short_row_decomposition((0, 100))
    assert len(parts) == 2
    y = np.zeros(rows, npd)
    for part, (skel, kw) in zip(parts, (("S1", {"m": 64}), ("T1", {"slice": 1024, "group": 16, "b": 2048}))):
        part.remove_empty_rows()
        part.execute_strategy(K.COMPRESS_NONE)
        tp = SK.apply_skeleton(part, 0, skel, **kw)[0]
        b = A.Builder(part)
        b.set_template(0, tp)
        b.compile().upload(gpu)
        print("case: decomposition part", skel, K.TEMPLATE_NAMES[tp], flush=True)
        y_part = b.spmv(x)
        assert len(y_part) == rows
        y += y_part
        b.close()
    assert_y(y, y_ref, mag, npd, "long/short decomposition")


def _dense_rows():
    """12 rows x 2100 columns, row i dense in columns [37 i, 37 i + 1500 + 11 i)."""
    rng = np.random.default_rng(17)
    spans = [(37 * i, 37 * i + 1500 + 11 * i) for i in range(12)]
    r = np.concatenate([np.full(hi - lo, i) for i, (lo, hi) in enumerate(spans)])
    c = np.concatenate([np.arange(lo, hi) for lo, hi in spans])
    return 12, 2100, r, c, rng.uniform(-1, 1, len(r)), rng.uniform(-1, 1, 2100)


@pytest.mark.parametrize("vdt", [K.FLOAT, K.DOUBLE], ids=["fp32", "fp64"])
@pytest.mark.parametrize("sort", [False, True], ids=["plain", "sorted"])
@pytest.mark.parametrize("threads", [1024, 256])
def test_tile_template_in_column_run_form(gpu, vdt, sort, threads):
    """The tile kernel reading run starts and run masks instead of one column per element: same y as the CPU CSR
    oracle on dense 3 x 3 blocks (slices that cut through blocks, a last slice shorter than the others) and on a
    matrix of a few dense rows."""
    for gen, slice_width, group in ((lambda: S.fem_blocks(3000, 27, 400), 4000, 1024),
                                    (lambda: S.fem_blocks(700, 9, 60, seed=3), 500, 64),
                                    (_dense_rows, 512, 8)):
        rows, cols, r, c, v, x = gen()
        npd = NP[vdt]
        v, x = v.astype(npd), x.astype(npd)
        y_ref, mag = oracle_y(rows, r, c, v, x)
        m = A.Matrix.from_coo(rows, cols, r, c, v.astype(np.float64), vdt, wave=64)
        if sort:
            m.execute_strategy(K.DENSE_ROW_COARSE_SORT_FIXED, -1, (1,))
        m.execute_strategy(K.COMPRESS_NONE)
        tp = SK.apply_skeleton(m, 0, "T1", slice=slice_width, group=group, b=4096)[0]
        b = A.Builder(m)
        b.set_template(0, tp)
        assert b.set_column_runs(0)
        b.set_launch(0, thread_num_in_block=threads)
        b.compile().upload(gpu)
        print("case: column runs", rows, cols, len(r), slice_width, group, threads, flush=True)
        assert "col_run_mask" in b.kernel_source()
        assert_y(b.spmv(x), y_ref, mag, npd, "tile template, column runs")
        b.close()


@pytest.mark.parametrize("vdt", [K.FLOAT, K.DOUBLE], ids=["fp32", "fp64"])
@pytest.mark.parametrize("sort", [False, True], ids=["plain", "sorted"])
@pytest.mark.parametrize("runs", [False, True], ids=["columns", "runs"])
@pytest.mark.parametrize("threads", [1024, 256])
def test_tile_template_under_row_ownership(gpu, vdt, sort, runs, threads):
    """The tile kernel with whole row groups per workgroup (rows stored to y, no atomics, no clear): same y as the CPU
    CSR oracle on banded matrices of dense 3 x 3 blocks (row groups that meet two or three slices, a last slice and
    a last row group shorter than the others, rows at the ragged edge of the band that miss a slice of their group:
    lanes closed where the next row of the group has no element in the slice); y holds NaN before the call."""
    for gen, slice_width, group in ((lambda: S.fem_blocks(3000, 27, 400), 4000, 250), (lambda: S.fem_blocks(1000, 9, 60, seed=3), 500, 100),
                                    (lambda: S.fem_blocks(2000, 27, 100, seed=9), 1000, 120)):
        rows, cols, r, c, v, x = gen()
        npd = NP[vdt]
        v, x = v.astype(npd), x.astype(npd)
        y_ref, mag = oracle_y(rows, r, c, v, x)
        m = A.Matrix.from_coo(rows, cols, r, c, v.astype(np.float64), vdt, wave=64)
        if sort:
            m.execute_strategy(K.DENSE_ROW_COARSE_SORT_FIXED, -1, (1,))
        m.execute_strategy(K.COMPRESS_NONE)
        tp = SK.apply_skeleton(m, 0, "T1", slice=slice_width, group=group, b=4096)[0]
        b = A.Builder(m)
        b.set_template(0, tp)
        if runs and not b.set_column_runs(0):
            b.close()
            continue                                             # scattered columns: the column-run form is turned down
        assert b.set_row_ownership(0), (rows, slice_width, group)
        b.set_launch(0, thread_num_in_block=threads)
        b.compile().upload(gpu)
        print("case: row ownership", rows, cols, len(r), slice_width, group, threads, sort, runs, flush=True)
        assert not b.clears_y() and "cur_group" in b.kernel_source()
        assert_y(b.spmv(x), y_ref, mag, npd, "tile template, row ownership")
        assert_y(b.spmv_device(x), y_ref, mag, npd, "tile template, row ownership, y = NaN before the call")
        b.close()


@pytest.mark.parametrize("vdt", [K.FLOAT, K.DOUBLE], ids=["fp32", "fp64"])
@pytest.mark.parametrize("runs", [False, True], ids=["columns", "runs"])
@pytest.mark.parametrize("threads", [1024, 256])
def test_tile_template_with_row_blocks(gpu, vdt, runs, threads):
    """The tile kernel under row ownership with blocks of rows as pieces (the rows of a block hold the same columns;
    one set of columns and lane words, one value per row and element): same y as the CPU CSR oracle on matrices of
    dense 3 x 3, 2 x 2 and 4 x 4 blocks, with row groups that meet one, two or three windows of x, a last row group
    shorter than the others, block rows at the ragged edge of the band; y holds NaN before the call."""
    def blocks_of(height, block_rows, per_row, band, seed):
        # dense height x height blocks from the 3 x 3 generator's block pattern
        rows3, cols3, r3, c3, v3, _ = S.fem_blocks(block_rows, per_row, band, seed=seed)
        br, bc = np.asarray(r3[::9]) // 3, np.asarray(c3[::9]) // 3              # one entry per block, row-major
        blocks = np.unique(br.astype(np.int64) * block_rows + bc)
        br, bc = blocks // block_rows, blocks % block_rows
        i, j = np.meshgrid(np.arange(height), np.arange(height), indexing="ij")
        order = np.lexsort((bc, br))
        br, bc = br[order], bc[order]
        # row-major over the whole matrix: block row, row inside the block, block column, column inside the block
        rr, cc = [], []
        for q in range(height):
            rr.append(np.repeat(br * height + q, height))
            cc.append((bc[:, None] * height + np.arange(height)[None, :]).ravel())
        rr, cc = np.concatenate(rr), np.concatenate(cc)
        order = np.lexsort((cc, rr))
        rr, cc = rr[order], cc[order]
        rng = np.random.default_rng(seed)
        n = block_rows * height
        return n, n, rr.astype(np.uint64), cc.astype(np.uint64), rng.uniform(-1, 1, len(rr)), rng.uniform(-1, 1, n)
    for height, gen, slice_width, group in ((3, lambda: S.fem_blocks(3000, 27, 400), 4000, 252),
                                            (3, lambda: S.fem_blocks(1000, 9, 60, seed=3), 500, 96),
                                            (2, lambda: blocks_of(2, 3000, 27, 200, 7), 1000, 256),
                                            (4, lambda: blocks_of(4, 900, 9, 50, 8), 700, 128)):
        rows, cols, r, c, v, x = gen()
        npd = NP[vdt]
        v, x = v.astype(npd), x.astype(npd)
        y_ref, mag = oracle_y(rows, r, c, v, x)
        m = A.Matrix.from_coo(rows, cols, r, c, v.astype(np.float64), vdt, wave=64)
        m.execute_strategy(K.COMPRESS_NONE)
        tp = SK.apply_skeleton(m, 0, "T1", slice=slice_width, group=group, b=4096)[0]
        b = A.Builder(m)
        b.set_template(0, tp)
        if runs:
            assert b.set_column_runs(0)
        assert b.set_row_ownership(0), (rows, slice_width, group)
        assert b.set_row_blocks(0, height), (rows, slice_width, group, height)
        b.set_launch(0, thread_num_in_block=threads)
        b.compile().upload(gpu)
        print("case: row blocks", height, rows, cols, len(r), slice_width, group, threads, runs, flush=True)
        assert not b.clears_y() and "cell += %du" % height in b.kernel_source()
        assert_y(b.spmv(x), y_ref, mag, npd, "tile template, row blocks")
        assert_y(b.spmv_device(x), y_ref, mag, npd, "tile template, row blocks, y = NaN before the call")
        b.close()


@pytest.mark.parametrize("vdt", [K.FLOAT, K.DOUBLE], ids=["fp32", "fp64"])
@pytest.mark.parametrize("form", ["columns", "runs", "blocks"])
def test_tile_template_under_row_ownership_with_a_row_group_without_elements(gpu, vdt, form):
    """A row group that holds no element has no run under row ownership, so its owner never stores its rows: the
    builder must clear y for such a graph.  Rows 756..1007 (one whole row group of 252 rows) of a banded block matrix
    are emptied; y holds NaN before the call and must come back as A x with zeros in the emptied rows."""
    rows, cols, r, c, v, x = S.fem_blocks(3000, 27, 400)
    keep = (np.asarray(r) < 756) | (np.asarray(r) >= 1008)
    r, c, v = r[keep], c[keep], v[keep]
    npd = NP[vdt]
    v, x = v.astype(npd), x.astype(npd)
    y_ref, mag = oracle_y(rows, r, c, v, x)
    assert (y_ref[756:1008] == 0).all()
    m = A.Matrix.from_coo(rows, cols, r, c, v.astype(np.float64), vdt, wave=64)
    m.execute_strategy(K.COMPRESS_NONE)
    b = A.Builder(m)
    b.set_template(0, SK.apply_skeleton(m, 0, "T1", slice=4000, group=252, b=4096)[0])
    if form != "columns":
        assert b.set_column_runs(0)
    assert b.set_row_ownership(0)
    if form == "blocks":
        assert b.set_row_blocks(0, 3)
    assert b.describe(0)["row_groups_without_elements"] == 1 and b.clears_y()
    b.compile().upload(gpu)
    print("case: row ownership, empty row group", form, vdt, flush=True)
    y = b.spmv_device(x)
    assert not np.isnan(y).any() and (y[756:1008] == 0).all()
    assert_y(y, y_ref, mag, npd, "tile template, row ownership, a row group without elements")
    b.close()


@pytest.mark.parametrize("position", [K.END_PADDING, K.TOP_PADDING], ids=["end", "top"])
@pytest.mark.parametrize("skel,kw", [("S5", {}), ("S1", {"m": 64}), ("T1", {"slice": 1024, "group": 512, "b": 2048})],
                         ids=["S5", "S1", "T1"])
def test_spmv_of_padded_matrix(gpu, position, skel, kw):
    """total_row_level_padding to a multiple of 256 rows, then dense_col_level_padding of every third row: y has the
    padded length, holds A x in the rows of A (shifted by the rows added at the top) and zeros in the added rows."""
    rows, cols, r, c, v, x = S.power_law(3001, max_len=60, mean_len=6.0, seed=21)
    v, x = v.astype(np.float32), x.astype(np.float32)
    y_ref, mag = oracle_y(rows, r, c, v, x)
    m = A.Matrix.from_coo(rows, cols, r, c, v.astype(np.float64), K.FLOAT, wave=64)
    m.total_row_level_padding(256, position, 0 if position == K.TOP_PADDING else 7)
    padded = m.info()["rows"]
    assert padded == 3072 and m.y_rows() == padded
    lens = np.bincount(m.get_u64(-1, 103, 0)[0].astype(np.int64), minlength=padded)
    picked = np.arange(0, padded, 3)
    m.dense_col_level_padding(picked, lens[picked] + 2)
    m.execute_strategy(K.COMPRESS_NONE)
    tp = SK.apply_skeleton(m, 0, skel, **kw)[0]
    b = A.Builder(m)
    b.set_template(0, tp)
    b.compile().upload(gpu)
    print("case: padded matrix", position, skel, K.TEMPLATE_NAMES[tp], flush=True)
    y = b.spmv(x)
    b.close()
    assert len(y) == padded
    first = padded - rows if position == K.TOP_PADDING else 0
    assert_y(y[first:first + rows], y_ref, mag, np.float32, "padded matrix")
    added = np.concatenate([y[:first], y[first + rows:]])
    assert len(added) == padded - rows and not added.any()


@pytest.mark.parametrize("vdt", [K.FLOAT, K.DOUBLE], ids=["fp32", "fp64"])
@pytest.mark.parametrize("launch", [{}, {"vec_width": 2}, {"vec_width": 4, "thread_num_in_block": 128}], ids=["v1", "v2", "v4"])
def test_ell_template_with_relative_columns(gpu, vdt, launch):
    """The ELL kernel with its columns stored as 16-bit differences to the TLB number: same y as the CPU CSR oracle,
    on a stencil (rows beyond 32767) and on banded FEM blocks."""
    for gen in (lambda: S.laplacian_5pt(256), lambda: S.fem_blocks(700, 27, 200)):
        rows, cols, r, c, v, x = gen()
        npd = NP[vdt]
        v, x = v.astype(npd), x.astype(npd)
        y_ref, mag = oracle_y(rows, r, c, v, x)
        m = A.Matrix.from_coo(rows, cols, r, c, v.astype(np.float64), vdt, wave=64)
        m.execute_strategy(K.COMPRESS_NONE)
        tp = SK.apply_skeleton(m, 0, "S5")[0]
        b = A.Builder(m)
        b.set_template(0, tp)
        assert b.set_relative_columns(0)
        if launch:
            b.set_launch(0, **launch)
        b.compile().upload(gpu)
        print("case: relative columns", rows, launch, flush=True)
        assert_y(b.spmv(x), y_ref, mag, npd, "relative columns")
        b.close()
    # switched on after an upload: the arrays are uploaded again
    rows, cols, r, c, v, x = S.laplacian_5pt(200)
    npd = NP[vdt]
    v, x = v.astype(npd), x.astype(npd)
    y_ref, mag = oracle_y(rows, r, c, v, x)
    m = A.Matrix.from_coo(rows, cols, r, c, v.astype(np.float64), vdt, wave=64)
    m.execute_strategy(K.COMPRESS_NONE)
    b = A.Builder(m)
    b.set_template(0, SK.apply_skeleton(m, 0, "S5")[0])
    b.compile().upload(gpu)
    assert_y(b.spmv(x), y_ref, mag, npd, "32-bit columns")
    assert b.set_relative_columns(0)
    b.compile().upload(gpu)
    assert_y(b.spmv(x), y_ref, mag, npd, "relative columns after an upload")
    b.close()


@pytest.mark.parametrize("vdt", [K.FLOAT, K.DOUBLE], ids=["fp32", "fp64"])
@pytest.mark.parametrize("launch", [{}, {"vec_width": 2}, {"vec_width": 4, "thread_num_in_block": 128}], ids=["v1", "v2", "v4"])
def test_ell_template_with_diagonal_columns(gpu, vdt, launch):
    """The ELL kernel in diagonal form (columns computed from the slot's diagonal, no column array) on 5-point
    stencils of two sizes, also switched on after an upload and on top of relative columns."""
    for grid, order in ((256, "dia"), (131, "rel+dia"), (200, "late")):
        rows, cols, r, c, v, x = S.laplacian_5pt(grid)
        npd = NP[vdt]
        v, x = v.astype(npd), x.astype(npd)
        y_ref, mag = oracle_y(rows, r, c, v, x)
        m = A.Matrix.from_coo(rows, cols, r, c, v.astype(np.float64), vdt, wave=64)
        m.execute_strategy(K.COMPRESS_NONE)
        b = A.Builder(m)
        b.set_template(0, SK.apply_skeleton(m, 0, "S5")[0])
        if order == "late":
            b.compile().upload(gpu)
            assert_y(b.spmv(x), y_ref, mag, npd, "32-bit columns")
        if order == "rel+dia":
            assert b.set_relative_columns(0)
        assert b.set_diagonal_columns(0)
        if launch:
            b.set_launch(0, **launch)
        b.compile().upload(gpu)
        print("case: diagonal columns", grid, order, launch, flush=True)
        assert_y(b.spmv(x), y_ref, mag, npd, "diagonal columns " + order)
        b.close()


def test_golden_case_formats_run_on_gpu(gpu):
    """The small fixtures used for the bit-exact format parity, rebuilt at wave 64 and executed."""
    for case in cases.FORMAT_CASES + cases.EXTENSION_CASES:
        _, mname, dense, skel, kw = case
        gen, vdt = cases.MATRICES[mname]
        kw = {k: v for k, v in kw.items() if k != "wave"}
        run_case(gpu, gen(), vdt, dense, skel, kw)


# ---- full-size configuration 2 (the benchmark workload): size-independent properties ------------
@pytest.fixture(scope="module")
def laplacian_full(gpu):
    rows, cols, r, c, v, x = S.laplacian_5pt(2048)
    m = A.Matrix.from_coo(rows, cols, r, c, v.astype(np.float64), K.FLOAT, wave=64)
    m.execute_strategy(K.COMPRESS_NONE)
    SK.apply_skeleton(m, 0, "S5")
    b = A.Builder(m)
    b.set_template(0, K.DIRECT_ATOM_TEMPLATE_WARP_BLOCK_COMPRESS)
    b.compile().upload(gpu)
    yield b, (rows, cols, r, c, v, x)
    b.close()


def test_full_laplacian_matches_oracle(laplacian_full):
    b, (rows, cols, r, c, v, x) = laplacian_full
    assert rows == 4194304 and len(r) == 20963328
    y_ref, mag = oracle_y(rows, r, c, v, x)
    assert_y(b.spmv(x), y_ref, mag, np.float32, "C2 ELL")
    assert not b.clears_y()  # direct stores, every row has elements: the SpMV is one kernel
    assert_y(b.spmv_device(x), y_ref, mag, np.float32, "C2 ELL (y = NaN before the call)")


def test_full_laplacian_closed_form_and_linearity(laplacian_full):
    b, (rows, cols, r, c, v, x) = laplacian_full
    g = 2048
    y = b.spmv(np.ones(cols, np.float32)).reshape(g, g)
    assert np.all(y[1:-1, 1:-1] == 0) and np.all(y[0, 1:-1] == 1) and y[0, 0] == 2
    x2 = np.random.default_rng(5).uniform(-1, 1, cols).astype(np.float32)
    y1, y2 = b.spmv(x).astype(np.float64), b.spmv(x2).astype(np.float64)
    y3 = b.spmv((2 * x - 3 * x2).astype(np.float32)).astype(np.float64)
    assert np.max(np.abs(y3 - (2 * y1 - 3 * y2))) <= 64 * np.finfo(np.float32).eps * 8 * 5


# ---- full-size configurations 3, 4 and 5 through the graphs the search returns for them -----------------------
def _full_c3():
    return S.power_law(), K.FLOAT, (48, "T1", {}, 1024, False), ("T2", {"slice": 16384, "group": 4096}, 1024)


def _full_c4():
    return S.fem_blocks(), K.DOUBLE, None, ("T1", {"slice": 16384, "group": 4092}, 1024)


def _full_c5():
    return (S.extreme_irregular(target_nnz=60_000_000), K.DOUBLE, (16, "T1", {"slice": 16384, "group": 4096}, 1024, False),
            ("T2", {"slice": 16384, "group": 4096}, 1024))


@pytest.mark.parametrize("make", [_full_c3, _full_c4, _full_c5], ids=["C3", "C4", "C5"])
def test_full_size_tile_and_product_bin_graphs(gpu, make, capsys):
    """The benchmark matrices at their real size through the graphs the search returns for them -- C3 (2 M rows,
    32 M elements, fp32) and C5 (8 M rows, 60 M elements, fp64): coarse sort, two row strips, the tile kernel on the
    long rows and the product-bin kernel on the others; C4 (1 M rows, 81 M elements, fp64): the tile kernel on the
    whole matrix, column-run form under row ownership with blocks of three rows as pieces.  y against the CPU CSR oracle, and two properties that do not depend on the
    size: x = 1 gives the row sums of the values, and A (2 x - 3 z) = 2 A x - 3 A z within the rounding of the row.
    Most of a case's time is the generation of the matrix: the phases are announced past the capture."""
    def say(what):
        with capsys.disabled():
            print("[full size %s] %s" % (make.__name__[-2:], what), flush=True)
    say("generating the matrix")
    (rows, cols, r, c, v, x), vdt, long_strip, (skel, kw, threads) = make()
    npd = NP[vdt]
    v, x = v.astype(npd), x.astype(npd)
    say("%d rows, %d elements: building the format" % (rows, len(r)))
    m = A.Matrix.from_coo(rows, cols, r, c, v.astype(np.float64), vdt, wave=64)
    if long_strip:
        low = long_strip[0]
        m.execute_strategy(K.DENSE_ROW_COARSE_SORT_FIXED, -1, (1,))
        m.execute_strategy(K.DENSE_ROW_DIV_ACC_TO_EXPONENTIAL_INCREASE_ROW_NNZ, -1, (low, low, 2, 0))
    m.execute_strategy(K.COMPRESS_NONE)
    strips = ([long_strip[1:4]] if long_strip else []) + [(skel, kw, threads)]
    assert m.info()["n_sub"] == len(strips)
    chosen = [SK.apply_skeleton(m, s, sk, **k)[0] for s, (sk, k, _) in enumerate(strips)]
    b = A.Builder(m)
    for s, tp in enumerate(chosen):
        b.set_template(s, tp)
        b.set_launch(s, thread_num_in_block=strips[s][2])
    if not long_strip:
        # C4, dense 3 x 3 blocks: column runs, whole row groups per workgroup, blocks of three rows as pieces
        assert b.set_column_runs(0) and b.set_row_ownership(0) and b.set_row_blocks(0, 3)
    b.set_serial_launch(True)
    b.compile().upload(gpu)
    say("on the device: y against the oracle, row sums, linearity")
    y_ref, mag = oracle_y(rows, r, c, v, x)
    y1 = b.spmv(x)
    assert_y(y1, y_ref, mag, npd, make.__name__)
    # every row is stored once in all three graphs (finish kernels, or the row groups' owners): no clear of y
    assert not b.clears_y()
    assert_y(b.spmv_device(x), y_ref, mag, npd, make.__name__ + " (y = NaN before the call)")
    eps = np.finfo(npd).eps
    off = np.concatenate([[0], np.cumsum(np.bincount(np.asarray(r, np.int64), minlength=rows))])
    row_sum = np.add.reduceat(v.astype(np.float64), off[:-1])
    row_mag = np.add.reduceat(np.abs(v).astype(np.float64), off[:-1])
    y_ones = b.spmv(np.ones(cols, npd)).astype(np.float64)
    assert np.all(np.abs(y_ones - row_sum) <= 64 * eps * row_mag + 1e-300)
    z = np.random.default_rng(5).uniform(-1, 1, cols).astype(npd)
    y2 = b.spmv(z).astype(np.float64)
    y3 = b.spmv((2 * x - 3 * z).astype(npd)).astype(np.float64)
    assert np.all(np.abs(y3 - (2 * y1.astype(np.float64) - 3 * y2)) <= 64 * eps * 8 * row_mag + 1e-300)
    b.close()


@pytest.mark.parametrize("vdt", [K.FLOAT, K.DOUBLE], ids=["fp32", "fp64"])
def test_finish_of_a_tile_strip_carried_by_the_next_strips_kernel(gpu, vdt):
    """Coarse sort, a tile strip (row sums through a scratch vector and a finish kernel) in front of a product-bin
    strip, kernels one after the other: the finish kernel is not launched, the first workgroups of the product-bin
    template's first kernel move the rows to y -- or, where both strips have workgroups of the same size, the two
    strips' first kernels are one launch and the product-bin template's second kernel moves the rows.  y against the
    oracle with the hand-over on and off, fused and not, on y = NaN, call after call (the scratch vector is left
    cleared), after measurements of one strip alone (which use the strip's own kernels), and on concurrent streams
    (no hand-over)."""
    rows, cols, r, c, v, x = S.power_law(30000, max_len=4000, mean_len=12.0, seed=11)
    npd = NP[vdt]
    v, x = v.astype(npd), x.astype(npd)
    m = A.Matrix.from_coo(rows, cols, r, c, v.astype(np.float64), vdt, wave=64)
    m.execute_strategy(K.DENSE_ROW_COARSE_SORT_FIXED, -1, (1,))
    m.execute_strategy(K.DENSE_ROW_DIV_ACC_TO_EXPONENTIAL_INCREASE_ROW_NNZ, -1, (16, 16, 2, 0))
    m.execute_strategy(K.COMPRESS_NONE)
    assert m.info()["n_sub"] == 2
    b = A.Builder(m)
    b.set_template(0, SK.apply_skeleton(m, 0, "T1", slice=1024, group=512, b=2048)[0])
    b.set_template(1, SK.apply_skeleton(m, 1, "T2", slice=1024, group=4096, b=2048)[0])
    y_ref, mag = oracle_y(rows, r, c, v, x)
    z = np.random.default_rng(2).uniform(-1, 1, cols).astype(npd)
    z_ref, z_mag = oracle_y(rows, r, c, v, z)
    assert b.finish_carrier(0) == -1                             # concurrent streams: every strip its own kernels
    b.set_serial_launch(True)
    assert b.finish_carrier(0) == 1 and b.finish_carrier(1) == -1
    for threads in (256, 1024):
        b.set_launch(1, thread_num_in_block=threads)
        b.compile().upload(gpu)
        src = b.kernel_source()
        assert "carried_sum" in src and "spmv_0_finish" in src and not b.clears_y()
        # workgroups of the same size in both strips (the tile strip has 1024 threads): one launch for both first kernels
        assert b.launch_is_fused(0) == (threads == 1024) and ("fused_on" in src) == (threads == 1024)
        print("case: carried finish, %d threads" % threads, flush=True)
        assert_y(b.spmv_device(x), y_ref, mag, npd, "carried finish, y = NaN before the call")
        if threads == 1024:
            b.set_fuse_launches(False)
            b.compile().upload(gpu)
            assert not b.launch_is_fused(0) and b.finish_carrier(0) == 1 and "fused_on" not in b.kernel_source()
            assert_y(b.spmv_device(x), y_ref, mag, npd, "carried finish, launches not fused")
            b.set_fuse_launches(True)
            b.compile().upload(gpu)
        assert_y(b.spmv_device(z), z_ref, z_mag, npd, "carried finish, second call with another x")
        assert_y(b.spmv_device(x, no_alloc=True), y_ref, mag, npd, "carried finish, static scratch")
        # one strip alone: its own kernels (the tile strip its finish kernel, the product-bin kernel nothing to carry)
        for sub in (0, 1):
            assert b.time_sub_matrix(sub, 3)[0] > 0
        assert b.time_sub_matrix_pass(1, 1, 3) > 0 and b.time_sub_matrix_pass(0, 1, 3) > 0 and b.time_sub_matrix_pass(0, 2, 3) > 0
        assert_y(b.spmv_device(x), y_ref, mag, npd, "carried finish, after the per-strip measurements")
        ms, gf = b.time(5)
        assert ms > 0
        assert_y(b.spmv_device(x), y_ref, mag, npd, "carried finish, after the timing loop")
    b.set_finish_carry(False)
    assert b.finish_carrier(0) == -1
    b.compile().upload(gpu)
    assert "carried_sum" not in b.kernel_source()
    assert_y(b.spmv_device(x), y_ref, mag, npd, "finish kernel of its own")
    b.set_finish_carry(True).set_serial_launch(False)
    b.compile().upload(gpu)
    assert "carried_sum" not in b.kernel_source()
    assert_y(b.spmv_device(x), y_ref, mag, npd, "concurrent streams")
    b.close()
    # rows that already come longest first: the sort leaves them where they are, the tile strip's places in y are
    # a closed form (no array is passed) and the carrying kernel computes them
    order = np.argsort(-np.bincount(np.asarray(r, np.int64), minlength=rows), kind="stable")
    new_row = np.empty(rows, np.int64)
    new_row[order] = np.arange(rows)
    r2 = new_row[np.asarray(r, np.int64)]
    keep = np.lexsort((np.asarray(c, np.int64), r2))
    r2, c2, v2 = r2[keep].astype(np.uint64), np.asarray(c)[keep], v[keep]
    y_ref, mag = oracle_y(rows, r2, c2, v2, x)
    m = A.Matrix.from_coo(rows, cols, r2, c2, v2.astype(np.float64), vdt, wave=64)
    m.execute_strategy(K.DENSE_ROW_COARSE_SORT_FIXED, -1, (1,))
    m.execute_strategy(K.DENSE_ROW_DIV_ACC_TO_EXPONENTIAL_INCREASE_ROW_NNZ, -1, (16, 16, 2, 0))
    m.execute_strategy(K.COMPRESS_NONE)
    b = A.Builder(m)
    b.set_template(0, SK.apply_skeleton(m, 0, "T1", slice=1024, group=512, b=2048)[0])
    b.set_template(1, SK.apply_skeleton(m, 1, "T2", slice=1024, group=4096, b=2048)[0])
    b.set_serial_launch(True)
    b.compile().upload(gpu)
    src = b.kernel_source()
    print("case: carried finish, rows already sorted; places passed as an array:", "carried_place" in src, flush=True)
    assert b.finish_carrier(0) == 1 and "carried_sum" in src
    assert_y(b.spmv_device(x), y_ref, mag, npd, "carried finish, rows already in sorted order")
    assert_y(b.spmv_device(z), *oracle_y(rows, r2, c2, v2, z), npd, "carried finish, rows already in sorted order, second call")
    b.close()


def test_empty_template_launches_nothing_and_leaves_zeros(gpu):
    """A graph whose second strip holds only explicit zeros and has EMPTY_TEMPLATE: y = A x with zeros in the rows of
    that strip, from a y full of NaN."""
    from test_format_invariants import _matrix_with_a_strip_of_zeros
    m, r, c, v, x = _matrix_with_a_strip_of_zeros()
    for sub in (0, 1):
        SK.apply_skeleton(m, sub, "S1", m=64)
    b = A.Builder(m)
    b.set_template(0, K.DIRECT_ATOM_TEMPLATE_WARP_COMPRESS)
    b.set_template(1, K.EMPTY_TEMPLATE)
    b.compile().upload(gpu)
    y_ref, mag = oracle_y(300, r.astype(np.uint64), c.astype(np.uint64), v, x)
    y = b.spmv_device(x)
    assert (y[200:] == 0).all()
    assert_y(y, y_ref, mag, np.float64, "EMPTY_TEMPLATE on the strip of zeros")
    assert_y(b.spmv(x), y_ref, mag, np.float64, "EMPTY_TEMPLATE, host vectors")
    b.close()


def test_missing_library_is_an_error_not_a_fallback():
    """The product has no CPU execution path: without the HIP library nothing runs."""
    import importlib
    import alphasparse_amd._capi as capi
    saved, capi._lib = capi._lib, None
    path, capi.LIB_PATH = capi.LIB_PATH, capi.LIB_PATH + ".absent"
    try:
        with pytest.raises(capi.AlphaSparseError, match="no CPU fallback"):
            capi.lib()
    finally:
        capi.LIB_PATH, capi._lib = path, saved
