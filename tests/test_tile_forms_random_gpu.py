"""Seeded random cases through the forms of the tile template and the carried finish: banded matrices of dense h x h
blocks (h = 1..4) with random band, tile and launch parameters through column runs, row ownership (windows of x) and
row blocks, and power-law matrices through a sorted tile strip + a product-bin strip whose first kernel carries the
tile strip's finish.  y against the CPU CSR oracle, with y = NaN before every call."""
import numpy as np
import pytest

import spmv_oracle as O
import alphasparse_amd as A
from alphasparse_amd import _capi as K
from alphasparse_amd import skeletons as SK
from alphasparse_amd import synthetic as S

pytestmark = pytest.mark.gpu


def _block_matrix(rng, h, block_rows, per_row, band):
    """Dense h x h blocks: per_row block columns within +-band of the diagonal (clipped to the matrix) + the diagonal."""
    br = np.repeat(np.arange(block_rows), per_row)
    bc = np.clip(br + rng.integers(-band, band + 1, len(br)), 0, block_rows - 1)
    br, bc = np.concatenate([br, np.arange(block_rows)]), np.concatenate([bc, np.arange(block_rows)])
    blocks = np.unique(br.astype(np.int64) * block_rows + bc)
    br, bc = blocks // block_rows, blocks % block_rows
    rr = np.concatenate([np.repeat(br * h + q, h) for q in range(h)])
    cc = np.concatenate([(bc[:, None] * h + np.arange(h)[None, :]).ravel() for _ in range(h)])
    order = np.lexsort((cc, rr))
    n = block_rows * h
    return n, n, rr[order].astype(np.uint64), cc[order].astype(np.uint64), rng.uniform(-1, 1, len(rr)), rng.uniform(-1, 1, n)


def _check(b, x, y_ref, mag, npd, what):
    for y in (b.spmv(x), b.spmv_device(x)):
        rel, ratio, tol = O.check_y(y, y_ref, mag, npd)
        assert rel <= tol and ratio <= 1.0, "%s: rel L2 %.3e (tolerance %.0e), per-row ratio %.2f" % (what, rel, tol, ratio)


def test_random_block_matrices_through_the_tile_forms(gpu):
    owned = blocked = 0
    for case in range(36):
        rng = np.random.default_rng(9000 + case)
        h = int(rng.choice([1, 2, 3, 4]))
        block_rows, per_row, band = int(rng.integers(200, 5000)), int(rng.integers(2, 28)), int(rng.integers(5, 600))
        slice_width, group = int(rng.choice([128, 256, 500, 1000, 2048])), int(rng.choice([24, 48, 96, 252, 516]))
        threads = int(rng.choice([256, 512, 1024]))
        vdt = K.DOUBLE if rng.integers(2) else K.FLOAT
        runs, sort = bool(rng.integers(2)), bool(rng.integers(4) == 0)
        rows, cols, r, c, v, x = _block_matrix(rng, h, block_rows, per_row, band)
        npd = np.float64 if vdt == K.DOUBLE else np.float32
        v, x = v.astype(npd), x.astype(npd)
        what = "case %d: blocks of %d, %d block rows, %d per row, band %d, slice %d, group %d, %d threads, %s, runs %s, sort %s" % (
            case, h, block_rows, per_row, band, slice_width, group, threads, npd.__name__, runs, sort)
        print(what, flush=True)
        m = A.Matrix.from_coo(rows, cols, r, c, v.astype(np.float64), vdt, wave=64)
        if sort:
            m.execute_strategy(K.DENSE_ROW_COARSE_SORT_FIXED, -1, (1,))
        m.execute_strategy(K.COMPRESS_NONE)
        tp = SK.apply_skeleton(m, 0, "T1", slice=slice_width, group=group, b=int(rng.choice([256, 1000, 4096])))[0]
        b = A.Builder(m)
        b.set_template(0, tp)
        if runs:
            b.set_column_runs(0)
        if b.set_row_ownership(0):
            owned += 1
            if h > 1 and not sort and b.set_row_blocks(0, h):
                blocked += 1
        b.set_launch(0, thread_num_in_block=threads)
        b.compile().upload(gpu)
        y_ref, mag = O.spmv_csr(O.coo_to_csr(rows, r), c.astype(np.uint32), v, x)
        _check(b, x, y_ref, mag, npd, what)
        b.close()
    assert owned >= 8 and blocked >= 4       # the seeds reach the forms


def test_random_two_strip_graphs_with_the_finish_carried(gpu):
    for case in range(14):
        rng = np.random.default_rng(300 + case)
        rows, max_len, mean = int(rng.integers(2000, 120000)), int(rng.integers(200, 8000)), float(rng.uniform(4, 20))
        cut = int(rng.choice([16, 64]))
        vdt = K.DOUBLE if rng.integers(2) else K.FLOAT
        s1, g1 = int(rng.choice([512, 1024, 4096])), int(rng.choice([128, 512, 2048]))
        s2, g2 = int(rng.choice([512, 1024, 4096])), int(rng.choice([1024, 4096, 65536]))
        t1, t2 = int(rng.choice([512, 1024])), int(rng.choice([256, 512, 1024]))
        what = "case %d: %d rows, longest %d, mean %.1f, cut at %d, tile %d x %d @%d, product-bin %d x %d @%d" % (
            case, rows, max_len, mean, cut, g1, s1, t1, g2, s2, t2)
        print(what, flush=True)
        rows, cols, r, c, v, x = S.power_law(rows, max_len=min(max_len, rows), mean_len=mean, seed=300 + case)
        npd = np.float64 if vdt == K.DOUBLE else np.float32
        v, x = v.astype(npd), x.astype(npd)
        m = A.Matrix.from_coo(rows, cols, r, c, v.astype(np.float64), vdt, wave=64)
        m.execute_strategy(K.DENSE_ROW_COARSE_SORT_FIXED, -1, (1,))
        m.execute_strategy(K.DENSE_ROW_DIV_ACC_TO_EXPONENTIAL_INCREASE_ROW_NNZ, -1, (cut, cut, 2, 0))
        m.execute_strategy(K.COMPRESS_NONE)
        if m.info()["n_sub"] != 2:
            continue
        b = A.Builder(m)
        b.set_template(0, SK.apply_skeleton(m, 0, "T1", slice=s1, group=g1, b=2048)[0])
        b.set_template(1, SK.apply_skeleton(m, 1, "T2", slice=s2, group=g2, b=2048)[0])
        b.set_launch(0, thread_num_in_block=t1)
        b.set_launch(1, thread_num_in_block=t2)
        b.set_serial_launch(True)
        assert b.finish_carrier(0) == 1
        b.compile().upload(gpu)
        y_ref, mag = O.spmv_csr(O.coo_to_csr(rows, r), c.astype(np.uint32), v, x)
        _check(b, x, y_ref, mag, npd, what)
        b.time(3)
        _check(b, x, y_ref, mag, npd, what + ", after a timing loop")
        b.close()


def test_random_two_strip_graphs_in_one_launch(gpu):
    """The same shape of graph with workgroups of one size in both strips, so that the tile trips and the first pass of
    the product-bin template are one launch and the second pass carries the tile strip's finish.  Rows of two classes
    of length in random proportion: where the short rows are the minority the product-bin template keeps the rows of y
    by rank (sparse form) instead of a rank for every row of y; rows without a short neighbour, bands of y that the
    strip does not touch, more tile trips than first-pass trips and the other way round all come up.  Fused and not
    fused against the oracle, y = NaN before every call, again after a timing loop."""
    import cases
    fused = sparse = 0
    for case in range(18):
        rng = np.random.default_rng(700 + case)
        rows = int(rng.integers(3000, 90000))
        share_short = float(rng.choice([0.15, 0.4, 0.7, 0.95]))
        short = rng.integers(1, int(rng.choice([4, 9, 15])), rows)
        long_ = rng.integers(16, int(rng.choice([64, 400, 2500])), rows)
        lens = np.where(rng.random(rows) < share_short, short, long_)
        if lens.sum() > 6_000_000:      # keep the case small: shorter long rows, still 16 or more elements
            lens = np.where(lens >= 16, np.maximum(16, lens * 6_000_000 // lens.sum()), lens)
        cols = int(rng.choice([rows, 2 * rows, 70000]))
        vdt = K.DOUBLE if rng.integers(2) else K.FLOAT
        s1, g1 = int(rng.choice([512, 1024, 4096])), int(rng.choice([128, 512, 2048]))
        s2, g2 = int(rng.choice([512, 1024, 4096])), int(rng.choice([256, 1024, 4096]))
        threads = int(rng.choice([256, 512, 1024]))
        what = "case %d: %d rows x %d columns, %.0f %% short rows, tile %d x %d, product-bin %d x %d, %d threads, %s" % (
            case, rows, cols, 100 * share_short, g1, s1, g2, s2, threads, "fp64" if vdt == K.DOUBLE else "fp32")
        print(what, flush=True)
        rows, cols, r, c, v, x = cases._steps(lens, max(cols, int(lens.max())), 700 + case)
        npd = np.float64 if vdt == K.DOUBLE else np.float32
        v, x = v.astype(npd), x.astype(npd)
        m = A.Matrix.from_coo(rows, cols, r, c, v.astype(np.float64), vdt, wave=64)
        m.execute_strategy(K.DENSE_ROW_COARSE_SORT_FIXED, -1, (1,))
        m.execute_strategy(K.DENSE_ROW_DIV_ACC_TO_EXPONENTIAL_INCREASE_ROW_NNZ, -1, (16, 16, 2, 0))
        m.execute_strategy(K.COMPRESS_NONE)
        assert m.info()["n_sub"] == 2
        b = A.Builder(m)
        b.set_template(0, SK.apply_skeleton(m, 0, "T1", slice=s1, group=g1, b=2048)[0])
        b.set_template(1, SK.apply_skeleton(m, 1, "T2", slice=s2, group=g2, b=2048)[0])
        b.set_launch(0, thread_num_in_block=threads)
        b.set_launch(1, thread_num_in_block=threads)
        b.set_serial_launch(True)
        b.compile().upload(gpu)
        assert b.launch_is_fused(0) and b.finish_carrier(0) == 1
        fused += 1
        sparse += b.describe(1)["dense_y"] == 0
        y_ref, mag = O.spmv_csr(O.coo_to_csr(rows, r), c.astype(np.uint32), v, x)
        _check(b, x, y_ref, mag, npd, what)
        b.time(3)
        _check(b, x, y_ref, mag, npd, what + ", after a timing loop")
        b.set_fuse_launches(False)
        b.compile().upload(gpu)
        assert not b.launch_is_fused(0) and b.finish_carrier(0) == 1
        _check(b, x, y_ref, mag, npd, what + ", launches not fused")
        b.close()
    assert fused == 18 and sparse >= 3, (fused, sparse)
