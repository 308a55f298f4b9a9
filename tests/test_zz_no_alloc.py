"""as_builder_spmv_device_no_alloc: the SpMV entry point that allocates nothing (its kernels' scratch arrays are
pieces of the library's static device array) against as_builder_spmv_device on the same builder, and against the
CPU CSR oracle.  Two calls in a row on graphs that use scratch, the second on a smaller matrix; a graph that needs
more scratch than the array holds is rejected."""
import numpy as np
import pytest

import spmv_oracle as O
import alphasparse_amd as A
from alphasparse_amd import _capi as K
from alphasparse_amd import skeletons as SK
from alphasparse_amd import synthetic as S

pytestmark = pytest.mark.gpu

NP = {K.FLOAT: np.float32, K.DOUBLE: np.float64}
STATIC_SCRATCH_BYTES = 64 << 20


def _two_strip_builder(gpu, rows, max_len, seed, vdt):
    """Coarse sort, rows of 16 or more elements through the tile template (scratch: the strip's row sums, must start
    at zero), the others through the product-bin template (scratch: the products): the shape of the graphs the
    search returns for the power-law and the extremely irregular workloads."""
    gen = S.power_law(rows, max_len=max_len, mean_len=12.0, seed=seed)
    rows, cols, r, c, v, x = gen
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
    b.set_serial_launch(True)
    b.compile().upload(gpu)
    y_ref, mag = O.spmv_csr(O.coo_to_csr(rows, r), c.astype(np.uint32), v, x)
    return b, x, y_ref, mag, npd


def _check(y, y_ref, mag, npd, what):
    rel, ratio, tol = O.check_y(y, y_ref, mag, npd)
    assert rel <= tol and ratio <= 1.0, "%s: rel L2 %.3e (tolerance %.0e), per-row ratio %.2f" % (what, rel, tol, ratio)


@pytest.mark.parametrize("vdt", [K.FLOAT, K.DOUBLE], ids=["fp32", "fp64"])
def test_no_alloc_entry_point_matches_the_allocating_one(gpu, vdt):
    big = _two_strip_builder(gpu, 20000, 3000, 31, vdt)
    small = _two_strip_builder(gpu, 3000, 700, 32, vdt)
    for name, (b, x, y_ref, mag, npd) in (("first call", big), ("second call, smaller matrix", small), ("third call", big)):
        print("case: no-alloc", name, b.rows, flush=True)
        need = b.static_scratch_need()
        assert 0 < need <= STATIC_SCRATCH_BYTES
        y_alloc = b.spmv_device(x)
        y_static = b.spmv_device(x, no_alloc=True)
        _check(y_alloc, y_ref, mag, npd, name + ": as_builder_spmv_device against the oracle")
        _check(y_static, y_ref, mag, npd, name + ": as_builder_spmv_device_no_alloc against the oracle")
        # against each other, to the bar of the y parity (the row sums of the tile strip are added in LDS in an
        # order that differs from launch to launch, so fp sums are not bit-reproducible between two launches)
        _check(y_static, y_alloc.astype(np.float64), mag, npd, name + ": the two entry points against each other")
        # the product-bin strip adds in a fixed order: its rows are bit-identical
        assert np.mean(y_static == y_alloc) > 0.5
    for b, *_ in (big, small):
        b.close()


def test_no_alloc_entry_point_rejects_what_does_not_fit(gpu):
    """9.4 M fp64 products = 75 MB of scratch for the product-bin template: more than the static array."""
    rows, cols, r, c, v, x = S.uniform_rows(1 << 20, 9, seed=4, dtype=np.float64)
    m = A.Matrix.from_coo(rows, cols, r, c, v.astype(np.float64), K.DOUBLE, wave=64)
    m.execute_strategy(K.COMPRESS_NONE)
    b = A.Builder(m)
    b.set_template(0, SK.apply_skeleton(m, 0, "T2", slice=16384, group=8192, b=8192)[0])
    b.compile().upload(gpu)
    assert b.static_scratch_need() > STATIC_SCRATCH_BYTES
    with pytest.raises(K.AlphaSparseError, match="static scratch array"):
        b.spmv_device(x, no_alloc=True)
    y_ref, mag = O.spmv_csr(O.coo_to_csr(rows, r), c.astype(np.uint32), v, x)
    _check(b.spmv_device(x), y_ref, mag, np.float64, "as_builder_spmv_device still runs it")
    b.close()


def test_no_alloc_entry_point_needs_an_uploaded_builder(gpu):
    rows, cols, r, c, v, x = S.laplacian_5pt(64)
    m = A.Matrix.from_coo(rows, cols, r, c, v.astype(np.float64), K.FLOAT, wave=64)
    m.execute_strategy(K.COMPRESS_NONE)
    b = A.Builder(m)
    b.set_template(0, SK.apply_skeleton(m, 0, "S5")[0])
    b.compile().upload(gpu)
    x = x.astype(np.float32)
    y_ref, mag = O.spmv_csr(O.coo_to_csr(rows, r), c.astype(np.uint32), v.astype(np.float32), x)
    assert b.static_scratch_need() == 0
    _check(b.spmv_device(x, no_alloc=True), y_ref, mag, np.float32, "a graph without scratch")
    b.set_launch(0, thread_num_in_block=128)  # changes the module: it would have to be compiled and loaded again
    with pytest.raises(K.AlphaSparseError, match="upload"):
        b.spmv_device(x, no_alloc=True)
    b.close()
