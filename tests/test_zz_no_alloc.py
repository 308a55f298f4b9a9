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


def _two_strip_builder(gpu, rows, max_len, seed, vdt, serial=True, carry=True):
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
    b.set_serial_launch(serial)
    b.set_finish_carry(carry)
    b.compile().upload(gpu)
    b.coo = (rows, r, c, v)       # for callers that check other vectors x
    y_ref, mag = O.spmv_csr(O.coo_to_csr(rows, r), c.astype(np.uint32), v, x)
    return b, x, y_ref, mag, npd


def _check(y, y_ref, mag, npd, what):
    rel, ratio, tol = O.check_y(y, y_ref, mag, npd)
    assert rel <= tol and ratio <= 1.0, "%s: rel L2 %.3e (tolerance %.0e), per-row ratio %.2f" % (what, rel, tol, ratio)


@pytest.mark.parametrize("vdt", [K.FLOAT, K.DOUBLE], ids=["fp32", "fp64"])
@pytest.mark.parametrize("serial,carry", [(True, True), (True, False), (False, True)],
                         ids=["serial_carried", "serial_own_finish", "concurrent_streams"])
def test_no_alloc_entry_point_matches_the_allocating_one(gpu, vdt, serial, carry):
    big = _two_strip_builder(gpu, 20000, 3000, 31, vdt, serial, carry)
    small = _two_strip_builder(gpu, 3000, 700, 32, vdt, serial, carry)
    for name, (b, x, y_ref, mag, npd) in (("first call", big), ("second call, smaller matrix", small), ("third call", big)):
        print("case: no-alloc", name, b.rows, "serial" if serial else "concurrent", "carried" if carry else "own finish", flush=True)
        need = b.static_scratch_need()
        assert 0 < need <= STATIC_SCRATCH_BYTES
        # both strips have workgroups of 1024 threads: with the carried finish their first kernels are one launch
        assert b.launch_is_fused(0) == (serial and carry)
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


def test_no_alloc_call_leaves_device_memory_as_it_was(gpu):
    """Free device memory (hipMemGetInfo) is the same before and after calls of the entry point that allocates
    nothing, on buffers allocated beforehand."""
    b, x, y_ref, mag, npd = _two_strip_builder(gpu, 20000, 3000, 31, K.DOUBLE)
    dx, dy = A.DeviceArray(x), A.DeviceArray(np.full(b.rows, np.nan, npd))
    b.spmv_device_async(dx, dy, None, no_alloc=True)       # first call: nothing left to set up afterwards
    b.sync()
    before = A.device_memory_free_bytes()
    for _ in range(5):
        b.spmv_device_async(dx, dy, None, no_alloc=True)
    b.sync()
    assert A.device_memory_free_bytes() == before
    _check(dy.get(), y_ref, mag, npd, "no-alloc calls on buffers of the caller")
    dx.free()
    dy.free()
    b.close()


@pytest.mark.parametrize("vdt", [K.FLOAT, K.DOUBLE], ids=["fp32", "fp64"])
def test_no_alloc_async_call_replayed_as_a_hip_graph(gpu, vdt):
    """as_builder_spmv_device_no_alloc_async recorded by a stream capture (it allocates nothing, waits for nothing and
    clears with fill kernels, not memset nodes) and replayed three times with a different x each time, the program's
    own eager work and waits in between: every replay must give A x for the x of that replay.  Two graphs: the
    two-strip graph (scratch of both strips in the static array, the tile strip's piece cleared by the fill kernel,
    finish carried), the same with the strips on concurrent streams (the capture records the fork and the join) and
    a graph that starts with a clear of y."""
    npd = NP[vdt]
    cases = [_two_strip_builder(gpu, 20000, 3000, 31, vdt),
             # the strips' kernels on streams of their own, which fork from and join the capturing stream by events
             _two_strip_builder(gpu, 12000, 2000, 33, vdt, serial=False)]
    rows, cols, r, c, v, x = S.power_law(8000, max_len=900, mean_len=20.0, seed=5)
    m = A.Matrix.from_coo(rows, cols, r, c, v.astype(np.float64), vdt, wave=64)
    m.execute_strategy(K.COMPRESS_NONE)
    bt = A.Builder(m)
    bt.set_template(0, SK.apply_skeleton(m, 0, "T1", slice=1024, group=512, b=2048)[0])
    bt.compile().upload(gpu)
    assert bt.clears_y()
    bt.coo = (rows, r, c, v.astype(npd))
    y_ref, mag = O.spmv_csr(O.coo_to_csr(rows, r), c.astype(np.uint32), v.astype(npd), x.astype(npd))
    cases.append((bt, x.astype(npd), y_ref, mag, npd))
    stream = A.Stream()
    for which, (b, x, y_ref, mag, _) in enumerate(cases):
        rows, r, c, v = b.coo
        row_ptr, col32 = O.coo_to_csr(rows, r), np.asarray(c).astype(np.uint32)
        dx, dy = A.DeviceArray(x), A.DeviceArray(np.full(b.rows, np.nan, npd))
        b.spmv_device_async(dx, dy, stream, no_alloc=True)       # eager, before the capture
        stream.sync()
        _check(dy.get(), y_ref, mag, npd, "eager call before the capture")
        print("case: capture", which, b.rows, vdt, flush=True)
        stream.capture_begin()
        b.spmv_device_async(dx, dy, stream, no_alloc=True)
        graph = stream.capture_end()
        rng = np.random.default_rng(11 + which)
        for replay in range(3):
            x2 = rng.uniform(-1, 1, b.cols).astype(npd)
            dx.set(x2)
            dy.set(np.full(b.rows, np.nan, npd))
            stream.graph_launch(graph)
            stream.sync()
            y2 = dy.get()
            y_want, mag2 = O.spmv_csr(row_ptr, col32, v, x2)
            _check(y2, y_want, mag2, npd, "replay %d" % replay)
            # eager work of the program between two replays: the allocating entry point on the same x
            _check(b.spmv_device(x2), y_want, mag2, npd, "eager call between replays")
        dx.set(x)                                                # and the first x once more, through the graph
        stream.graph_launch(graph)
        stream.sync()
        _check(dy.get(), y_ref, mag, npd, "replay with the first x")
        stream.graph_destroy(graph)
        dx.free()
        dy.free()
        b.close()
    stream.destroy()
