"""The enqueue-only SpMV entry points (as_builder_spmv_device_async and its twin that allocates nothing): many calls
back to back on a stream of the caller with one wait at the end, against the CPU CSR oracle -- for a one-kernel
graph, a two-strip graph whose first strip's finish is carried by the second strip's kernel, and a graph that starts
with a clear of y.  y holds NaN before the first call and every call must leave A x, not a sum over calls."""
import numpy as np
import pytest

import spmv_oracle as O
import alphasparse_amd as A
from alphasparse_amd import _capi as K
from alphasparse_amd import skeletons as SK
from alphasparse_amd import synthetic as S

pytestmark = pytest.mark.gpu
NP = {K.FLOAT: np.float32, K.DOUBLE: np.float64}


def _check(y, y_ref, mag, npd, what):
    rel, ratio, tol = O.check_y(y, y_ref, mag, npd)
    assert rel <= tol and ratio <= 1.0, "%s: rel L2 %.3e (tolerance %.0e), per-row ratio %.2f" % (what, rel, tol, ratio)


def graphs(gpu, vdt):
    """(name, builder, rows, r, c, v) of the three kinds of launch sequence."""
    npd = NP[vdt]
    out = []
    # one kernel, every row stored once: ELL on a stencil
    rows, cols, r, c, v, x = S.laplacian_5pt(96)
    m = A.Matrix.from_coo(rows, cols, r, c, v.astype(np.float64), vdt, wave=64)
    m.execute_strategy(K.COMPRESS_NONE)
    b = A.Builder(m)
    b.set_template(0, SK.apply_skeleton(m, 0, "S5")[0])
    out.append(("one kernel", b, rows, cols, r, c, v.astype(npd)))
    # coarse sort, tile strip (scratch vector + finish) and product-bin strip (products in scratch, two kernels)
    rows, cols, r, c, v, x = S.power_law(20000, max_len=3000, mean_len=12.0, seed=31)
    m = A.Matrix.from_coo(rows, cols, r, c, v.astype(np.float64), vdt, wave=64)
    m.execute_strategy(K.DENSE_ROW_COARSE_SORT_FIXED, -1, (1,))
    m.execute_strategy(K.DENSE_ROW_DIV_ACC_TO_EXPONENTIAL_INCREASE_ROW_NNZ, -1, (16, 16, 2, 0))
    m.execute_strategy(K.COMPRESS_NONE)
    b = A.Builder(m)
    b.set_template(0, SK.apply_skeleton(m, 0, "T1", slice=1024, group=512, b=2048)[0])
    b.set_template(1, SK.apply_skeleton(m, 1, "T2", slice=1024, group=4096, b=2048)[0])
    out.append(("two strips", b, rows, cols, r, c, v.astype(npd)))
    # the tile template without a sort adds into y with atomics: the call starts with a clear of y
    rows, cols, r, c, v, x = S.power_law(8000, max_len=900, mean_len=20.0, seed=5)
    m = A.Matrix.from_coo(rows, cols, r, c, v.astype(np.float64), vdt, wave=64)
    m.execute_strategy(K.COMPRESS_NONE)
    b = A.Builder(m)
    b.set_template(0, SK.apply_skeleton(m, 0, "T1", slice=1024, group=512, b=2048)[0])
    out.append(("clear of y", b, rows, cols, r, c, v.astype(npd)))
    return out


@pytest.mark.parametrize("vdt", [K.FLOAT, K.DOUBLE], ids=["fp32", "fp64"])
@pytest.mark.parametrize("no_alloc", [False, True], ids=["alloc", "no_alloc"])
def test_a_hundred_enqueued_calls_then_one_wait(gpu, vdt, no_alloc):
    npd = NP[vdt]
    stream = A.Stream()
    for name, b, rows, cols, r, c, v in graphs(gpu, vdt):
        for serial, carry in ((True, True), (True, False), (False, True)) if name == "two strips" else ((True, True),):
            b.set_serial_launch(serial)
            b.set_finish_carry(carry)
            b.compile().upload(gpu)
            assert b.clears_y() == (name == "clear of y")
            assert (b.finish_carrier(0) == 1) == (name == "two strips" and serial and carry)
            rng = np.random.default_rng(3)
            xs = [rng.uniform(-1, 1, cols).astype(npd) for _ in range(2)]
            dx = [A.DeviceArray(x) for x in xs]
            dy = [A.DeviceArray(np.full(rows, np.nan, npd)) for _ in xs]
            print("case: async", name, "serial" if serial else "concurrent", "carried" if carry else "own finish",
                  "no_alloc" if no_alloc else "alloc", flush=True)
            for call in range(100):                      # two vectors in turn, nothing waits in between
                b.spmv_device_async(dx[call % 2], dy[call % 2], stream, no_alloc=no_alloc)
            stream.sync()
            for x, y in zip(xs, dy):
                y_ref, mag = O.spmv_csr(O.coo_to_csr(rows, r), np.asarray(c).astype(np.uint32), v, x)
                _check(y.get(), y_ref, mag, npd, name)
            # the blocking call is the same launches on the builder's own stream + a wait
            b.spmv_device_async(dx[0], dy[1], None, no_alloc=no_alloc)
            b.sync()
            y_ref, mag = O.spmv_csr(O.coo_to_csr(rows, r), np.asarray(c).astype(np.uint32), v, xs[0])
            _check(dy[1].get(), y_ref, mag, npd, name + ", builder's own stream")
            for d in dx + dy:
                d.free()
        b.close()
    stream.destroy()


def test_enqueue_only_call_on_the_default_stream(gpu):
    """A null stream argument is HIP's default stream (not the builder's own): calls through the C-ABI with NULL, a
    device-wide wait, y against the oracle -- for the two-strip graph one after the other and on concurrent streams
    (which then fork from and join the default stream)."""
    import ctypes as C
    L = K.lib()
    for serial in (True, False):
        name, b, rows, cols, r, c, v = graphs(gpu, K.FLOAT)[1]
        b.set_serial_launch(serial)
        b.compile().upload(gpu)
        rng = np.random.default_rng(3)
        row_ptr, col32 = O.coo_to_csr(rows, r), np.asarray(c).astype(np.uint32)
        dx, dy = A.DeviceArray(np.zeros(cols, np.float32)), A.DeviceArray(np.full(rows, np.nan, np.float32))
        for call in range(5):
            x = rng.uniform(-1, 1, cols).astype(np.float32)
            dx.set(x)
            for no_alloc in (False, True):
                f = L.as_builder_spmv_device_no_alloc_async if no_alloc else L.as_builder_spmv_device_async
                K.check(f(b._h, dx.ptr, dy.ptr, C.c_void_p(None)), L)
                assert L.as_hip_device_sync() == 0
                y_ref, mag = O.spmv_csr(row_ptr, col32, v, x)
                _check(dy.get(), y_ref, mag, np.float32, "default stream, call %d, %s, %s" % (call, "serial" if serial else "concurrent", "no_alloc" if no_alloc else "alloc"))
        dx.free()
        dy.free()
        b.close()
