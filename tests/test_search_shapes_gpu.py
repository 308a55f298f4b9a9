"""The search on matrices at the edges of what it was written for: a single element, a single row, a column vector, a
diagonal, rows of one element over a wide x, a few giant rows among singles, a tall thin matrix, a small dense one,
every row length from 1 to 2000.  Each search must come back with a graph whose y agrees with the CPU CSR oracle and
without a failed candidate."""
import numpy as np
import pytest

import cases
import spmv_oracle as O
import alphasparse_amd as A
from alphasparse_amd import _capi as K

pytestmark = pytest.mark.gpu


def _shapes():
    rng = np.random.default_rng(1)
    n = 10000
    return {
        "1x1": cases._steps([1], 1, 1),
        "one row of 5000": cases._steps([5000], 5000, 2),
        "column vector": cases._steps([1] * 3000, 1, 3),
        "diagonal": (n, n, np.arange(n, dtype=np.uint64), np.arange(n, dtype=np.uint64), rng.uniform(-1, 1, n), rng.uniform(-1, 1, n)),
        "rows of one element": cases._steps([1] * 50000, 200000, 5),
        "three giant rows among singles": cases._steps([60000, 50000, 40000] + [1] * 20000, 300000, 6),
        "two per row, wide x": cases._steps([2] * 300000, 3000000, 7),
        "tall thin": cases._steps(list(rng.integers(1, 4, 400000)), 50, 8),
        "small dense": cases._steps([300] * 300, 300, 9),
        "lengths 1..2000": cases._steps(list(range(1, 2001)), 4000, 10),
    }


@pytest.mark.parametrize("vdt,npd", [(K.FLOAT, np.float32), (K.DOUBLE, np.float64)], ids=["fp32", "fp64"])
def test_search_on_edge_shapes(gpu, vdt, npd):
    for name, (rows, cols, r, c, v, x) in _shapes().items():
        v, x = np.asarray(v).astype(npd), np.asarray(x).astype(npd)
        m = A.Matrix.from_coo(rows, cols, r, c, v.astype(np.float64), vdt, wave=64)
        res = A.find_best_graph(m, total_time_s=2.0, device=gpu, timed_region_ms=2.0)
        b = res.build_best()
        b.compile().upload(gpu)
        y = b.spmv_device(x)
        y_ref, mag = O.spmv_csr(O.coo_to_csr(rows, r), np.asarray(c).astype(np.uint32), v, x)
        rel, ratio, tol = O.check_y(y, y_ref, mag, npd)
        print("%s: %.2f GFLOP/s, %d candidates, %s" % (name, res.gflops, res.candidates, [b.describe(s)["template"] for s in range(int(res.n_sub))]), flush=True)
        assert res.candidates > 0 and res.failed_candidates == 0, name
        assert rel <= tol and ratio <= 1.0, "%s: rel L2 %.3e, per-row ratio %.2f" % (name, rel, ratio)
        b.close()
