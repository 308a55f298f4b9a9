"""Seeded random cases through every graph skeleton (the nine of the white list, the two general templates, the x-slice,
tile and product-bin templates): random row-length laws, sizes, dense operators (none, coarse sort, sort + row
division), knobs and launch settings, both value types.  y against the CPU CSR oracle, twice in a row and with y = NaN
before the call (run_case of test_spmv_gpu.py).  Where a skeleton does not apply to the matrix that came up (a format
that would pad too much, a row too long for a template) the case is counted as turned down, not as passed."""
import numpy as np
import pytest

import cases
import alphasparse_amd as A
from alphasparse_amd import _capi as K
from test_spmv_gpu import run_case, SORT

pytestmark = pytest.mark.gpu


def _matrix(rng, seed):
    rows = int(rng.integers(300, 12000))
    law = rng.choice(["uniform", "power", "two classes", "steps"])
    if law == "uniform":
        lens = np.full(rows, int(rng.integers(1, 48)))
    elif law == "power":
        lens = np.minimum(rng.zipf(float(rng.uniform(1.5, 2.5)), rows) * int(rng.integers(1, 6)), min(rows, 3000))
    elif law == "two classes":
        lens = np.where(rng.random(rows) < rng.uniform(0.05, 0.95), rng.integers(1, 6, rows), rng.integers(20, 300, rows))
    else:
        lens = np.repeat(rng.integers(1, 200, 8), -(-rows // 8))[:rows]
    cols = int(rng.choice([rows, rows + 3, 3 * rows + 1, 20011]))
    cols = max(cols, int(lens.max()))
    return law, cases._steps(lens, cols, seed)


KNOBS = {
    "S5": lambda g: {}, "S1": lambda g: {"m": int(g.choice([32, 64, 128, 256]))}, "S9": lambda g: {"t": int(g.choice([2, 3, 4, 8, 32]))},
    "S4": lambda g: {"c": int(g.choice([16, 32, 64]))}, "S6": lambda g: {"m": int(g.choice([2, 4])), "len": 1, "c": int(g.choice([16, 32]))},
    "S7": lambda g: {"n": int(g.choice([512, 896, 2048])), "c": int(g.choice([16, 64]))}, "S8": lambda g: {"b": int(g.choice([64, 128, 512, 1024]))},
    "S2": lambda g: {"m": int(g.choice([32, 64])), "len": 1, "s": int(g.choice([3, 4, 10]))}, "S3": lambda g: {"n": int(g.choice([512, 896])), "s": int(g.choice([3, 7]))},
    "B1": lambda g: {"m": int(g.choice([32, 64, 96])), "w": int(g.choice([8, 16]))}, "B2": lambda g: {"n": int(g.choice([512, 1024])), "w": int(g.choice([4, 8])), "s": int(g.choice([3, 7]))},
    "X1": lambda g: {"slice": int(g.choice([128, 512, 1024, 16384]))},
    "T1": lambda g: {"slice": int(g.choice([128, 512, 1024, 16384])), "group": int(g.choice([16, 128, 512, 4096])), "b": int(g.choice([300, 1024, 8192]))},
    "T2": lambda g: {"slice": int(g.choice([128, 512, 1024, 16384])), "group": int(g.choice([64, 512, 4096])), "b": int(g.choice([300, 1024, 8192]))},
}


def test_random_matrices_through_every_skeleton(gpu):
    names = sorted(KNOBS)
    ran, turned_down = {}, []
    for case in range(84):
        rng = np.random.default_rng(4100 + case)
        skel = names[case % len(names)]
        law, gen = _matrix(rng, 4100 + case)
        kw = KNOBS[skel](rng)
        dense = [[], SORT, SORT + [(K.DENSE_ROW_DIV_ACC_TO_EXPONENTIAL_INCREASE_ROW_NNZ, (int(rng.choice([8, 32])), 2048, 4, 0))]][int(rng.integers(3))]
        launch = {"thread_num_in_block": int(rng.choice([64, 128, 256, 512, 1024]))} if rng.integers(2) else {}
        vdt = K.DOUBLE if rng.integers(2) else K.FLOAT
        print("case %d: %s %s, %d rows x %d columns, %d elements (%s), dense %d, launch %s, %s" % (
            case, skel, kw, gen[0], gen[1], len(gen[2]), law, len(dense), launch, "fp64" if vdt == K.DOUBLE else "fp32"), flush=True)
        try:
            run_case(gpu, gen, vdt, dense, skel, kw, (launch,))
            ran[skel] = ran.get(skel, 0) + 1
        except (K.AlphaSparseError, AssertionError) as e:
            # a y that differs is an AssertionError of assert_y ("relative L2 error" / "exceeds its error bound"): never turned down
            if isinstance(e, AssertionError) and ("error" in str(e) or "bound" in str(e)):
                raise
            turned_down.append((case, skel, str(e)[:100]))
            print("   turned down:", str(e)[:200], flush=True)
    print("ran", ran, "turned down", len(turned_down), flush=True)
    assert sum(ran.values()) >= 50 and all(ran.get(s, 0) >= 2 for s in names), (ran, turned_down)
