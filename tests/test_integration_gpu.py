"""The reference-side binding of part_execute_code_builder (executor.hpp:12-17): a body that keeps the reference's own
signature and calls the C-ABI,
compiled as a C++ program against include/alphasparse_amd.h (tests/integration/part_execute_wrapper.cc, built by
alphasparse_amd/csrc/Makefile) and run on the GPU: repeat = 0 must take the reference's own launch count
(executor.cc:247-255: 185.2e9 / padded elements, at least 2)."""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
WRAPPER = os.path.join(HERE, "integration", "part_execute_wrapper")


@pytest.mark.gpu
def test_documented_part_execute_wrapper_runs(gpu):
    assert os.path.exists(WRAPPER), "build it with make -C alphasparse_amd/csrc"
    grid = 1024
    print("case: part_execute_code_builder wrapper, %d x %d stencil" % (grid, grid), flush=True)
    p = subprocess.run([WRAPPER, str(grid)], capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stdout + p.stderr
    out = dict(line.split(":", 1) for line in p.stdout.strip().splitlines())
    nnz, padded = int(out["nnz"]), int(out["padded_nnz"])
    time_ms, gflops = float(out["time_ms"]), float(out["gflops"])
    assert nnz == 5 * grid * grid - 4 * grid and padded == 5 * grid * grid
    assert time_ms > 0 and gflops > 0
    # gflops = 2 nnz repeat / time: the launch count that was used
    repeat = gflops * 1e9 * time_ms * 1e-3 / (2.0 * nnz)
    want = max(2, 185200000000 // padded)
    assert abs(repeat - want) <= 0.01 * want, (repeat, want)
    # one launch + synchronisation of this small stencil takes microseconds, not milliseconds
    assert time_ms / want < 1.0
