"""The white-list search end to end on the GPU: every dense-view strategy, the rebuilt best graph
against the CPU CSR oracle, the report text, the executor entry points and the command-line driver."""
import os
import re
import subprocess

import numpy as np
import pytest

import alphasparse_amd as A
import cases
from alphasparse_amd import _capi as K
from alphasparse_amd import synthetic as S
import spmv_oracle as O

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
NP = {K.FLOAT: np.float32, K.DOUBLE: np.float64}


def _oracle(rows, r, c, v, x):
    return O.spmv_csr(O.coo_to_csr(rows, r), np.asarray(c).astype(np.uint32), v, x)


def _check_best(res, rows, r, c, v, x, gpu, npd):
    b = res.build_best()
    b.compile().upload(gpu)
    y_ref, mag = _oracle(rows, r, c, v.astype(npd), x.astype(npd))
    rel, ratio, tol = O.check_y(b.spmv(x.astype(npd)), y_ref, mag, npd)
    assert rel <= tol and ratio <= 1.0, (rel, ratio)
    return b


def _template_types(numbers):
    """Template type of every sub-matrix in the flat description of a graph."""
    at = 1 + 5 * numbers[0]
    out = []
    n_sub = numbers[at]
    at += 1
    for _ in range(n_sub):
        at += 1 + 5 * numbers[at]
        out.append(numbers[at])
        at += 4
    assert at == len(numbers)
    return out


CASES = {
    "laplacian": (lambda: S.laplacian_5pt(160), K.FLOAT),
    "power_law": (lambda: S.power_law(30000, max_len=5000, mean_len=14.0, seed=7), K.FLOAT),
    "fem_fp64": (lambda: S.fem_blocks(2000, 27, 300), K.DOUBLE),
    "irregular_fp64": (lambda: S.extreme_irregular(60000, 8, 3000, 40000, seed=9), K.DOUBLE),
}


@pytest.mark.parametrize("name", sorted(CASES))
def test_search_result_is_correct_and_reported(gpu, name):
    gen, vdt = CASES[name]
    rows, cols, r, c, v, x = gen()
    m = A.Matrix.from_coo(rows, cols, r, c, v.astype(np.float64), vdt, wave=64)
    res = A.find_best_graph(m, total_time_s=12.0, device=gpu, timed_region_ms=3.0)
    print(name, "best %.1f GFLOP/s, %d candidates, %.1f s" % (res.gflops, res.candidates, res.seconds), flush=True)
    assert res.gflops > 0 and res.candidates > 0
    # report: input node first, one "sub_matrix_id:i" per strip, one kernel resource node per strip
    rep = res.report
    assert rep.startswith("{\nstrategy_type:DENSE_BEGIN_MEMORY_CACHE_INPUT_FILE_DIRECT_PARAM_STRATEGY\nnode_type:BEGIN_MEMORY_CACHE_INPUT_FILE\n")
    assert "nnz:%d\n" % len(r) in rep and "row_index_max:%d\n" % (rows - 1) in rep
    assert re.findall(r"sub_matrix_id:(\d+)", rep) == [str(i) for i in range(int(res.n_sub))]
    assert rep.count("kernel_node_type:SET_RESOURCE") == int(res.n_sub)
    assert "node_type:COMPRESS\n" in rep
    log = res.log
    assert log.endswith("finish search\n") and ("gflops:%g\n" % res.gflops) in log
    # the report is, byte for byte, what as_graph_report makes of the best graph's numbers, and the log ends with
    # that text in the frame of upstream's main
    import search_hooks as H
    numbers = res.best_graph()
    assert H.without_extra_keys(rep) == H.graph_report_of_numbers(K.lib(), "as_", numbers)
    # ... and what upstream's own report function returns for the same graph built with upstream's own node adders
    # (the compiled upstream code travels with the tree; without it the committed answers of
    # tests/test_search_control.py pin the same functions)
    import ref_lib
    upstream_only = all(t < 10 for t in _template_types(numbers))
    if ref_lib.available() and upstream_only:
        want = H.graph_report_of_numbers(ref_lib.lib(), "ref_", numbers)
        assert H.without_extra_keys(rep) == want, (rep, want)
        framed = H.graph_report_of_numbers(ref_lib.lib(), "ref_", numbers, frame=(res.gflops, res.time_ms))
        assert H.without_extra_keys(log).endswith(framed), (log[-len(framed) - 200:], framed)
        print(name, "report equals upstream's text for the same graph (%d bytes)" % len(want), flush=True)
    b = _check_best(res, rows, r, c, v, x, gpu, NP[vdt])
    # executor entry points on the rebuilt graph
    ok, ms, gf = A.part_execute_code_builder(b, list(range(int(res.n_sub))), 20)
    assert ok and ms > 0 and gf > 0
    rep_n, ms, gf = A.execute_code_builder(b, seconds=0.05)
    assert rep_n >= 2 and gf > 0
    b.close()


def test_search_stores_a_block_matrix_by_blocks_of_rows(gpu):
    """A banded matrix of dense 3 x 3 blocks whose x does not fit the L2 cache of an XCD (540,000 columns, fp64): the
    search offers the tile skeleton with row groups of whole blocks, and the tile template wins in its column-run
    form under row ownership with blocks of three rows as pieces.  The report says so, and the graph rebuilt from the
    report's nodes gives A x."""
    rows, cols, r, c, v, x = S.fem_blocks(180000, 9, 2000, seed=12)
    m = A.Matrix.from_coo(rows, cols, r, c, v.astype(np.float64), K.DOUBLE, wave=64)
    res = A.find_best_graph(m, total_time_s=30.0, device=gpu, timed_region_ms=5.0, only_dense_strategy=1)
    print("block matrix: best %.1f GFLOP/s, %d candidates, %.1f s" % (res.gflops, res.candidates, res.seconds), flush=True)
    assert res.failed_candidates == 0
    rep = res.report
    assert "kernel_node_type:SHARED_MEM_X_SLICE" in rep, rep
    assert "col_index_runs:1\n" in rep and "y_rows_owned:1\n" in rep and "row_block:3\n" in rep, rep
    assert re.search(r"row_group_size:(\d+)", rep) and int(re.search(r"row_group_size:(\d+)", rep).group(1)) % 3 == 0
    b = _check_best(res, rows, r, c, v, x, gpu, np.float64)
    d = b.describe(0)
    assert d["row_block"] == 3 and "run_row_group" in d["arrays"] and not b.clears_y()
    y_ref, mag = _oracle(rows, r, c, v, x)
    rel, ratio, tol = O.check_y(b.spmv_device(x), y_ref, mag, np.float64)
    assert rel <= tol and ratio <= 1.0, (rel, ratio)
    b.close()


def test_configuration_1_at_its_stated_shape(gpu):
    """Benchmark configuration 1 exactly as stated: 4096 x 4096, 8 elements in every row at seeded uniform columns
    (32,768 elements), values and x in [-1, 1], fp32.  A short search, then the rebuilt best graph against the CPU
    CSR oracle, with y full of NaN before the call as well."""
    rows, cols, r, c, v, x = S.uniform_rows()
    assert (rows, cols, len(r)) == (4096, 4096, 32768) and v.dtype == np.float32
    assert np.all(np.bincount(np.asarray(r, np.int64), minlength=rows) == 8)
    assert np.all(np.abs(v) <= 1) and np.all(np.abs(x) <= 1)
    m = A.Matrix.from_coo(rows, cols, r, c, v.astype(np.float64), K.FLOAT, wave=64)
    res = A.find_best_graph(m, total_time_s=8.0, device=gpu, timed_region_ms=3.0)
    print("C1 best %.1f GFLOP/s, %d candidates, %.1f s" % (res.gflops, res.candidates, res.seconds), flush=True)
    assert res.gflops > 0 and res.candidates > 0 and res.failed_candidates == 0
    b = _check_best(res, rows, r, c, v, x, gpu, np.float32)
    y_ref, mag = _oracle(rows, r, c, v, x)
    rel, ratio, tol = O.check_y(b.spmv_device(x), y_ref, mag, np.float32)
    assert rel <= tol and ratio <= 1.0, (rel, ratio)
    b.close()


def _random_rows(rows, cols, per_row, seed):
    """rows x cols, per_row elements in every row at sorted random columns, fp values in [-1, 1)."""
    rng = np.random.default_rng(seed)
    c = np.concatenate([np.sort(rng.choice(cols, size=min(per_row, cols), replace=False)) for _ in range(rows)])
    r = np.repeat(np.arange(rows), min(per_row, cols))
    return rows, cols, r, c, rng.uniform(-1, 1, len(r)), rng.uniform(-1, 1, cols)


EDGE_SHAPES = {
    "tiny_8x8": lambda: _random_rows(8, 8, 3, 1),
    "single_row": lambda: _random_rows(1, 5000, 1000, 2),
    "one_column": lambda: _random_rows(5000, 1, 1, 3),
    "identity_70000": lambda: (70000, 70000, np.arange(70000), np.arange(70000),
                               np.random.default_rng(4).uniform(-1, 1, 70000), np.random.default_rng(5).uniform(-1, 1, 70000)),
    "wide_64x2M": lambda: _random_rows(64, 2000000, 3000, 6),
    "tall_100000x40": lambda: _random_rows(100000, 40, 10, 7),
}


@pytest.mark.parametrize("name", sorted(EDGE_SHAPES))
def test_search_on_edge_shapes(gpu, name):
    """Shapes at the ends of what the search may be handed: a few rows, one row, one column, one element per row
    beyond 65535 rows, rows far wider than tall and the reverse.  The best graph must give A x."""
    rows, cols, r, c, v, x = EDGE_SHAPES[name]()
    print("case: edge shape", name, rows, cols, len(r), flush=True)
    for vdt in (K.FLOAT, K.DOUBLE):
        m = A.Matrix.from_coo(rows, cols, r, c, v.astype(np.float64), vdt, wave=64)
        res = A.find_best_graph(m, total_time_s=6.0, device=gpu, timed_region_ms=2.0)
        print(name, K.DTYPE_NAMES[vdt], "best %.2f GFLOP/s, %d candidates, %.1f s" % (res.gflops, res.candidates, res.seconds), flush=True)
        assert res.gflops > 0 and res.candidates > 0
        _check_best(res, rows, r, c, v, x, gpu, NP[vdt]).close()


def _random_matrix(seed):
    """One of six families by seed % 6 (equal rows, power-law lengths, band, short rows plus a few giant ones, a
    few very wide rows, a mix of lengths), sizes drawn from the seed; no row without elements."""
    rng = np.random.default_rng(seed)
    kind = seed % 6
    if kind == 0:
        rows = int(rng.integers(50, 300000)); per = int(rng.integers(1, 40)); cols = int(rng.integers(per, 400000))
        lens = np.full(rows, per)
    elif kind == 1:
        rows = int(rng.integers(100, 200000)); cols = int(rng.integers(1000, 3000000))
        lens = np.minimum((rng.pareto(1.2, rows) * 3 + 1).astype(np.int64), cols)
    elif kind == 2:
        rows = int(rng.integers(100, 300000)); cols = rows
        lens = rng.integers(1, 12, rows)
    elif kind == 3:
        rows = int(rng.integers(1000, 400000)); cols = int(rng.integers(50000, 3000000))
        lens = rng.integers(1, 4, rows)
        giant = rng.choice(rows, size=int(rng.integers(1, 20)), replace=False)
        lens[giant] = rng.integers(1000, min(cols, 60000), len(giant))
    elif kind == 4:
        rows = int(rng.integers(1, 200)); cols = int(rng.integers(1000, 5000000))
        lens = rng.integers(1, min(cols, 20000), rows)
    else:
        rows = int(rng.integers(1000, 100000)); cols = int(rng.integers(100, 1000000))
        lens = np.minimum(rng.choice([1, 2, 5, 17, 64, 130, 700], rows, p=[.3, .2, .2, .15, .1, .04, .01]), cols)
    lens = np.maximum(lens, 1).astype(np.int64)
    r = np.repeat(np.arange(rows), lens)
    c = np.clip(r + rng.integers(-6, 7, len(r)), 0, cols - 1) if kind == 2 else rng.integers(0, cols, len(r))
    key = np.unique(r.astype(np.int64) * cols + c)          # sorted by (row, column), duplicates dropped
    r, c = key // cols, key % cols
    return rows, cols, r, c, rng.uniform(-1, 1, len(r)), rng.uniform(-1, 1, cols)


@pytest.mark.parametrize("seed", [6, 13, 20, 27, 34, 41])
def test_search_on_random_matrices(gpu, seed):
    """A short search on a matrix drawn from the seed (one per family; fp32 for even seeds, fp64 for odd ones, the
    general templates for every third): no candidate may fail to build and the best graph must give A x."""
    rows, cols, r, c, v, x = _random_matrix(seed)
    vdt = K.DOUBLE if seed % 2 else K.FLOAT
    print("case: random matrix seed", seed, rows, cols, len(r), K.DTYPE_NAMES[vdt], flush=True)
    m = A.Matrix.from_coo(rows, cols, r, c, v.astype(np.float64), vdt, wave=64)
    res = A.find_best_graph(m, total_time_s=4.0, device=gpu, timed_region_ms=1.0, general_templates=seed % 3 == 0)
    print("seed", seed, "best %.1f GFLOP/s, %d candidates, %d strips" % (res.gflops, res.candidates, res.n_sub), flush=True)
    assert res.failed_candidates == 0, [ln for ln in res.log.splitlines() if "failed" in ln or "rejected" in ln][:5]
    _check_best(res, rows, r, c, v, x, gpu, NP[vdt]).close()


def test_search_rejects_candidates_with_a_wrong_result(gpu):
    """Every candidate runs once on x = 1 and is compared with the row sums before it is timed.  With a NaN among
    the values no candidate can agree with the row sums, so each one is rejected and the search ends without a
    graph; with the check switched off the same input is only timed and a graph comes out."""
    rows, cols, r, c, v, x = S.power_law(3000, max_len=200, mean_len=6.0, seed=3)
    v = v.astype(np.float64)
    v[len(v) // 2] = np.nan
    m = A.Matrix.from_coo(rows, cols, r, c, v, K.FLOAT, wave=64)
    with pytest.raises(A.AlphaSparseError, match="no working candidate"):
        A.find_best_graph(m, total_time_s=3.0, device=gpu, timed_region_ms=1.0, only_dense_strategy=1)
    res = A.find_best_graph(m, total_time_s=3.0, device=gpu, timed_region_ms=1.0, only_dense_strategy=1, skip_verification=True)
    assert res.gflops > 0 and res.failed_candidates == 0


def test_search_with_the_general_templates(gpu):
    """general_templates: the DIRECT_ATOM / SHARED_MEMORY skeletons (G1, G2) are tried next to the white list, every
    candidate of theirs runs, and the result is still checked against the CPU CSR oracle."""
    rows, cols, r, c, v, x = S.uniform_rows(20000, 24, seed=4)
    m = A.Matrix.from_coo(rows, cols, r, c, v.astype(np.float64), K.FLOAT, wave=64)
    res = A.find_best_graph(m, total_time_s=15.0, device=gpu, timed_region_ms=2.0, only_dense_strategy=1, general_templates=True)
    assert " G1 knobs" in res.log and " G2 knobs" in res.log and res.failed_candidates == 0
    assert " DIRECT_ATOM_TEMPLATE threads" in res.log and " SHARED_MEMORY_TEMPLATE threads" in res.log
    _check_best(res, rows, r, c, v, x, gpu, np.float32).close()
    plain = A.find_best_graph(m, total_time_s=6.0, device=gpu, timed_region_ms=2.0, only_dense_strategy=1)
    assert " G1 knobs" not in plain.log


@pytest.mark.parametrize("strategy", [1, 2, 3])
def test_each_dense_strategy_alone(gpu, strategy):
    # row lengths already grouped in bands, so the row division of strategy 2 yields three strips
    # (on an unsorted matrix it yields more than four and the strategy is skipped, as upstream does)
    rows, cols, r, c, v, x = cases._steps([3] * 6000 + [50] * 2000 + [300] * 300, 9000, 3)
    m = A.Matrix.from_coo(rows, cols, r, c, v.astype(np.float64), K.FLOAT, wave=64)
    res = A.find_best_graph(m, total_time_s=8.0, device=gpu, timed_region_ms=2.0, only_dense_strategy=strategy)
    assert int(res.dense_strategy) == strategy
    if strategy == 1:
        assert int(res.n_sub) == 1
    else:
        assert 2 <= int(res.n_sub) <= 4 and "node_type:DENSE_ROW_DIV\n" in res.report
    if strategy == 3:
        assert "node_type:DENSE_ROW_COARSE_SORT\n" in res.report
    _check_best(res, rows, r, c, v, x, gpu, np.float32).close()


def test_search_rejects_unsorted_and_empty_rows(gpu):
    m = A.Matrix.from_coo(4, 4, [0, 2, 3], [0, 1, 2], np.ones(3), K.FLOAT, wave=64)   # row 1 is empty
    with pytest.raises(K.AlphaSparseError, match="rows without elements"):
        A.find_best_graph(m, total_time_s=1.0, device=gpu)
    m = A.Matrix.from_coo(3, 4, [0, 2, 1], [0, 1, 2], np.ones(3), K.FLOAT, wave=64)
    with pytest.raises(K.AlphaSparseError, match="sorted"):
        A.find_best_graph(m, total_time_s=1.0, device=gpu)


def test_search_removes_empty_rows_on_request(gpu):
    """Upstream stops at rows without elements (main.cc:604-621) and so does the search by default; with
    remove_empty_rows it compacts them away first and the best graph still produces the full-length y."""
    rows, cols, r, c, v, x = S.power_law(6000, max_len=900, mean_len=10.0, seed=9)
    rng = np.random.default_rng(9)
    keep = ~(rng.uniform(size=rows) < 0.4)[np.asarray(r, np.int64)]
    r, c, v = r[keep], c[keep], v[keep]
    m = A.Matrix.from_coo(rows, cols, r, c, v.astype(np.float64), K.FLOAT, wave=64)
    assert m.has_empty_row()
    with pytest.raises(A.AlphaSparseError, match="rows without elements"):
        A.find_best_graph(m, total_time_s=3, device=gpu)
    res = A.find_best_graph(m, total_time_s=6, device=gpu, remove_empty_rows=True)
    assert res.gflops > 0 and "rows without elements are removed" in res.log
    b = res.build_best()
    b.compile().upload(gpu)
    y = b.spmv(x)
    y_ref, mag = O.spmv_csr(O.coo_to_csr(rows, r), c.astype(np.uint32), v, x)
    rel, ratio, tol = O.check_y(y, y_ref, mag, np.float32)
    assert len(y) == rows and rel <= tol and ratio <= 1.0
    b.close()


def test_checkpoint_files_of_each_strategy(gpu, tmp_path):
    rows, cols, r, c, v, x = S.power_law(8000, max_len=2500, mean_len=10.0, seed=4)
    m = A.Matrix.from_coo(rows, cols, r, c, v.astype(np.float64), K.FLOAT, wave=64)
    A.find_best_graph(m, total_time_s=6.0, device=gpu, timed_region_ms=2.0, checkpoint_dir=str(tmp_path))
    names = sorted(os.listdir(tmp_path))
    assert "best_result_of_strategy1" in names
    text = open(os.path.join(tmp_path, "best_result_of_strategy1")).read()
    assert text.startswith("gflops:") and "sub_matrix_id:0" in text


def test_command_line_driver(gpu, tmp_path):
    exe = os.path.join(ROOT, "alphasparse_amd", "asx_main")
    if not os.path.exists(exe):
        pytest.fail("alphasparse_amd/asx_main is not built (make -C alphasparse_amd/csrc)")
    rows, cols, r, c, v, x = S.uniform_rows(3000, 8, seed=2)
    m = A.Matrix.from_coo(rows, cols, r, c, v.astype(np.float64), K.FLOAT, wave=64)
    path = str(tmp_path / "u.mtx.coo")
    m.write_coo_file(path)
    p = subprocess.run([exe, path, "float", "4", str(gpu)], capture_output=True, text=True, timeout=110)
    assert p.returncode == 0, p.stdout[-2000:] + p.stderr[-2000:]
    out = p.stdout
    assert re.search(r"^gflops:[0-9.e+]+$", out, re.M) and re.search(r"^time:[0-9.e+-]+$", out, re.M)
    assert out.index("finish search") < out.index("final_gflops:") < out.index("final_time:")
    assert float(re.search(r"^final_gflops:([0-9.e+]+)$", out, re.M).group(1)) > 0


def test_command_line_driver_reads_mtx_and_binary_files(gpu, tmp_path):
    """The driver picks the reader by file name: a Matrix Market file is prepared in-process, the binary cache read as is."""
    exe = os.path.join(ROOT, "alphasparse_amd", "asx_main")
    if not os.path.exists(exe):
        pytest.fail("alphasparse_amd/asx_main is not built (make -C alphasparse_amd/csrc)")
    rows, cols, r, c, v, x = S.uniform_rows(2000, 6, seed=4)
    m = A.Matrix.from_coo(rows, cols, r, c, v.astype(np.float64), K.FLOAT, wave=64)
    coo, mtx, binary = (str(tmp_path / n) for n in ("u.mtx.coo", "u.mtx", "u.bin"))
    m.write_coo_file(coo)
    lines = open(coo).read().splitlines()
    rng = np.random.default_rng(0)
    body = [lines[i + 1] for i in rng.permutation(len(lines) - 1)]       # Matrix Market entries come in any order
    open(mtx, "w").write("%%MatrixMarket matrix coordinate real general\n% shuffled\n" + "\n".join([lines[0]] + body) + "\n")
    m.write_binary_file(binary)
    for path in (mtx, binary):
        p = subprocess.run([exe, path, "float", "2", str(gpu)], capture_output=True, text=True, timeout=110)
        assert p.returncode == 0, p.stdout[-2000:] + p.stderr[-2000:]
        assert "nnz:%d\n" % len(r) in p.stdout and "finish search" in p.stdout
        assert float(re.search(r"^final_gflops:([0-9.e+]+)$", p.stdout, re.M).group(1)) > 0
