"""ctypes access to the search-control / report hooks that the product library and the upstream
harness export under the same names (prefix as_ / ref_)."""
import ctypes as C

import numpy as np

LP = C.POINTER(C.c_long)


def _longs(v):
    a = (C.c_long * len(v))(*[int(x) for x in v])
    return a


def enumerate_params(L, prefix, low, up, step):
    f = getattr(L, prefix + "selftest_param_enumerator")
    f.restype = C.c_int64
    f.argtypes = [C.c_int, LP, LP, LP, LP, C.c_uint64]
    n = len(low)
    cap = 4096 * n
    out = (C.c_long * cap)()
    cnt = f(n, _longs(low), _longs(up), _longs(step), out, cap)
    assert 0 <= cnt * n <= cap
    return np.array(out[:cnt * n], dtype=np.int64).reshape(cnt, n)


def stop_rule(L, prefix, struggle, gflops):
    f = getattr(L, prefix + "selftest_search_strategy")
    f.argtypes = [C.c_uint64, C.POINTER(C.c_float), C.c_int, C.POINTER(C.c_int)]
    g = (C.c_float * len(gflops))(*gflops)
    go = (C.c_int * len(gflops))()
    assert f(struggle, g, len(gflops), go) == 0
    return list(go)


def _text(f, *args):
    buf = C.create_string_buffer(8192)
    n = f(*args, buf, 8192)
    assert 0 <= n < 8192, n
    return buf.value.decode()


def strategy_report(L, prefix, strategy, p):
    f = getattr(L, prefix + "strategy_report")
    f.restype = C.c_int64
    f.argtypes = [C.c_int, LP, C.c_char_p, C.c_uint64]
    p = list(p) + [0] * (4 - len(p))
    return _text(f, strategy, _longs(p))


def template_node_report(L, prefix, tp, blocks, threads, row_reduce):
    f = getattr(L, prefix + "template_node_report")
    f.restype = C.c_int64
    f.argtypes = [C.c_int, C.c_long, C.c_long, C.c_long, C.c_char_p, C.c_uint64]
    return _text(f, tp, blocks, threads, row_reduce)


def graph_description(dense, subs):
    """Flat numbers of a graph: dense = [(strategy, knobs)], subs = [([(strategy, knobs)], (template, blocks, threads,
    row_reduce))]; the input node's knobs are (element count, value type, largest column, largest row)."""
    def nodes(v):
        out = [len(v)]
        for s, p in v:
            out += [s] + list(p) + [0] * (4 - len(p))
        return out
    d = nodes(dense) + [len(subs)]
    for v, tpl in subs:
        d += nodes(v) + list(tpl)
    return d


def graph_report(L, prefix, dense, subs, frame=None):
    """The assembled report of a whole graph; frame = (gflops, time_ms): with the lines printed around it."""
    f = getattr(L, prefix + "graph_report")
    f.restype = C.c_int64
    f.argtypes = [LP, C.c_int64, C.c_int, C.c_float, C.c_float, C.c_char_p, C.c_uint64]
    d = graph_description(dense, subs)
    buf = C.create_string_buffer(1 << 16)
    n = f(_longs(d), len(d), 0 if frame is None else 1, *(frame or (0.0, 0.0)), buf, 1 << 16)
    assert 0 <= n < (1 << 16), n
    return buf.value.decode()


def graph_report_of_numbers(L, prefix, numbers, frame=None):
    """graph_report for a graph already given as its flat list of numbers (as_search_best_graph)."""
    f = getattr(L, prefix + "graph_report")
    f.restype = C.c_int64
    f.argtypes = [LP, C.c_int64, C.c_int, C.c_float, C.c_float, C.c_char_p, C.c_uint64]
    buf = C.create_string_buffer(1 << 16)
    n = f(_longs(numbers), len(numbers), 0 if frame is None else 1, *(frame or (0.0, 0.0)), buf, 1 << 16)
    assert 0 <= n < (1 << 16), n
    return buf.value.decode()


# keys of the kernel resource node that upstream does not have (column forms and row forms of this library's kernels)
EXTRA_REPORT_KEYS = ("col_index_relative:1\n", "col_index_diagonal:1\n", "col_index_runs:1\n", "y_rows_owned:1\n")


def without_extra_keys(report):
    import re
    for k in EXTRA_REPORT_KEYS:
        report = report.replace(k, "")
    return re.sub(r"row_block:\d+\n", "", report)


# inputs shared by the fixture generator and the tests
ENUM_CASES = [([0], [3], [1]), ([2], [32], [7]), ([64], [64], [64]), ([0, 64], [2, 256], [1, 64]),
              ([2, 32, 1], [4, 96, 10], [2, 32, 3])]
STOP_CASES = [
    (10, [1.0] * 40),
    (10, [1, 2, 3, 4, 5, 6] + [0.5] * 60),
    (10, [10, 10.5, 10.7, 300] + [1.0] * 50),
    (3, [5, 4, 4, 4, 4, 4, 4.9, 5.1] + [0.0] * 30),
    (0, [100.0] + [50.0] * 30),
    (10, [0.0] * 30),
]
STRATEGY_CASES = [(0, (64, 1)), (1, (128,)), (2, (2048,)), (3, (4096,)), (4, (8,)), (5, (64,)), (6, ()), (7, (4,)), (8, (5,)),
                  (9, (1,)), (11, ()), (12, (32, 2048, 4, 0))]
TEMPLATE_NODE_CASES = [(tp, 4096, 256, rr) for tp in range(10) for rr in (1, 16)]
# whole graphs: (dense nodes, [(sub-matrix nodes, (template, tblock_num, thread_num_in_block, thread_num_of_row_reduce))]).
# Strategy 10 = the input node (element count, value type 10 = FLOAT / 11 = DOUBLE, largest column, largest row).
INPUT_F32 = (10, (32768, 10, 4095, 4095))
INPUT_F64 = (10, (5000, 11, 99999, 49999))
GRAPH_CASES = [
    # dense strategy 1, one strip, ELL
    ([INPUT_F32, (11, ())], [([(0, (64, 1)), (6, ())], (2, 64, 256, 1))]),
    # dense strategy 1, SELL with an LDS reduction
    ([INPUT_F32, (11, ())], [([(0, (64, 4)), (1, (64,)), (7, (4,))], (4, 512, 128, 16))]),
    # dense strategy 2: row division, two strips with different templates
    ([INPUT_F64, (12, (32, 2048, 4, 0)), (11, ())],
     [([(8, (5,))], (9, 0, 128, 1)), ([(3, (4096,))], (5, 977, 1024, 1))]),
    # dense strategy 3: coarse sort + row division, three strips, three templates
    ([INPUT_F64, (9, (1,)), (12, (16, 1024, 8, 0)), (11, ())],
     [([(0, (64, 1)), (1, (128,)), (6, ())], (1, 391, 128, 1)),
      ([(2, (2048,)), (5, (64,))], (6, 120, 512, 4)),
      ([(5, (32,))], (7, 4096, 256, 1))]),
    # a CSR5-like strip
    ([INPUT_F32, (11, ())], [([(8, (3,))], (8, 1366, 64, 1))]),
]
FRAME_CASES = [(123.456, 0.01875), (2058.31, 0.0203694), (1e-3, 12345.678), (0.0, 99999999999.0)]
