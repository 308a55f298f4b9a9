"""Search control (parameter enumerator, stop rule) and report text against the upstream code:
committed answers in tests/golden/search_control.json (written by tests/golden/make_golden_search.py
from the upstream library), plus the upstream library itself on more inputs where it is built."""
import json
import os

import numpy as np
import pytest

import search_hooks as H
from alphasparse_amd import _capi as K

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "search_control.json")


# no GPU needed: run in the CPU suite and once more, under the `gpu` marker, in the suite of the GPU box
EVERYWHERE = pytest.mark.parametrize("where", ["cpu", pytest.param("gpu_box", marks=pytest.mark.gpu)])


@pytest.fixture(scope="module")
def want():
    with open(GOLDEN) as f:
        return json.load(f)


@EVERYWHERE
def test_param_enumerator_matches_upstream(want, where):
    for case, w in zip(H.ENUM_CASES, want["enumerator"]):
        got = H.enumerate_params(K.lib(), "as_", *case)
        assert got.tolist() == w, case


def test_param_enumerator_is_an_odometer():
    got = H.enumerate_params(K.lib(), "as_", [1, 10], [3, 30], [1, 10])
    assert got.tolist() == [[a, b] for b in (10, 20, 30) for a in (1, 2, 3)]   # knob 0 fastest


@EVERYWHERE
def test_stop_rule_matches_upstream(want, where):
    for (struggle, g), w in zip(H.STOP_CASES, want["stop_rule"]):
        assert H.stop_rule(K.lib(), "as_", struggle, g) == w, (struggle, g[:8])


def test_stop_rule_window_and_struggle_steps():
    # first result 1.0: window = clamp(5 * 1.0, 5, 25) = 5 steps, then 10 struggle steps, then stop
    go = H.stop_rule(K.lib(), "as_", 10, [1.0] + [0.5] * 30)
    assert go[:16] == [1] * 16 and go[16:] == [0] * 15
    # an improvement of 300 opens the largest window (25)
    go = H.stop_rule(K.lib(), "as_", 0, [300.0] + [1.0] * 40)
    assert go[:26] == [1] * 26 and go[26] == 0


@EVERYWHERE
def test_strategy_report_matches_upstream(want, where):
    for (s, p), w in zip(H.STRATEGY_CASES, want["strategy_report"]):
        assert H.strategy_report(K.lib(), "as_", s, p) == w


@EVERYWHERE
def test_template_node_report_matches_upstream(want, where):
    for case, w in zip(H.TEMPLATE_NODE_CASES, want["template_node_report"]):
        assert H.template_node_report(K.lib(), "as_", *case) == w, K.TEMPLATE_NAMES[case[0]]


@EVERYWHERE
def test_graph_report_matches_upstream(want, where):
    """The assembled report of whole graphs (one to three strips, every dense strategy, nine template types),
    byte for byte what upstream's own functions return for graphs built with upstream's own node adders; and with
    the lines upstream's main prints around it."""
    for g, w in zip(H.GRAPH_CASES, want["graph_report"]):
        assert H.graph_report(K.lib(), "as_", *g) == w
    for g, ws in zip(H.GRAPH_CASES[:2], want["graph_report_framed"]):
        for f, w in zip(H.FRAME_CASES, ws):
            assert H.graph_report(K.lib(), "as_", *g, frame=f) == w, f


def test_graph_report_shape():
    """Known answers that do not need the fixture: node order, sub_matrix_id lines, brace nesting of the kernel nodes."""
    text = H.graph_report(K.lib(), "as_", *H.GRAPH_CASES[2])
    assert text.startswith("{\nstrategy_type:DENSE_BEGIN_MEMORY_CACHE_INPUT_FILE_DIRECT_PARAM_STRATEGY\nnode_type:BEGIN_MEMORY_CACHE_INPUT_FILE\n"
                           "{\nnnz:5000\ndata_type:DOUBLE\ncol_index_max:99999\nrow_index_max:49999\n}\n}\n")
    assert text.count("sub_matrix_id:") == 2 and text.index("sub_matrix_id:0\n") < text.index("sub_matrix_id:1\n")
    assert text.index("node_type:COMPRESS\n") < text.index("sub_matrix_id:0\n")
    framed = H.graph_report(K.lib(), "as_", *H.GRAPH_CASES[0], frame=(0.0, 5.0))
    assert framed == "gflops:0\ntime:5\nerror\nfinish search\n"
    framed = H.graph_report(K.lib(), "as_", *H.GRAPH_CASES[0], frame=(12.5, 0.25))
    assert framed == "gflops:12.5\ntime:0.25\n" + H.graph_report(K.lib(), "as_", *H.GRAPH_CASES[0]) + "\nfinish search\n"


@EVERYWHERE
def test_live_upstream_on_random_inputs(where):
    import ref_lib
    if not ref_lib.available():
        pytest.skip("oracle/_ref is not built here (upstream sources absent); the committed answers cover this")
    R, L = ref_lib.lib(), K.lib()
    rng = np.random.default_rng(5)
    for _ in range(40):
        n = int(rng.integers(1, 4))
        low = rng.integers(0, 50, n)
        step = rng.integers(1, 9, n)
        up = low + rng.integers(0, 20, n)
        a = H.enumerate_params(L, "as_", low, up, step)
        b = H.enumerate_params(R, "ref_", low, up, step)
        assert a.tolist() == b.tolist(), (low, up, step)
    for _ in range(40):
        g = list(np.round(rng.gamma(2.0, 20.0, 80) * (rng.random(80) < 0.3), 2))
        struggle = int(rng.integers(0, 12))
        assert H.stop_rule(L, "as_", struggle, g) == H.stop_rule(R, "ref_", struggle, g)
    for s, p in H.STRATEGY_CASES:
        p2 = tuple(int(x) for x in rng.integers(1, 5000, len(p)))
        assert H.strategy_report(L, "as_", s, p2) == H.strategy_report(R, "ref_", s, p2)
    for tp in range(10):
        args = (tp, int(rng.integers(1, 1 << 20)), 64 * int(rng.integers(1, 17)), int(2 ** rng.integers(0, 7)))
        assert H.template_node_report(L, "as_", *args) == H.template_node_report(R, "ref_", *args)
    # whole graphs with random knobs and launch parameters
    for dense, subs in H.GRAPH_CASES:
        dense2 = [(s, tuple(int(x) for x in rng.integers(1, 5000, len(p))) if s != 10 else p) for s, p in dense]
        subs2 = [([(s, tuple(int(x) for x in rng.integers(1, 5000, len(p)))) for s, p in nodes],
                  (tpl[0], int(rng.integers(1, 1 << 20)), 64 * int(rng.integers(1, 17)), int(2 ** rng.integers(0, 7))))
                 for nodes, tpl in subs]
        frame = (float(np.float32(rng.gamma(2.0, 300.0))), float(np.float32(rng.gamma(2.0, 0.05))))
        assert H.graph_report(L, "as_", dense2, subs2) == H.graph_report(R, "ref_", dense2, subs2)
        assert H.graph_report(L, "as_", dense2, subs2, frame) == H.graph_report(R, "ref_", dense2, subs2, frame)
