"""Writes tests/golden/search_control.json: what the UPSTREAM parameter enumerator, stop rule and
report-text functions answer for the inputs in tests/search_hooks.py.  Needs oracle/_ref/libasref.so.

    python tests/golden/make_golden_search.py
"""
import json
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
for p in (ROOT, os.path.join(ROOT, "oracle"), os.path.join(ROOT, "tests")):
    sys.path.insert(0, p)

import ref_lib  # noqa: E402
import search_hooks as H  # noqa: E402


def main():
    if not ref_lib.available():
        raise SystemExit("oracle/_ref/libasref.so is missing: run `make -C oracle ref` first")
    L = ref_lib.lib()
    out = {
        "enumerator": [H.enumerate_params(L, "ref_", *c).tolist() for c in H.ENUM_CASES],
        "stop_rule": [H.stop_rule(L, "ref_", s, g) for s, g in H.STOP_CASES],
        "strategy_report": [H.strategy_report(L, "ref_", s, p) for s, p in H.STRATEGY_CASES],
        "template_node_report": [H.template_node_report(L, "ref_", *c) for c in H.TEMPLATE_NODE_CASES],
        "graph_report": [H.graph_report(L, "ref_", *g) for g in H.GRAPH_CASES],
        "graph_report_framed": [[H.graph_report(L, "ref_", *g, frame=f) for f in H.FRAME_CASES] for g in H.GRAPH_CASES[:2]],
    }
    path = os.path.join(HERE, "search_control.json")
    with open(path, "w") as f:
        json.dump(out, f, indent=1)
    print("wrote", os.path.relpath(path, ROOT), os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
