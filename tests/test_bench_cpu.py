"""bench.py's own arithmetic and the shape of its JSON line, without a GPU."""
import json
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)

import bench  # noqa: E402


def test_bytes_of_the_headline_workload():
    shape = (8, 19, 1024, 1024)
    E, P = 8 * 19 * 1024 * 1024, 8 * 1024 * 1024
    fwd, bwd = bench.algorithmic_bytes("lsr", shape)
    assert fwd == 4 * E + 8 * P + 4 * P and bwd == 8 * E + 8 * P + 4 * P         # the Function-level contract
    assert fwd + bwd == 2113929216
    mf, mb = bench.module_bytes("lsr", shape, "f32")
    assert mf + mb == 12 * E + 16 * P == 2046820352                                 # what `value` divides
    mf16, mb16 = bench.module_bytes("lsr", shape, "bf16")
    assert mf16 + mb16 == 6 * E + 16 * P
    ff, fb = bench.module_bytes("focal", (16, 80, 128, 128), "f32")
    assert ff + fb == 20 * 16 * 80 * 128 * 128 == 419430400


def test_cpu_threads_follow_the_box(monkeypatch):
    monkeypatch.setenv("OMP_NUM_THREADS", "16")
    assert bench.cpu_threads() == 16
    monkeypatch.delenv("OMP_NUM_THREADS")
    assert 1 <= bench.cpu_threads() <= 16


def _fake(ms, nbytes, with_thread=False):
    step = {"warm": {"median": ms}, "graph": {"ms": ms * 1.01}}
    if with_thread:
        step["calling_thread"] = {"ms": ms * 0.9}
    return {"ms_per_step": ms, "algorithmic_bytes_per_step": nbytes, "step_ms": step,
            "kernels": {"forward": {"ms": ms / 3}, "backward": {"ms": 2 * ms / 3}}}


def test_targets_block_holds_every_target_and_is_short():
    main = {"ms_per_step": 0.335, "bytes": 2046820352, "step_ms": {"warm": {"median": 0.334}, "graph": {"ms": 0.345}},
            "roofline": {"forward": {"ms": 0.112}, "backward": {"ms": 0.229}}}
    others = {"lmargin": _fake(0.348, 2046820352), "focal": _fake(0.0727, 419430400, True),
              "focal_seg": _fake(0.512, 3187671040), "lovasz": {"error": "RuntimeError: x"}}
    t = bench.targets_block("lsr", main, others, None, with_cpu=False)
    assert list(t)[:2] == ["unit", "peak_GBps"] and [k for k in t if k in bench.TARGETS] == list(bench.TARGETS)
    assert t["lsr"]["ms"] == 0.335 and abs(t["lsr"]["frac"] - 2046820352 / 0.335e-3 / 8e12) < 1e-4
    assert t["lsr"]["fwd_ms"] == 0.112 and t["lsr"]["bwd_ms"] == 0.229 and t["lsr"]["graph_ms"] == 0.345
    assert t["focal"]["calling_thread_ms"] == round(0.0727 * 0.9, 4) or abs(t["focal"]["calling_thread_ms"] - 0.06543) < 1e-4
    assert "calling_thread_ms" not in t["lmargin"]
    assert t["lovasz"] == {"error": "RuntimeError: x"}
    assert len(json.dumps(t)) < 1500            # a record that keeps the last kilobytes of the line keeps all of it


def test_workload_table_is_consistent():
    for name, w in bench.WORKLOADS.items():
        assert len(w["shape"]) in (2, 4) and w["desc"]
        if "base" in w:
            assert w["base"] in bench.WORKLOADS and "base" not in bench.WORKLOADS[w["base"]]
    for t in bench.TARGETS:
        assert t in bench.WORKLOADS
    for (name, shape) in bench.SYNTH_CONFIG:
        assert bench.WORKLOADS[name]["shape"] == shape
