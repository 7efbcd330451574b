"""Host logic of bench.py that needs no GPU: argument handling, the work accounting of the workloads, and the assembly
of results from the measuring child processes (a workload that ends its process must not cost the others theirs)."""
import json
import os
import subprocess
import sys
import types

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
import bench  # noqa: E402


def _args(**kw):
    d = dict(steps=5, warmup=1, trace_steps=2, no_cpu=True, cpu_time_allowance=240.0)
    d.update(kw)
    return types.SimpleNamespace(**d)


def test_results_of_a_child_that_ended_early_are_kept(monkeypatch):
    lines = [bench.RESULT_TAG + json.dumps(dict(workload="layer_norm", value=1.0)), "some other output",
             bench.RESULT_TAG + json.dumps(dict(workload="xentropy", value=2.0)), bench.RESULT_TAG + "{broken"]
    seen = {}

    def fake_run(cmd, **kw):
        seen["cmd"] = cmd
        return subprocess.CompletedProcess(cmd, -6, stdout="\n".join(lines))
    monkeypatch.setattr(subprocess, "run", fake_run)
    got = bench._in_child(["layer_norm", "xentropy", "generator_loss"], _args(), 10)
    assert [r["workload"] for r in got] == ["layer_norm", "xentropy", "generator_loss"]
    assert got[0]["value"] == 1.0 and got[1]["value"] == 2.0 and "status -6" in got[2]["error"]
    cmd = seen["cmd"]
    assert "--in-process" in cmd and "--emit-results" in cmd and "--no-cpu" in cmd
    assert cmd[cmd.index("--workload") + 1] == "layer_norm,xentropy,generator_loss"


def test_results_of_a_child_that_ran_into_the_time_limit_are_kept(monkeypatch):
    def fake_run(cmd, **kw):
        raise subprocess.TimeoutExpired(cmd, kw["timeout"], output=(bench.RESULT_TAG + json.dumps(dict(workload="mlp", value=3.0))).encode())
    monkeypatch.setattr(subprocess, "run", fake_run)
    got = bench._in_child(["mlp", "self_attn"], _args(), 7)
    assert got[0]["value"] == 3.0 and "stopped after 7 s" in got[1]["error"]


def test_more_than_one_gpu_and_unknown_workloads_are_refused():
    for extra in (["--gpus", "2"], ["--workload", "no_such_workload"]):
        r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py")] + extra, capture_output=True, text=True, timeout=300)
        assert r.returncode == 2 and r.stdout == "" and r.stderr.strip()


@pytest.mark.parametrize("name", list(bench.WORKLOADS))
def test_work_accounting_is_positive_and_names_a_kernel_group(name):
    w = bench.WORKLOADS[name]()
    assert w.name == name and w.bound in ("hbm", "mfma") and w.description
    assert w.peak in (bench.HBM_PEAK_GBS, bench.MFMA_PEAK_TFLOPS)


def test_relative_attention_flop_count():
    w = bench.RelSelfAttnWL()
    t, b, e, h = w.T, w.B, w.E, w.H
    tok, d = t * b, e // h
    products_fwd = {"in": 2 * tok * e * 3 * e, "pos": 2 * tok * e * e, "ac": 2 * b * h * t * t * d, "bd": 2 * b * h * t * t * d,
                    "pv": 2 * b * h * t * t * d, "out": 2 * tok * e * e}
    total = sum(products_fwd.values()) + 2 * sum(v for k, v in products_fwd.items() if k != "pos") + products_fwd["pos"]
    assert w.work_per_step() == total
