"""bench.py's handling of its child process (the step variants that are not the library's defaults
run there): whatever the child does -- an error status, no output, lines that are not JSON, running
past its time -- the parent keeps the lines the child had written and says how it ended.  No GPU."""
import argparse
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
import bench  # noqa: E402


def _args():
    return argparse.Namespace(steps=2, warmup=1, batch=1, no_graph=False, serial_only=True,
                              no_autotune=True)


def _with_child(monkeypatch, code):
    monkeypatch.setattr(bench, "CANDIDATE_COMMAND", [sys.executable, "-c", code])


def test_complete_child(monkeypatch):
    _with_child(monkeypatch, "import sys, json\n"
                "assert sys.argv[1:] == ['--candidates', '--steps', '2', '--warmup', '1', '--batch', '1',"
                " '--serial-only', '--no-autotune'], sys.argv\n"
                "print(json.dumps({'candidate': 'a', 'ms_per_step': 1.5, 'enqueue_ms_per_step': 0.1}))\n"
                "print(json.dumps({'done': True}))")
    lines, note = bench.candidates_from_child(_args())
    assert note is None
    assert lines[0]["candidate"] == "a" and lines[-1] == {"done": True}


def test_child_that_dies_keeps_its_lines(monkeypatch):
    _with_child(monkeypatch, "import os, sys, json\n"
                "print(json.dumps({'candidate': 'a', 'ms_per_step': 1.5, 'enqueue_ms_per_step': 0.1}))\n"
                "print('not json at all')\nprint('[1, 2]')\n"
                "sys.stdout.flush()\nos.abort()")
    lines, note = bench.candidates_from_child(_args())
    assert [d.get("candidate") for d in lines] == ["a"]
    assert note is not None and "status" in note


def test_child_that_overruns_is_stopped(monkeypatch):
    _with_child(monkeypatch, "import sys, json, time\n"
                "print(json.dumps({'candidate': 'a', 'error': 'x'}))\nsys.stdout.flush()\ntime.sleep(60)")
    lines, note = bench.candidates_from_child(_args(), timeout_s=2)
    assert [d.get("candidate") for d in lines] == ["a"]
    assert "stopped" in note


def test_child_that_cannot_start(monkeypatch):
    monkeypatch.setattr(bench, "CANDIDATE_COMMAND", ["/nonexistent/interpreter"])
    lines, note = bench.candidates_from_child(_args())
    assert lines == [] and note


def test_more_than_one_gpu_is_refused():
    import subprocess
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"],
                       stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
    assert p.returncode == 2 and "one GPU" in p.stderr
