"""bin/trace_run as a user runs it: a child process fed one JSON step a line, answering
``done <step>`` and writing <step>.f32; every way of cutting the requests is compared with
the plain implementation, in 32-bit and in bfloat16."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain
import tiny
import traces

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TOL = {"float32": 2e-5, "bfloat16": 2e-2}        # as in test_engine_gpu.py


def run_trace(model_dir, dtype, steps, out_dir, max_tokens, extra=()):
    cmd = [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", model_dir,
           "--dtype", dtype, "--out", out_dir, "--max-tokens", str(max_tokens)] + list(extra)
    p = subprocess.Popen(cmd, stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)
    try:
        for st in steps:
            p.stdin.write(json.dumps(st) + "\n")
            p.stdin.flush()
            line = p.stdout.readline().strip()      # the next step only after this answer
            assert line == f"done {st['step']}", f"step {st['step']}: got {line!r}"
        p.stdin.close()
        assert p.wait(timeout=120) == 0
    finally:
        if p.poll() is None:
            p.kill()
    return {st["step"]: np.fromfile(os.path.join(out_dir, f"{st['step']}.f32"), dtype="<f4")
            for st in steps if any(e["want"] for e in st["entries"])}


@pytest.mark.parametrize("name,dtype", [("A", "float32"), ("D", "bfloat16"), ("B", "bfloat16"),
                                        ("D", "float32"), ("E", "bfloat16")])
def test_every_cutting_through_trace_run(name, dtype, tmp_path):
    store = torch.float32 if dtype == "float32" else torch.bfloat16
    model_dir = tiny.model_dir_of(name, str(tmp_path), store)
    cfg = tiny.CONFIGS[name]
    V = cfg["vocab_size"]
    lens = {"A": (40, 70, 5, 100), "B": (33, 130, 64, 9, 80), "D": (97, 300, 31, 150, 64),
            "E": (40, 150, 64, 333, 20)}[name]
    requests = {f"t{i}": tiny.random_tokens(n, V, 900 + i) for i, n in enumerate(lens)}
    w = tiny.weights_of(name, store)
    ref = {rid: plain.model_forward_batched(cfg, w, t).numpy() for rid, t in requests.items()}
    # one trace: whole, then most + last 32 one by one, then changing portions, then mixed
    steps = []
    for k, mode in enumerate((traces.whole, traces.prefill_then_single,
                              traces.changing_portions, traces.mixed)):
        renamed = {f"{rid}/{k}": t for rid, t in requests.items()}
        for st in mode(renamed):
            st["step"] = len(steps)
            steps.append(st)
    peak = traces.peak_tokens(steps, 64)
    # the configuration's own page size goes through the program's option (B: pages of 8)
    outs = run_trace(model_dir, dtype, steps, str(tmp_path / "out"), peak,
                     ["--page-size", str(tiny.PAGE_SIZE[name])])
    got = traces.collect(steps, outs, V)
    assert len(got) == 4 * len(requests)
    for rid_k, rows in got.items():
        rid = rid_k.split("/")[0]
        err = np.abs(rows.astype(np.float64) - ref[rid]).max(axis=1) / np.abs(ref[rid]).max()
        bad = np.nonzero(err > TOL[dtype])[0]
        assert bad.size == 0, f"{rid_k}: first wrong position {bad[0]} (error {err[bad[0]]:.3g})"
    # the pool was made for `peak` tokens: pages were used again
    total = sum((len(t) + 63) // 64 * 64 for t in requests.values()) * 4
    assert peak < total


def test_pool_and_slots_from_options(tmp_path):
    """--num-pages and --max-requests size the pool and the slots themselves: a trace that
    fits runs, one page or one slot fewer is CacheFull."""
    model_dir = tiny.model_dir_of("B", str(tmp_path), torch.float32)
    cfg = tiny.CONFIGS["B"]
    V = cfg["vocab_size"]
    reqs = {f"n{i}": tiny.random_tokens(n, V, 40 + i) for i, n in enumerate((20, 9, 17))}
    w = tiny.weights_of("B", torch.float32)
    steps = [{"step": 0, "entries": [{"id": r, "tokens": t, "want": [len(t) - 1], "start": 0}
                                     for r, t in reqs.items()], "end": list(reqs)}]
    pages = sum((len(t) + 3) // 4 for t in reqs.values())       # pages of 4 tokens
    base = ["--page-size", "4"]
    outs = run_trace(model_dir, "float32", steps, str(tmp_path / "o1"), 64,
                     base + ["--num-pages", str(pages), "--max-requests", "3"])
    got = outs[0].reshape(3, V)
    for i, (r, t) in enumerate(reqs.items()):
        ref = plain.model_forward_batched(cfg, w, t).numpy()[-1]
        assert np.abs(got[i] - ref).max() <= TOL["float32"] * np.abs(ref).max()
    for extra in (["--num-pages", str(pages - 1), "--max-requests", "3"],
                  ["--num-pages", str(pages), "--max-requests", "2"]):
        cmd = [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", model_dir,
               "--dtype", "float32", "--out", str(tmp_path / "o2"), "--max-tokens", "64"] \
            + base + extra
        r = subprocess.run(cmd, input=json.dumps(steps[0]) + "\n", capture_output=True,
                           text=True, timeout=300)
        assert r.returncode == 1 and "CacheFull" in r.stderr and "done" not in r.stdout, extra


def test_a_position_gap_is_an_error(tmp_path):
    """An entry that says where it starts must start where the request's tokens end."""
    model_dir = tiny.model_dir_of("A", str(tmp_path), torch.float32)
    cmd = [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", model_dir,
           "--dtype", "float32", "--out", str(tmp_path / "o"), "--max-tokens", "128"]
    first = {"step": 0, "entries": [{"id": "a", "tokens": [1, 2, 3], "want": [], "start": 0}],
             "end": []}
    for start, words in ((5, "tokens 3..4 were never given"), (2, "tokens 2..2 are held already")):
        second = {"step": 1, "entries": [{"id": "a", "tokens": [4, 5], "want": [1],
                                          "start": start}], "end": []}
        r = subprocess.run(cmd, input=json.dumps(first) + "\n" + json.dumps(second) + "\n",
                           capture_output=True, text=True, timeout=300)
        assert r.returncode == 1 and "done 0" in r.stdout and "done 1" not in r.stdout
        assert "PositionGap" in r.stderr and "'a'" in r.stderr and words in r.stderr, r.stderr
    # a new request must start at 0
    r = subprocess.run(cmd, input=json.dumps({"step": 0, "entries": [
        {"id": "z", "tokens": [1], "want": [0], "start": 7}], "end": []}) + "\n",
        capture_output=True, text=True, timeout=300)
    assert r.returncode == 1 and "PositionGap" in r.stderr


def test_errors_are_reported_not_papered_over(tmp_path):
    model_dir = tiny.model_dir_of("A", str(tmp_path), torch.float32)
    cmd = [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", model_dir,
           "--dtype", "float32", "--out", str(tmp_path / "o"), "--max-tokens", "64"]
    step = {"step": 0, "entries": [{"id": "a", "tokens": [1] * 65, "want": []}], "end": []}
    r = subprocess.run(cmd, input=json.dumps(step) + "\n", capture_output=True, text=True,
                       timeout=300)
    assert r.returncode == 1 and "CacheFull" in r.stderr and "done" not in r.stdout
    bad = tmp_path / "bad"
    bad.mkdir()
    (bad / "config.json").write_text(json.dumps(dict(tiny.TINY_A, model_type="mystery",
                                                     architectures=["Mystery"])))
    cmd[cmd.index("--model") + 1] = str(bad)
    r = subprocess.run(cmd, input="", capture_output=True, text=True, timeout=300)
    assert r.returncode == 1 and "UnsupportedModelType" in r.stderr
