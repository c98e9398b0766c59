"""bin/trace_run as a user runs it: a subprocess fed steps on standard input."""

import json
import subprocess
from pathlib import Path

import numpy as np
import pytest
import torch

from . import schedules
from .helpers import TINY, make_folder, random_tokens, read_folder
from .plain import llama as plain

pytestmark = pytest.mark.gpu
ROOT = Path(__file__).resolve().parent.parent


def replay(folder, dtype, steps, out_dir, max_tokens):
    """Run bin/trace_run, feeding one step at a time and waiting for its ``done`` line."""
    cmd = [str(ROOT / "bin" / "trace_run"), "--model", str(folder), "--dtype", dtype, "--out", str(out_dir), "--max-tokens", str(max_tokens)]
    proc = subprocess.Popen(cmd, stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True)
    try:
        for s in steps:
            proc.stdin.write(json.dumps(s) + "\n")
            proc.stdin.flush()
            line = proc.stdout.readline().strip()
            assert line == f"done {s['step']}", f"expected 'done {s['step']}', got {line!r}"
        proc.stdin.close()
        assert proc.wait(timeout=120) == 0
    finally:
        if proc.poll() is None:
            proc.kill()
    out = {}
    for s, where in zip(steps, schedules.positions_of(steps)):
        f = Path(out_dir) / f"{s['step']}.f32"
        if not where:
            assert not f.exists()
            continue
        arr = np.fromfile(f, dtype="<f4")
        arr = arr.reshape(len(where), -1)
        for key, row in zip(where, arr):
            out[key] = torch.from_numpy(row.copy())
    return out


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_mixed_schedule(tmp_path, dtype):
    cfg_dict = TINY["B"]
    folder = make_folder(tmp_path / "model", cfg_dict, seed=21, dtype=torch.bfloat16, sharpen=True)
    cfg, weights = read_folder(folder)
    requests = {f"q{i}": random_tokens(n, cfg["vocab_size"], 300 + i) for i, n in enumerate([70, 33, 120, 48, 64])}
    steps = schedules.mixed(requests)
    # a step in which nothing is wanted writes no file
    steps[1]["entries"][0]["want"] = steps[1]["entries"][0]["want"][:0] if len(steps[1]["entries"]) == 1 else steps[1]["entries"][0]["want"]
    got = replay(folder, dtype, steps, tmp_path / "out", schedules.max_live_tokens(steps))
    truth = {rid: plain.forward(weights, cfg, t, torch.float32) for rid, t in requests.items()}
    if dtype == "float32":
        tol = 2e-5
    else:
        tol = 2 * max((plain.forward(weights, cfg, t, torch.bfloat16).float() - truth[rid]).abs().max().item() for rid, t in requests.items())
    assert got
    for (rid, pos), row in got.items():
        assert row.shape[0] == cfg["vocab_size"]
        assert (row - truth[rid][pos]).abs().max().item() <= tol, f"{rid} position {pos}"


def test_trace_run_whole_equals_tail_bitwise_in_float32(tmp_path):
    cfg_dict = TINY["A"]
    folder = make_folder(tmp_path / "model", cfg_dict, seed=22, dtype=torch.bfloat16, sharpen=True)
    requests = {"a": random_tokens(80, 256, 1), "b": random_tokens(45, 256, 2)}
    a = replay(folder, "float32", schedules.whole(requests), tmp_path / "o1", 128)
    b = replay(folder, "float32", schedules.tail(requests), tmp_path / "o2", 128)
    assert set(a) == set(b) and all(torch.equal(a[k], b[k]) for k in a)
