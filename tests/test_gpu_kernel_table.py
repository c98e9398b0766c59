"""The table of measured matrix-product kernel choices, carried from one engine to another: kernels
differ in rounding (the order of a sum split along K, a library's tiles), so bfloat16 logits repeat
bit for bit only between engines that run from the same table."""

import json
import os
import subprocess
import sys

import pytest
import torch

from . import schedules
from .helpers import TINY_B, make_folder, random_tokens
from .test_gpu_engine import run_trace

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
# K = 256 is a multiple of 128, so all three kinds of kernel are candidates for this model's matrices
CONFIG = dict(TINY_B, num_hidden_layers=2, num_key_value_heads=2, intermediate_size=640)


def _trace():
    requests = {f"r{i}": random_tokens(n, CONFIG["vocab_size"], 900 + i) for i, n in enumerate([70, 41, 100, 35, 50])}
    return schedules.mixed(requests)


def test_engines_built_from_one_table_agree_bit_for_bit(tmp_path, monkeypatch):
    from torchllms_amd.engine import Engine
    from torchllms_amd.kernels import ops, products

    folder = make_folder(tmp_path / "m", CONFIG, seed=2, dtype=torch.bfloat16, sharpen=True)
    steps = _trace()
    pool = -(-schedules.max_live_tokens(steps) // 16)
    ops.clear_kernel_table()
    first = Engine.from_folder(folder, dtype="bfloat16", page_size=16, num_pages=pool, max_seqs=4)
    table = first.kernel_table()
    # an entry for every matrix shape of the model, every row bucket and the use the part makes of it
    shapes = {(tuple(shape), use) for (shape, use, _) in first.model.linear_weights()}
    assert {tuple(k.split(",")[:2] + [k.split(",")[3]]) for k in table} == {(str(s[0]), str(s[1]), use) for s, use in shapes}
    assert len(table) == len(shapes) * len(ops.ROW_BUCKETS)
    want = run_trace(first, steps)
    path = tmp_path / "kernels.json"
    ops.save_kernel_table(path, shapes)
    assert json.loads(path.read_text()) == table

    # another engine, as another process would build it: nothing measured yet, the table from the file,
    # and no stopwatch (a measurement now would be a fault)
    ops.clear_kernel_table()
    monkeypatch.setattr(torch.cuda.Event, "elapsed_time", lambda *a: pytest.fail("the engine measured although it had a table"))
    second = Engine.from_folder(folder, dtype="bfloat16", page_size=16, num_pages=pool, max_seqs=4, kernel_table=str(path))
    assert second.kernel_table() == table
    got = run_trace(second, steps)
    assert all(torch.equal(got[k], want[k]) for k in want)

    # the table decides, not the rule of sizes: with every product sent to the library the engine obeys
    ops.clear_kernel_table()
    library = {k: None for k in table}
    third = Engine.from_folder(folder, dtype="bfloat16", page_size=16, num_pages=pool, max_seqs=4, kernel_table=library)
    assert third.kernel_table() == library
    x = torch.zeros((4, 256), dtype=torch.bfloat16, device="cuda:0")
    assert ops.linear_choice(x, third.model.blocks[0].mixer.wo, "sum") is None
    near = run_trace(third, steps)
    worst = max((near[k] - want[k]).abs().max().item() for k in want)
    assert worst < 0.5  # the same model through other kernels: near, not equal
    ops.clear_kernel_table()

    # without a table and without measurement the choice is a fixed rule, the same in every process
    plain_rule = Engine.from_folder(folder, dtype="bfloat16", page_size=16, num_pages=pool, max_seqs=4, tune_kernels=False)
    assert plain_rule.kernel_table() == {} and products.LINEAR_CHOICE == {}
    assert ops.linear_choice(x, plain_rule.model.blocks[0].mixer.wo, "sum") == ("stream", 0)


def test_a_table_that_names_no_launch_is_refused():
    from torchllms_amd.kernels import ops

    for bad in ({"256,256,8": None}, {"256,256,7,plain": None}, {"256,256,8,plain": ["wide", 1, 1, 3]},
                {"256,256,64,plain": ["stream", 0]}, {"256,256,64,plain": ["wide", 9, 9, 9]}, {"256,200,64,plain": ["wide", 1, 1, 3]},
                {"256,256,8,plain": ["stream", 0, 8]}, {"256,256,8,magic": None}):
        with pytest.raises(ValueError, match="kernel table"):
            ops.load_kernel_table(bad)


def test_trace_run_writes_and_reads_a_kernel_table(tmp_path):
    folder = make_folder(tmp_path / "m", CONFIG, seed=2, dtype=torch.bfloat16, sharpen=True)
    steps = _trace()
    text = "".join(json.dumps(s) + "\n" for s in steps)
    table = tmp_path / "kernels.json"
    outs = []
    for run in range(2):
        out = tmp_path / f"out{run}"
        cmd = [os.path.join(ROOT, "bin", "trace_run"), "--model", str(folder), "--dtype", "bfloat16", "--out", str(out),
               "--max-tokens", str(schedules.max_live_tokens(steps)), "--kernel-table", str(table)]
        proc = subprocess.run(cmd, input=text, capture_output=True, text=True, timeout=300)
        assert proc.returncode == 0, proc.stderr[-2000:]
        assert "matrix-product kernels" in proc.stderr
        assert table.is_file()
        outs.append({p.name: p.read_bytes() for p in sorted(out.glob("*.f32"))})
    assert outs[0].keys() == outs[1].keys() and len(outs[0]) == len(steps)
    assert outs[0] == outs[1]  # two processes, one table: the same bits
