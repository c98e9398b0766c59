"""The engine at the layer sizes of a real model (hidden 4096, 32 heads in 8 groups of head size
128, feed-forward 14336, llama3 rope scaling; two layers and a small vocabulary to keep it quick):
the kernels' paths that tiny configurations do not reach (the decode products' measured launch
choices, the MFMA attention kernels at head size 128, long rows in the norms)."""

import pytest
import torch

from . import schedules
from .helpers import make_folder, random_tokens, read_folder
from .plain import llama as plain
from .test_gpu_engine import FP32_ATOL, run_trace

pytestmark = pytest.mark.gpu

REAL = dict(
    architectures=["LlamaForCausalLM"], hidden_size=4096, num_hidden_layers=2, num_attention_heads=32,
    num_key_value_heads=8, head_dim=128, intermediate_size=14336, vocab_size=1000, rms_norm_eps=1e-5,
    rope_theta=500000.0, max_position_embeddings=8192, tie_word_embeddings=False,
    rope_scaling=dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                      original_max_position_embeddings=8192),
)
LENGTHS = [150, 70, 333, 40]


@pytest.fixture(scope="module")
def real(tmp_path_factory):
    folder = make_folder(tmp_path_factory.mktemp("real") / "m", REAL, seed=3, dtype=torch.bfloat16, norm_jitter=0.1, sharpen=True)
    cfg, weights = read_folder(folder)
    requests = {f"r{i}": random_tokens(n, REAL["vocab_size"], 40 + i) for i, n in enumerate(LENGTHS)}
    truth = {rid: plain.forward(weights, cfg, t, torch.float32) for rid, t in requests.items()}
    yard = {rid: plain.forward(weights, cfg, t, torch.bfloat16).float() for rid, t in requests.items()}
    traces = {"whole": schedules.whole(requests), "tail": schedules.tail(requests), "mixed": schedules.mixed(requests)}
    return folder, requests, truth, yard, traces


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_real_layer_sizes_match_the_plain_model_under_every_schedule(real, dtype):
    from torchllms_amd.engine import Engine

    folder, requests, truth, yard, traces = real
    pool_tokens = max(schedules.max_live_tokens(t) for t in traces.values())
    eng = Engine.from_folder(folder, dtype=dtype, page_size=16, num_pages=-(-pool_tokens // 16), max_seqs=4)
    results = {name: run_trace(eng, trace) for name, trace in traces.items()}
    for name, res in results.items():
        for (rid, pos), row in res.items():
            want = truth[rid][pos]
            if dtype == "float32":
                err = (row - want).abs().max().item()
                assert err < 10 * FP32_ATOL, f"{name}: {rid} position {pos}: {err}"  # sums are 64 times longer than in the tiny models
            else:
                tol = 2 * (yard[rid][pos] - want).abs().max().item() + 1e-3
                assert (row - want).abs().max().item() <= tol, f"{name}: {rid} position {pos}"
    if dtype == "float32":
        for name in ("tail", "mixed"):
            for key, row in results[name].items():
                assert torch.equal(row, results["whole"][key]), f"{name} differs from whole at {key}"
