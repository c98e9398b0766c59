"""Seeded random configurations of the architecture through the engine: head sizes in steps of 16
up to 256, any number of heads and groups (also more query heads per kv head than the MFMA kernels
take), widths, feed-forward sizes and vocabularies that are no power of two, every page size, with
and without biases, scaling and tied head.  Each runs the four schedules in both dtypes.

Yardsticks: in 32-bit the schedules agree bit for bit and the engine stays within 5e-5 of the
largest logit of the plain model (whose own 32-bit run differs from a 64-bit run by up to 1e-5 of
it at these depths; the engine adds each product in one ascending chain, the CPU library in
blocks).  In bfloat16 the engine may be twice as far from the 32-bit truth as the plain model run
in bfloat16."""

import random

import pytest
import torch

from . import schedules
from .helpers import make_folder, random_tokens, read_folder
from .plain import llama as plain
from .test_gpu_engine import _max_err, run_trace

pytestmark = pytest.mark.gpu


def random_config(seed: int):
    r = random.Random(seed)
    head_dim = r.choice(list(range(16, 257, 16)) + [32, 64, 128, 128])
    kv_heads = r.choice([1, 1, 2, 3, 4, 5, 8])
    group = r.choice([1, 2, 3, 4, 4, 5, 7, 8, 16, 17]) if head_dim <= 128 else r.choice([1, 2, 4, 8, 9])
    while kv_heads * group * head_dim > 4096 and kv_heads > 1:
        kv_heads //= 2
    while kv_heads * group * head_dim > 4096:
        group //= 2
    scaling = r.choice([None, {
        "rope_type": "llama3", "factor": r.choice([2.0, 8.0, 32.0]), "low_freq_factor": 1.0,
        "high_freq_factor": r.choice([2.0, 4.0]), "original_max_position_embeddings": r.choice([32, 64, 8192]),
    }])
    cfg = {
        "architectures": ["LlamaForCausalLM"],
        "hidden_size": r.choice([64, 96, 128, 256, 384, 200, 520, 1024, 136]),
        "num_hidden_layers": r.choice([1, 2, 3]),
        "num_attention_heads": kv_heads * group,
        "num_key_value_heads": kv_heads,
        "head_dim": head_dim,
        "intermediate_size": r.choice([192, 688, 208, 384, 1000, 256, 1408, 130]),
        "vocab_size": r.choice([256, 301, 512, 1000, 4099, 32003]),
        "max_position_embeddings": 1024,
        "rms_norm_eps": r.choice([1e-5, 1e-6, 3e-4]),
        "rope_theta": r.choice([10000.0, 500000.0, 1000.0]),
        "rope_scaling": scaling,
        "tie_word_embeddings": r.choice([True, False]),
        "attention_bias": r.choice([False, False, True]),
    }
    lengths = [r.choice([33, 34, 40, 47, 64, 65, 100, 129, 200, 333]) for _ in range(r.choice([3, 5, 6]))]
    return cfg, lengths, r.choice([4, 8, 16, 16, 32])


@pytest.mark.parametrize("seed", [3, 11, 14, 19, 101, 141, 153, 154, 180, 251])
def test_random_configuration(tmp_path, seed):
    from torchllms_amd.engine import Engine

    cfg, lengths, page = random_config(seed)
    print(f"seed {seed}: {cfg} lengths {lengths} page {page}", flush=True)
    folder = make_folder(tmp_path / "m", cfg, seed=seed, dtype=torch.bfloat16, norm_jitter=0.1, sharpen=True)
    cfg, weights = read_folder(folder)
    requests = {f"r{i}": random_tokens(n, cfg["vocab_size"], 100 * seed + i) for i, n in enumerate(lengths)}
    plain32 = {rid: plain.forward(weights, cfg, t, torch.float32) for rid, t in requests.items()}
    plain16 = {rid: plain.forward(weights, cfg, t, torch.bfloat16).float() for rid, t in requests.items()}
    largest = max(v.abs().max().item() for v in plain32.values())
    bf16_err = max((plain16[r] - plain32[r]).abs().max().item() for r in requests)
    traces = {name: getattr(schedules, name)(requests) for name in ("whole", "tail", "portions", "mixed")}
    pool = max(schedules.max_live_tokens(t) for t in traces.values())
    for dtype in ("float32", "bfloat16"):
        engine = Engine.from_folder(folder, dtype=dtype, page_size=page, num_pages=-(-pool // page), max_seqs=4)
        first = None
        for name, trace in traces.items():
            got = run_trace(engine, trace)
            err, where = _max_err(got, plain32)
            if dtype == "bfloat16":
                assert err <= 2 * bf16_err, f"{name}: {where} max abs error {err} vs plain bfloat16 {bf16_err}"
                continue
            assert err < 5e-5 * max(1.0, largest), f"{name}: {where} max abs error {err}, largest logit {largest}"
            if first is None:
                first = got
            else:
                diff = [k for k in first if not torch.equal(first[k], got[k])]
                assert not diff, f"{name}: {len(diff)} positions differ from whole, first {sorted(diff)[0]}"


@pytest.mark.parametrize("head_dim, heads, kv_heads, hidden, page", [(10, 4, 2, 64, 16), (36, 3, 1, 100, 5), (66, 4, 2, 136, 7), (250, 2, 1, 128, 16), (2, 3, 3, 30, 3)])
def test_head_sizes_that_are_no_multiple_of_16(tmp_path, head_dim, heads, kv_heads, hidden, page):
    """The configuration allows any even head size and the engine any page size: sizes that the MFMA kernels
    and the 16-byte loads do not fit (head sizes 2, 10, 36, 66, 250; pages of 3, 5 and 7 tokens) run through
    the plain kernels, right in both dtypes, not refused and not wrong."""
    from torchllms_amd.engine import Engine

    cfg = {"architectures": ["LlamaForCausalLM"], "hidden_size": hidden, "num_hidden_layers": 2, "num_attention_heads": heads,
           "num_key_value_heads": kv_heads, "head_dim": head_dim, "intermediate_size": 130, "vocab_size": 301,
           "max_position_embeddings": 512, "rms_norm_eps": 1e-5, "rope_theta": 10000.0, "tie_word_embeddings": False,
           "attention_bias": True}
    folder = make_folder(tmp_path / "m", cfg, seed=head_dim, dtype=torch.bfloat16, norm_jitter=0.1, sharpen=True)
    cfg, weights = read_folder(folder)
    requests = {f"r{i}": random_tokens(n, 301, 7 * head_dim + i) for i, n in enumerate([33, 70, 47, 129])}
    plain32 = {rid: plain.forward(weights, cfg, t, torch.float32) for rid, t in requests.items()}
    plain16 = {rid: plain.forward(weights, cfg, t, torch.bfloat16).float() for rid, t in requests.items()}
    largest = max(v.abs().max().item() for v in plain32.values())
    bf16_err = max((plain16[r] - plain32[r]).abs().max().item() for r in requests)
    traces = {name: getattr(schedules, name)(requests) for name in ("whole", "mixed")}
    pool = max(schedules.max_live_tokens(t) for t in traces.values())
    for dtype in ("float32", "bfloat16"):
        engine = Engine.from_folder(folder, dtype=dtype, page_size=page, num_pages=-(-pool // page) + 4, max_seqs=4)
        for name, trace in traces.items():
            err, where = _max_err(run_trace(engine, trace), plain32)
            bound = 2 * bf16_err if dtype == "bfloat16" else 5e-5 * max(1.0, largest)
            assert err <= bound, f"{dtype}/{name}: {where} max abs error {err}, bound {bound}"
