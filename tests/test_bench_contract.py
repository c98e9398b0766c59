"""What bench.py promises without a GPU: one GPU only, the headline's sizes by default, shapes whose
sizes the configuration class accepts, and a count of operations that follows the sizes."""

import importlib.util
from pathlib import Path

from torchllms_amd.config import LlamaConfig

spec = importlib.util.spec_from_file_location("bench", Path(__file__).resolve().parent.parent / "bench.py")
bench = importlib.util.module_from_spec(spec)
spec.loader.exec_module(bench)


def test_more_than_one_gpu_is_refused_with_a_line_and_status_2(capsys):
    assert bench.main(["--gpus", "2"]) == 2
    out = capsys.readouterr().out.strip().splitlines()
    assert len(out) == 1 and "one GPU" in out[0]


def test_defaults_are_the_headline():
    args = bench.parse_args([])
    assert (args.gpus, args.batch, args.context, args.prefill_tokens, args.points, args.shape, args.workload) == (1, 8, 8192, 2048, "1,64", "8b", "decode")
    cfg = LlamaConfig.from_dict(bench.SHAPES["8b"])
    assert (cfg.hidden_size, cfg.num_hidden_layers, cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim,
            cfg.intermediate_size, cfg.vocab_size) == (4096, 32, 32, 8, 128, 14336, 128256)


def test_every_shape_is_a_valid_configuration():
    sizes = {name: LlamaConfig.from_dict(shape) for name, shape in bench.SHAPES.items()}
    assert sizes["1b"].head_dim == 64 and sizes["1b"].tie_word_embeddings and sizes["1b"].num_hidden_layers == 16
    assert sizes["70b"].hidden_size == 8192 and sizes["70b"].num_hidden_layers == 80 and sizes["70b"].num_key_value_heads == 8
    assert set(bench.SHAPE_NAMES) == set(bench.SHAPES)


def test_prefill_operations_follow_the_sizes():
    cfg = LlamaConfig.from_dict(bench.SHAPES["8b"])
    one = bench.prefill_flops(cfg, 1, 2048)
    two = bench.prefill_flops(cfg, 2, 2048)
    head = 2 * cfg.hidden_size * cfg.vocab_size
    assert two - one == one - head  # every layer costs the same, the output matrix once for the one wanted row
    # per layer: projections 2 T D (Hq + 2 Hkv) dh + 2 T Hq dh D, feed-forward 6 T D F, attention 4 Hq dh T (T + 1) / 2
    T, D, F = 2048, cfg.hidden_size, cfg.intermediate_size
    layer = 2 * T * D * (32 + 16) * 128 + 2 * T * 32 * 128 * D + 6 * T * D * F + 4 * 32 * 128 * T * (T + 1) / 2
    assert one - head == layer
