"""Weight loading by name, its one error, re-layout of q/k rows, random-weights mode (CPU)."""

import json

import pytest
import torch
from safetensors.torch import save_file

from torchllms_amd.config import LlamaConfig, get_architecture, load_config
from torchllms_amd.parts import Model
from torchllms_amd.weights import (
    WeightError,
    half_split_to_interleaved,
    interleaved_to_half_split,
    load_weights,
    random_tensors,
)

from .helpers import TINY_A, TINY_B, TINY_C, make_folder, read_folder
from .plain import llama as plain


def _expected(cfg_dict):
    cfg = LlamaConfig.from_dict(cfg_dict)
    arch = get_architecture("LlamaForCausalLM")
    return cfg, arch, Model(arch.model_spec(cfg)).param_specs()


def _load(folder, cfg_dict, dtype=torch.float32):
    cfg, arch, expected = _expected(cfg_dict)
    ignore = ["head.weight"] if "head.weight" not in expected else []
    return load_weights(folder, arch.weight_rules(cfg), expected, dtype, ignore_when_present=ignore)


def test_permutation_matches_the_plain_one_and_inverts():
    torch.manual_seed(0)
    w = torch.randn(3 * 8, 5)
    assert torch.equal(half_split_to_interleaved(w, 3, 8), plain.permute_rows_for_interleaved(w, 3, 8))
    assert torch.equal(interleaved_to_half_split(half_split_to_interleaved(w, 3, 8), 3, 8), w)
    b = torch.randn(24)
    assert torch.equal(half_split_to_interleaved(b, 3, 8), plain.permute_rows_for_interleaved(b, 3, 8))
    with pytest.raises(ValueError):
        half_split_to_interleaved(w, 4, 8)


@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_folder_round_trip(tmp_path, name):
    cfg_dict = {"A": TINY_A, "B": TINY_B, "C": TINY_C}[name]
    folder = make_folder(tmp_path, cfg_dict, seed=3)
    cfg, arch, expected = _expected(cfg_dict)
    got = _load(folder, cfg_dict, torch.bfloat16)
    assert set(got) == set(expected)
    for n, spec in expected.items():
        assert tuple(got[n].shape) == spec.shape and got[n].dtype == torch.bfloat16
    # names in the file are the checkpoint's own, q/k rows in the checkpoint's layout
    _, raw = read_folder(folder)
    assert "model.layers.0.self_attn.q_proj.weight" in raw and "model.norm.weight" in raw
    assert ("lm_head.weight" in raw) == (not cfg.tie_word_embeddings)
    q = raw["model.layers.0.self_attn.q_proj.weight"]
    assert torch.equal(got["layers.0.mixer.wq.weight"], half_split_to_interleaved(q, cfg.num_attention_heads, cfg.head_dim))
    assert torch.equal(got["layers.0.mixer.wv.weight"], raw["model.layers.0.self_attn.v_proj.weight"])
    # the same values as the in-memory random mode
    direct = random_tensors(expected, 3, torch.bfloat16, norm_jitter=0.1)
    for n in expected:
        assert torch.equal(direct[n], got[n]), n


def test_random_values_do_not_depend_on_order_and_follow_the_rule():
    cfg, arch, expected = _expected(TINY_B)
    a = random_tensors(expected, 7, torch.float32)
    b = random_tensors(dict(reversed(list(expected.items()))), 7, torch.float32)
    for n in expected:
        assert torch.equal(a[n], b[n])
    assert torch.equal(a["layers.1.mixer_norm.weight"], torch.ones(256))
    w = a["layers.0.ffn.w1.weight"]
    assert abs(w.std().item() - 0.02) < 0.002 and abs(w.mean().item()) < 0.001
    c = random_tensors(expected, 8, torch.float32)
    assert not torch.equal(a["embed.weight"], c["embed.weight"])
    # bfloat16 values are the rounded 32-bit ones
    h = random_tensors(expected, 7, torch.bfloat16)
    assert torch.equal(h["embed.weight"], a["embed.weight"].bfloat16())


def test_reference_spelling_is_taken_as_is(tmp_path):
    cfg, arch, expected = _expected(TINY_A)
    internal = random_tensors(expected, 1, torch.float32)
    ref_names = {
        "embed.weight": "tok_embeddings.weight",
        "final_norm.weight": "norm.weight",
    }
    out = {}
    for n, t in internal.items():
        if n in ref_names:
            out[ref_names[n]] = t
        else:
            i = n.split(".")[1]
            rest = n.split(".", 2)[2]
            rest = (rest.replace("mixer_norm", "attention_norm").replace("mixer.", "attention.").replace("ffn.", "feed_forward."))
            out[f"layers.{i}.{rest}"] = t
    save_file(out, str(tmp_path / "model.safetensors"))
    cfg.save(tmp_path)
    got = _load(tmp_path, TINY_A)
    for n in expected:
        assert torch.equal(got[n], internal[n]), n


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    folder = make_folder(tmp_path, TINY_B, seed=0)
    _, raw = read_folder(folder)
    del raw["model.layers.1.mlp.up_proj.weight"]
    del raw["model.norm.weight"]
    raw["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(16)  # known and dropped
    raw["model.layers.7.mlp.up_proj.weight"] = torch.zeros(688, 256)  # no such layer
    raw["some.other.tensor"] = torch.zeros(3)
    raw["model.layers.2.self_attn.k_proj.weight"] = torch.zeros(64, 256)  # should be [32, 256]
    save_file(raw, str(folder / "model.safetensors"))
    with pytest.raises(WeightError) as ei:
        _load(folder, TINY_B)
    err = ei.value
    assert err.missing == ["model.layers.1.mlp.up_proj.weight", "model.norm.weight"]
    assert err.unexpected == ["model.layers.7.mlp.up_proj.weight", "some.other.tensor"]
    assert err.wrong_shape == [("model.layers.2.self_attn.k_proj.weight", (64, 256), (32, 256))]
    msg = str(err)
    for piece in ("missing (2)", "unexpected (2)", "wrong shape (1)", "model.norm.weight", "some.other.tensor", "[64, 256]", "[32, 256]"):
        assert piece in msg


def test_tied_and_untied_heads(tmp_path):
    # tied: an output matrix in the file is ignored with a warning
    folder = make_folder(tmp_path / "a", TINY_A, seed=0)
    _, raw = read_folder(folder)
    raw["lm_head.weight"] = torch.zeros(256, 64)
    save_file(raw, str(folder / "model.safetensors"))
    with pytest.warns(UserWarning, match="lm_head.weight"):
        got = _load(folder, TINY_A)
    assert "head.weight" not in got
    # untied: a missing output matrix is an error
    folder = make_folder(tmp_path / "b", TINY_B, seed=0)
    _, raw = read_folder(folder)
    del raw["lm_head.weight"]
    save_file(raw, str(folder / "model.safetensors"))
    with pytest.raises(WeightError, match="lm_head.weight"):
        _load(folder, TINY_B)


def test_dtypes(tmp_path):
    # stored bfloat16, asked float32: exact upcast
    folder = make_folder(tmp_path / "a", TINY_A, seed=0, dtype=torch.bfloat16)
    _, raw = read_folder(folder)
    got = _load(folder, TINY_A, torch.float32)
    assert got["embed.weight"].dtype == torch.float32
    assert torch.equal(got["embed.weight"], raw["model.embed_tokens.weight"].float())
    # stored float32, asked bfloat16: matrices are rounded, a vector stored in 32-bit stays so
    folder = make_folder(tmp_path / "b", TINY_A, seed=0, dtype=torch.float32)
    got = _load(folder, TINY_A, torch.bfloat16)
    assert got["layers.0.mixer.wq.weight"].dtype == torch.bfloat16
    assert got["layers.0.mixer_norm.weight"].dtype == torch.float32


def test_sharded_folder_and_missing_files(tmp_path):
    folder = make_folder(tmp_path, TINY_A, seed=0)
    _, raw = read_folder(folder)
    names = sorted(raw)
    half = len(names) // 2
    save_file({n: raw[n] for n in names[:half]}, str(folder / "model-00001-of-00002.safetensors"))
    save_file({n: raw[n] for n in names[half:]}, str(folder / "model-00002-of-00002.safetensors"))
    (folder / "model.safetensors").unlink()
    index = {"weight_map": {n: ("model-00001-of-00002.safetensors" if i < half else "model-00002-of-00002.safetensors") for i, n in enumerate(names)}}
    (folder / "model.safetensors.index.json").write_text(json.dumps(index))
    got = _load(folder, TINY_A)
    assert len(got) == len(raw)
    (folder / "model-00002-of-00002.safetensors").unlink()
    with pytest.raises(FileNotFoundError):
        _load(folder, TINY_A)
    empty = tmp_path / "empty"
    empty.mkdir()
    with pytest.raises(FileNotFoundError, match="no safetensors"):
        _load(empty, TINY_A)


def test_random_weights_mode_from_the_command_line(tmp_path):
    """``python -m torchllms_amd.weights.random_init``: a folder from a config.json and a seed; the
    same seed gives the same tensors, the loader takes the folder back without complaint."""
    from safetensors import safe_open

    from torchllms_amd.weights import random_init

    cfg_path = tmp_path / "config.json"
    cfg_path.write_text(json.dumps(TINY_B))
    for out in ("a", "b"):
        assert random_init.main(["--config", str(cfg_path), "--seed", "7", "--out", str(tmp_path / out)]) == 0
    assert json.loads((tmp_path / "a" / "config.json").read_text())["hidden_size"] == TINY_B["hidden_size"]
    with safe_open(str(tmp_path / "a" / "model.safetensors"), framework="pt") as fa, \
            safe_open(str(tmp_path / "b" / "model.safetensors"), framework="pt") as fb:
        assert sorted(fa.keys()) == sorted(fb.keys()) and "model.embed_tokens.weight" in fa.keys()
        for name in fa.keys():
            assert torch.equal(fa.get_tensor(name), fb.get_tensor(name))
            assert fa.get_tensor(name).dtype == torch.bfloat16
    arch, config = load_config(tmp_path / "a")
    expected = Model(arch.model_spec(config)).param_specs()
    tensors = load_weights(tmp_path / "a", arch.weight_rules(config), expected, torch.bfloat16)
    assert set(tensors) == set(expected)
