"""Random weights from a configuration and a seed, and a model folder written from them.

Every tensor has a generator of its own, seeded from ``(seed, tensor name)``, so a tensor's values
depend neither on the order of creation nor on which other tensors exist.  Matrices and embeddings
are N(0, 0.02), norm weights ones, biases zeros, as the reference initialises what a checkpoint
lacks (reference: torchllms/models/utils.py:197-214, networks.py:192-193).  Values are drawn in
32-bit and then cast, so a 32-bit and a bfloat16 model of one seed agree up to rounding.
"""

from __future__ import annotations

import hashlib
import json
from pathlib import Path
from typing import Dict, Optional

import torch

from ..config.registry import ArchSpec, architecture_of, get_architecture
from ..parts.base import ParamSpec
from ..parts.model import Model

INIT_STD = 0.02


def _tensor_seed(seed: int, name: str) -> int:
    digest = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    return int.from_bytes(digest[:8], "little") & 0x7FFFFFFFFFFFFFFF


def random_tensor(name: str, spec: ParamSpec, seed: int, dtype: torch.dtype, norm_jitter: float = 0.0, device="cpu") -> torch.Tensor:
    """One tensor of the random-weights mode.  ``norm_jitter`` > 0 draws "ones" tensors as
    1 + N(0, norm_jitter) instead, so a misplaced norm weight shows in a comparison."""
    gen = torch.Generator(device=device)
    gen.manual_seed(_tensor_seed(seed, name))
    if spec.kind == "int":
        return torch.zeros(spec.shape, dtype=torch.int32, device=device)
    if spec.init == "normal":
        t = torch.empty(spec.shape, dtype=torch.float32, device=device).normal_(0.0, INIT_STD, generator=gen)
    elif spec.init == "ones":
        t = torch.ones(spec.shape, dtype=torch.float32, device=device)
        if norm_jitter > 0:
            t += torch.empty(spec.shape, dtype=torch.float32, device=device).normal_(0.0, norm_jitter, generator=gen)
    elif spec.init == "zeros":
        t = torch.zeros(spec.shape, dtype=torch.float32, device=device)
        if norm_jitter > 0:
            t += torch.empty(spec.shape, dtype=torch.float32, device=device).normal_(0.0, INIT_STD, generator=gen)
    else:
        raise ValueError(f"{name}: unknown init {spec.init!r}")
    return t.to(dtype)


def random_tensors(
    expected: Dict[str, ParamSpec], seed: int, dtype: torch.dtype, norm_jitter: float = 0.0, device="cpu"
) -> Dict[str, torch.Tensor]:
    """All tensors of a model under the parts' own names.  With ``device`` a GPU the values are
    drawn there (faster for large models; they then differ from the CPU's for the same seed)."""
    return {name: random_tensor(name, spec, seed, dtype, norm_jitter, device) for name, spec in expected.items()}


def write_model_folder(
    folder,
    config,
    seed: int,
    dtype: torch.dtype = torch.bfloat16,
    norm_jitter: float = 0.0,
    arch: Optional[ArchSpec] = None,
) -> Path:
    """Write ``config.json`` and ``model.safetensors`` (checkpoint tensor names and layout) for a
    model of this configuration with random weights."""
    from safetensors.torch import save_file

    arch = arch or architecture_of(config)
    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    model = Model(arch.model_spec(config))
    rules = arch.weight_rules(config)
    tensors = {}
    for name, spec in model.param_specs().items():
        t = random_tensor(name, spec, seed, dtype, norm_jitter)
        for rule in rules:
            ext = rule.match_internal(name)
            if ext is not None:
                if rule.save is not None:
                    t = rule.save(t)
                tensors[ext] = t.contiguous()
                break
        else:
            raise KeyError(f"no rule names the tensor {name}")
    with open(folder / "config.json", "w") as f:
        json.dump(arch.config_json(config), f, indent=2)
    save_file(tensors, str(folder / "model.safetensors"), metadata={"format": "pt"})
    return folder


def main(argv=None) -> int:
    """``python -m torchllms_amd.weights.random_init --config config.json --seed 0 --out DIR``:
    the random-weights mode from the command line.  The architecture named in the configuration
    picks the model, as everywhere."""
    import argparse
    import json

    p = argparse.ArgumentParser(prog="python -m torchllms_amd.weights.random_init", description=main.__doc__)
    p.add_argument("--config", required=True, help="a config.json (or a model folder that holds one)")
    p.add_argument("--seed", type=int, default=0)
    p.add_argument("--out", required=True, help="folder that receives config.json and model.safetensors")
    p.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"], help="dtype of the stored tensors")
    p.add_argument("--norm-jitter", type=float, default=0.0, help="norm weights are 1 + N(0, this) instead of 1")
    args = p.parse_args(argv)
    path = Path(args.config)
    if path.is_dir():
        path = path / "config.json"
    with open(path) as f:
        raw = json.load(f)
    names = raw.get("architectures") or []
    if not names:
        raise SystemExit(f"{path} names no architecture (key \"architectures\")")
    arch = get_architecture(names[0])
    config = arch.config_from_dict(raw)
    dtype = torch.bfloat16 if args.dtype == "bfloat16" else torch.float32
    folder = write_model_folder(args.out, config, args.seed, dtype=dtype, norm_jitter=args.norm_jitter, arch=arch)
    print(f"wrote {folder / 'config.json'} and {folder / 'model.safetensors'} (seed {args.seed}, {args.dtype})")
    return 0


if __name__ == "__main__":
    import sys

    sys.exit(main())
