"""Reads a model folder's safetensors by tensor name and checks them against what the model expects.

Differences from the reference's loader, on purpose: the reference loads a pickled state dict with
``strict=False``, only warns about missing or unexpected names and re-initialises what is missing at
random (reference: torchllms/models/utils.py:96-164).  Here every expected tensor must be there
exactly once with the expected shape, and one error lists everything that is wrong.
"""

from __future__ import annotations

import json
import warnings
from pathlib import Path
from typing import Dict, Iterable, List, Tuple

import torch

from ..parts.base import ParamSpec
from .names import NameRule


class WeightError(RuntimeError):
    """The tensors in a model folder are not the ones the model needs.

    ``missing``, ``unexpected`` and ``wrong_shape`` hold the details the message lists.
    """

    def __init__(self, folder, missing, unexpected, wrong_shape, duplicates=()):
        self.missing = sorted(missing)
        self.unexpected = sorted(unexpected)
        self.wrong_shape = sorted(wrong_shape)
        self.duplicates = sorted(duplicates)
        lines = [f"weights in {folder} do not match the model:"]
        if self.missing:
            lines.append(f"  missing ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        if self.wrong_shape:
            lines.append(
                f"  wrong shape ({len(self.wrong_shape)}): "
                + ", ".join(f"{n} is {list(got)}, expected {list(want)}" for n, got, want in self.wrong_shape)
            )
        if self.duplicates:
            lines.append(f"  given twice ({len(self.duplicates)}): " + ", ".join(self.duplicates))
        super().__init__("\n".join(lines))


def safetensors_files(folder) -> List[Path]:
    """The shard files of a model folder: those the index names, else ``model.safetensors``, else
    every ``*.safetensors`` in name order (reference: checkpoint_converter.py:273-310 priority)."""
    folder = Path(folder)
    index = folder / "model.safetensors.index.json"
    if index.is_file():
        with open(index) as f:
            names = sorted(set(json.load(f)["weight_map"].values()))
        return [folder / n for n in names]
    single = folder / "model.safetensors"
    if single.is_file():
        return [single]
    files = sorted(folder.glob("*.safetensors"))
    if not files:
        raise FileNotFoundError(f"no safetensors file in {folder}")
    return files


def _final_dtype(spec: ParamSpec, stored: torch.dtype, compute: torch.dtype) -> torch.dtype:
    if spec.kind == "int":
        return torch.int32
    if compute == torch.float32:
        return torch.float32
    if spec.kind == "vector" and stored in (torch.float32, torch.float64):
        return torch.float32  # a tensor stored in 32-bit stays so
    return compute


def resolve_name(rules: Iterable[NameRule], external: str):
    """``(rule, internal name)``; internal None = known and dropped; rule None = unknown."""
    for rule in rules:
        m = rule.match_external(external)
        if m is not None:
            return rule, m[0]
    return None, None


def load_weights(
    folder,
    rules: List[NameRule],
    expected: Dict[str, ParamSpec],
    dtype: torch.dtype,
    device="cpu",
    ignore_when_present: Iterable[str] = (),
) -> Dict[str, torch.Tensor]:
    """Read every tensor of ``folder``, map its name through ``rules``, re-lay it out, check it
    against ``expected`` and move it to ``device`` in its final dtype.

    ``ignore_when_present``: internal names that may appear although the model has no such tensor
    (an output matrix beside tied embeddings); they are dropped with a warning.
    """
    from safetensors import safe_open

    ignore = set(ignore_when_present)
    out: Dict[str, torch.Tensor] = {}
    unexpected: List[str] = []
    wrong: List[Tuple[str, Tuple[int, ...], Tuple[int, ...]]] = []
    duplicates: List[str] = []
    for path in safetensors_files(folder):
        if not path.is_file():
            raise FileNotFoundError(f"{path} is named by the index but does not exist")
        with safe_open(str(path), framework="pt", device="cpu") as f:
            for ext_name in f.keys():
                rule, internal = resolve_name(rules, ext_name)
                if rule is None:
                    unexpected.append(ext_name)
                    continue
                if internal is None:
                    continue
                if internal not in expected:
                    if internal in ignore:
                        warnings.warn(f"{ext_name} in {path.name} is not used by this model and was ignored")
                    else:
                        unexpected.append(ext_name)
                    continue
                if internal in out:
                    duplicates.append(ext_name)
                    continue
                spec = expected[internal]
                t = f.get_tensor(ext_name)
                if tuple(t.shape) != tuple(spec.shape):
                    wrong.append((ext_name, tuple(t.shape), tuple(spec.shape)))
                    continue
                if rule.load is not None:
                    t = rule.load(t)
                t = t.to(dtype=_final_dtype(spec, t.dtype, dtype)).contiguous()
                out[internal] = t.to(device) if str(device) != "cpu" else t
    # report missing tensors under the names a checkpoint would use
    wrong_internal = set()
    for ext_name, _, _ in wrong:
        _, internal = resolve_name(rules, ext_name)
        wrong_internal.add(internal)
    missing = []
    for n in expected:
        if n in out or n in wrong_internal:
            continue
        ext = next((e for e in (r.match_internal(n) for r in rules) if e), n)
        missing.append(ext)
    if missing or unexpected or wrong or duplicates:
        raise WeightError(folder, missing, unexpected, wrong, duplicates)
    return out
