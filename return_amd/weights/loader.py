"""Weights from safetensors by tensor name.

The reference loads through HF from_pretrained in bf16 (rollout/engine_actor.py:14-21)
and has no checks of its own. Here the expected names and shapes come from the
model's spec; a folder that does not fit is refused with ONE error that lists
missing tensors, unexpected tensors and wrong shapes together. Stored dtypes are
kept: bfloat16 stays bfloat16, a tensor stored in 32-bit stays 32-bit, integer
tables become int32. What a kernel needs in another precision the part converts
when it is built.
"""
from __future__ import annotations

import json
import os
from typing import Dict, List

import torch
from safetensors import safe_open

from ..parts.spec import ModelSpec


class WeightError(ValueError):
    """The checkpoint does not fit the model: lists missing, unexpected and misshaped tensors."""

    def __init__(self, folder, missing, unexpected, misshaped, other=()):
        self.missing, self.unexpected, self.misshaped = list(missing), list(unexpected), list(misshaped)
        lines = [f"weights in {folder} do not fit the model:"]
        if self.missing:
            lines.append(f"  missing ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        if self.misshaped:
            lines.append(f"  wrong shape ({len(self.misshaped)}): " + "; ".join(
                f"{n} is {tuple(got)}, model wants {tuple(want)}" for n, got, want in self.misshaped))
        lines.extend(f"  {o}" for o in other)
        super().__init__("\n".join(lines))


def _shard_files(folder: str) -> List[str]:
    index = os.path.join(folder, "model.safetensors.index.json")
    single = os.path.join(folder, "model.safetensors")
    if os.path.exists(index):
        with open(index) as f:
            files = sorted(set(json.load(f)["weight_map"].values()))
        return [os.path.join(folder, name) for name in files]
    if os.path.exists(single):
        return [single]
    raise FileNotFoundError(f"{folder}: neither model.safetensors nor model.safetensors.index.json")


_KEEP = (torch.bfloat16, torch.float32)


def _stored(t: torch.Tensor) -> torch.Tensor:
    if t.dtype in _KEEP:
        return t
    if t.dtype in (torch.int8, torch.int16, torch.int32, torch.int64, torch.uint8, torch.bool):
        return t.to(torch.int32)
    if t.dtype in (torch.float16, torch.float64):
        return t.to(torch.float32)          # fp16 values do not all fit bfloat16
    raise TypeError(f"tensor dtype {t.dtype} is not supported")


def load_weights(folder: str, spec: ModelSpec, device="cpu") -> Dict[str, torch.Tensor]:
    """Every tensor the spec names, by name, on ``device``; WeightError if the folder does not fit."""
    expected = spec.expected_tensors()
    ignorable = set(spec.ignorable)
    files = _shard_files(folder)
    found: Dict[str, str] = {}
    shapes: Dict[str, tuple] = {}
    for path in files:
        with safe_open(path, framework="pt", device="cpu") as f:
            for name in f.keys():
                found[name] = path
                shapes[name] = tuple(f.get_slice(name).get_shape())
    missing = sorted(n for n in expected if n not in found)
    unexpected = sorted(n for n in found if n not in expected and n not in ignorable)
    misshaped = sorted((n, shapes[n], expected[n][0]) for n in expected
                       if n in found and shapes[n] != tuple(expected[n][0]))
    if missing or unexpected or misshaped:
        raise WeightError(folder, missing, unexpected, misshaped)
    out: Dict[str, torch.Tensor] = {}
    by_file: Dict[str, List[str]] = {}
    for name in expected:
        by_file.setdefault(found[name], []).append(name)
    for path, names in by_file.items():
        with safe_open(path, framework="pt", device="cpu") as f:
            for name in names:
                out[name] = _stored(f.get_tensor(name)).to(device)
    return out
