"""Random weights for a configuration and a seed, and the model folder they are written to.

The reference only has this in tests: AutoModelForCausalLM.from_config under
torch.manual_seed (opd/test_qwen.py:13-23). Here tensors are drawn in sorted name
order from one CPU generator, so that a seed always gives the same model:
matrices N(0, std), embedding tables N(0, embedding_std), norm weights
1 + N(0, norm_jitter). A part whose tensor needs another law (a decay that must stay
inside (0, 1), a parameter kept as a logarithm, a bias that starts at zero) gives it
itself: its random_init(params, role) returns a callable (shape, generator) -> tensor
in place of one of the three names.
"""
from __future__ import annotations

import os
from typing import Dict, Optional

import torch
from safetensors.torch import save_file

from ..config.base import ModelConfig, lookup_architecture

_DTYPES = {"bfloat16": torch.bfloat16, "float32": torch.float32}


def random_weights(spec, seed: int = 0, std: float = 0.02, embedding_std: Optional[float] = None,
                   norm_jitter: float = 0.01, dtype: str = "bfloat16", device="cpu",
                   generator_device="cpu") -> Dict[str, torch.Tensor]:
    """name -> tensor for every tensor the spec expects.

    generator_device "cpu" gives values that depend only on the seed; another device
    draws there (fast for large models, values differ from the CPU's).
    """
    embedding_std = std if embedding_std is None else embedding_std
    gen = torch.Generator(device=generator_device)
    gen.manual_seed(int(seed))
    out = {}
    expected = spec.expected_tensors()
    for name in sorted(expected):
        shape, draw = expected[name]
        if callable(draw):
            # the part's own law, drawn from the same generator (so the seed still fixes the model)
            x = draw(tuple(shape), gen)
            if not isinstance(x, torch.Tensor) or tuple(x.shape) != tuple(shape):
                raise ValueError(f"{name}: the part's own draw gave {getattr(x, 'shape', type(x))}, wanted {tuple(shape)}")
            # integer tables and tensors that the part wants in 32-bit whatever the model's precision stay as drawn
            out[name] = (x.to(_DTYPES[dtype]) if x.dtype in (torch.float32, torch.float64) and
                         not getattr(draw, "keep_dtype", False) else x).to(device)
            continue
        if draw not in ("matrix", "embedding", "norm"):
            raise ValueError(f"{name}: random_init gave {draw!r}; one of 'matrix', 'embedding', 'norm' or a callable")
        x = torch.randn(*shape, generator=gen, dtype=torch.float32, device=generator_device)
        if draw == "norm":
            x = 1.0 + norm_jitter * x
        elif draw == "embedding":
            x = embedding_std * x
        else:
            x = std * x
        out[name] = x.to(_DTYPES[dtype]).to(device)
    return out


def write_model_folder(folder: str, config: ModelConfig, seed: int = 0, std: float = 0.02,
                       embedding_std: Optional[float] = None, norm_jitter: float = 0.01,
                       dtype: str = "bfloat16") -> str:
    """config.json and model.safetensors of a random model; returns the folder."""
    _, build_spec = lookup_architecture(config.architecture)
    spec = build_spec(config)
    weights = random_weights(spec, seed, std, embedding_std, norm_jitter, dtype)
    os.makedirs(folder, exist_ok=True)
    config.save(folder)
    save_file({k: v.contiguous() for k, v in weights.items()},
              os.path.join(folder, "model.safetensors"), metadata={"format": "pt"})
    return folder
