"""Random weights from a configuration and a seed.

The reference draws parameters module by module from split keys (simply/model_lib.py:2854-2872,
Xavier-uniform linears simply/utils/initializer.py:92-125, norm scales zero model_lib.py:142-146).
Here every matrix is N(0, initializer_range) and every norm scale N(0, norm_std), drawn in float32
in the order of `model.expected_tensors()` from one generator, then cast: non-zero norm scales make
a `(1 + w)` gain differ from a `w` gain.
"""
from __future__ import annotations

import json
import os

import torch

from ..parts.base import ParamSpec


def _draw(spec: ParamSpec, gen: torch.Generator, std: float, norm_std: float, device) -> torch.Tensor:
    if spec.init == "zeros":
        return torch.zeros(spec.shape, dtype=torch.float32, device=device)
    s = norm_std if spec.init == "norm" else std
    return torch.randn(spec.shape, generator=gen, dtype=torch.float32, device=device) * s


def random_tensors(model, seed: int, dtype: torch.dtype, *, std: float | None = None, norm_std: float = 0.1,
                   device="cpu"):
    """Yields (name, tensor) for every tensor of the model."""
    gen = torch.Generator(device=device)
    gen.manual_seed(int(seed))
    std = model.spec.initializer_range if std is None else std
    for name, spec in model.expected_tensors().items():
        t = _draw(spec, gen, std, norm_std, device)
        yield name, (t.to(torch.int32) if spec.role == "table" else t.to(dtype))


def init_random(model, seed: int, activation_dtype: torch.dtype, device, *, std: float | None = None,
                norm_std: float = 0.1) -> None:
    """Fills `model` with random weights drawn on `device` (no files)."""
    model.load_tensors(dict(random_tensors(model, seed, activation_dtype, std=std, norm_std=norm_std, device=device)))


def write_random_model(config, out_dir: str, seed: int, dtype: torch.dtype = torch.bfloat16, *,
                       std: float | None = None, norm_std: float = 0.1) -> str:
    """Writes `config.json` and `model.safetensors` for `config` (a typed architecture config)."""
    from safetensors.torch import save_file

    from ..models import DecoderModel

    model = DecoderModel(config.model_spec())
    os.makedirs(out_dir, exist_ok=True)
    tensors = {n: t.contiguous() for n, t in random_tensors(model, seed, dtype, std=std, norm_std=norm_std)}
    save_file(tensors, os.path.join(out_dir, "model.safetensors"), metadata={"format": "pt"})
    d = config.to_dict()
    d["torch_dtype"] = str(dtype).replace("torch.", "")
    with open(os.path.join(out_dir, "config.json"), "w") as f:
        json.dump(d, f, indent=2)
    return out_dir
