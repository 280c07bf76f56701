"""Reads a model's tensors from safetensors files by tensor name.

The reference restores an Orbax tree and renames keys per checkpoint format
(simply/utils/checkpoint_lib.py:690-773); a shape mismatch is an error there
(:754-758), a missing tensor only a warning (:769-773), an unknown stored key is
ignored with a warning (:333).  Here missing tensors, unexpected tensors and wrong
shapes are all errors, reported together; one kind of extra tensor is allowed by
rule: a name that the model declares a copy of an expected tensor (the head of a
model with a tied head, stored once more as `lm_head.weight`) must equal that
tensor bit for bit and is then left unread.

Element types: floating tensors of role 'matrix' are held in the activation dtype
(wider parameters are cast down as simply/model_lib.py:2986-2998 does); 'vector'
tensors keep a 32-bit stored type; everything is float32 on the float32 path;
integer tensors are held as int32.
"""
from __future__ import annotations

import glob
import json
import os
from typing import Mapping

import torch

from ..parts.base import ParamSpec


class WeightsError(ValueError):
    """Lists every missing tensor, unexpected tensor and wrong shape at once."""

    def __init__(self, where: str, missing, unexpected, wrong_shape, other=()):
        self.missing, self.unexpected, self.wrong_shape = list(missing), list(unexpected), list(wrong_shape)
        lines = [f"{where}: the tensors do not match the model"]
        if self.missing:
            lines.append(f"  missing ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected ({len(self.unexpected)}): " + ", ".join(self.unexpected))
        if self.wrong_shape:
            lines.append(f"  wrong shape ({len(self.wrong_shape)}): " + "; ".join(
                f"{n}: file {list(got)}, model {list(want)}" for n, got, want in self.wrong_shape))
        lines.extend(f"  {o}" for o in other)
        super().__init__("\n".join(lines))


def weight_files(model_dir: str) -> list[str]:
    """model.safetensors, or the shards that model.safetensors.index.json names, or model*.safetensors
    (simply/tools/hf_to_orbax.py:67-85 globs the same pattern)."""
    single = os.path.join(model_dir, "model.safetensors")
    if os.path.isfile(single):
        return [single]
    index = os.path.join(model_dir, "model.safetensors.index.json")
    if os.path.isfile(index):
        with open(index) as f:
            names = sorted(set(json.load(f)["weight_map"].values()))
        return [os.path.join(model_dir, n) for n in names]
    files = sorted(glob.glob(os.path.join(model_dir, "model*.safetensors")))
    if not files:
        raise FileNotFoundError(f"{model_dir}: no model.safetensors (nor shards) in the model folder")
    return files


def target_dtype(stored: torch.dtype, spec: ParamSpec, activation_dtype: torch.dtype) -> torch.dtype:
    if not stored.is_floating_point or spec.role == "table":
        return torch.int32
    if activation_dtype == torch.float32:
        return torch.float32
    if spec.role == "vector" and stored == torch.float32:
        return torch.float32
    return activation_dtype


def check_names_and_shapes(where: str, expected: Mapping[str, ParamSpec], found: Mapping[str, tuple],
                           copies: Mapping[str, str] | None = None) -> None:
    """copies: stored name -> expected tensor that it must be a copy of; such a name is not unexpected, and its
    shape must be that tensor's."""
    copies = {n: of for n, of in (copies or {}).items() if of in expected and n not in expected}
    missing = [n for n in expected if n not in found]
    unexpected = [n for n in found if n not in expected and n not in copies]
    wrong = [(n, tuple(found[n]), tuple(expected[n].shape)) for n in expected
             if n in found and tuple(found[n]) != tuple(expected[n].shape)]
    wrong += [(n, tuple(found[n]), tuple(expected[of].shape)) for n, of in copies.items()
              if n in found and tuple(found[n]) != tuple(expected[of].shape)]
    if missing or unexpected or wrong:
        raise WeightsError(where, missing, unexpected, wrong)


def load_weights(model, model_dir: str, activation_dtype: torch.dtype, device) -> None:
    """Loads every tensor that `model.expected_tensors()` names into `model`."""
    from safetensors import safe_open

    expected = model.expected_tensors()
    files = weight_files(model_dir)
    where_of: dict[str, str] = {}
    shapes: dict[str, tuple] = {}
    duplicates = []
    handles = {}
    for path in files:
        h = safe_open(path, framework="pt", device="cpu")
        handles[path] = h
        for name in h.keys():
            if name in where_of:
                duplicates.append(name)
            where_of[name] = path
            shapes[name] = tuple(h.get_slice(name).get_shape())
    if duplicates:
        raise WeightsError(model_dir, [], [], [], [f"tensors stored in more than one file: {', '.join(duplicates)}"])
    copies = {n: of for n, of in getattr(model.spec, "copies", {}).items() if n in shapes and n not in expected}
    check_names_and_shapes(model_dir, expected, shapes, copies)
    differing = [f"{n} is stored beside {of}, of which the model makes it a copy, but the two differ"
                 for n, of in copies.items()
                 if not torch.equal(handles[where_of[n]].get_tensor(n), handles[where_of[of]].get_tensor(of))]
    if differing:
        raise WeightsError(model_dir, [], [], [], differing)
    tensors = {}
    for name, spec in expected.items():
        t = handles[where_of[name]].get_tensor(name)
        tensors[name] = t.to(device=device, dtype=target_dtype(t.dtype, spec, activation_dtype)).contiguous()
    model.load_tensors(tensors)
