"""From a model folder to a model with weights: the model class is chosen by config.json's
architecture name, as everywhere."""
from __future__ import annotations

import torch

from ..config import EngineConfig, load_config
from ..models import DecoderModel
from ..weights import init_random, load_weights


def load_model(model_dir: str, dtype: torch.dtype, device) -> tuple[DecoderModel, object]:
    """Returns (model with weights on `device`, typed configuration)."""
    config = load_config(model_dir)
    model = DecoderModel(config.model_spec())
    load_weights(model, model_dir, dtype, device)
    return model, config


def random_model(config, seed: int, dtype: torch.dtype, device, *, std: float | None = None,
                 norm_std: float = 0.1) -> DecoderModel:
    """A model of `config` with random weights drawn on the device, no files."""
    model = DecoderModel(config.model_spec())
    init_random(model, seed, dtype, device, std=std, norm_std=norm_std)
    return model
