"""Models by architecture name."""
from __future__ import annotations

from pathlib import Path

import torch

from ..config.base import ModelConfig, load_config, lookup_architecture
from ..weights.loader import check_and_load, parse_dtype
from . import lfm2  # noqa: F401  (registers Lfm2ForCausalLM)
from .base import LayerCall, Model


def build_model(config: ModelConfig, dtype) -> Model:
    """The model of ``config``'s architecture, without weights."""
    dtype = parse_dtype(dtype) if isinstance(dtype, str) else dtype
    return lookup_architecture(config.architecture).build_model(config, dtype)


def load_model(model_dir, dtype, device="cuda:0") -> Model:
    """Read ``config.json``, build the model its ``architectures`` entry names, check
    ``model.safetensors`` against it and bind the tensors on ``device``."""
    dtype = parse_dtype(dtype) if isinstance(dtype, str) else dtype
    config = load_config(model_dir)
    model = build_model(config, dtype)
    tensors = check_and_load(Path(model_dir), model.tensor_specs(), dtype, device)
    model.bind(tensors)
    return model


__all__ = ["LayerCall", "Model", "build_model", "load_model"]
