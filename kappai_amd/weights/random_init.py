"""Random-weights mode: make a model folder (config.json, model.safetensors) from a
configuration and a seed.  kappai has this only in its tests (an xorshift generator with
uniform matrices and norm weights 1 +- 0.15, src/test/test_synth_gguf.c:50-68); here it is
a mode of the framework so that every size can be run without a checkpoint.
"""
from __future__ import annotations

import hashlib
import json
from pathlib import Path
from typing import Dict, Iterable

import numpy as np
import torch

from .safetensors_io import write_safetensors
from .spec import INIT_NORMAL, INIT_ONES, INIT_SMALL, TensorSpec


def _generator(seed: int, name: str) -> np.random.Generator:
    digest = hashlib.sha256(name.encode()).digest()
    return np.random.default_rng([int(seed) & 0xFFFFFFFF, int.from_bytes(digest[:8], "little")])


def random_tensor(spec: TensorSpec, seed: int, std: float, norm_jitter: float,
                  vector_dtype=torch.bfloat16) -> torch.Tensor:
    """A tensor that depends only on (seed, tensor name, shape): every tensor has its own
    stream, so models that share a tensor name and shape share its values."""
    rng = _generator(seed, spec.name)
    if spec.init == INIT_ONES:
        a = np.ones(spec.shape, dtype=np.float32)
        if norm_jitter:
            a += rng.standard_normal(spec.shape, dtype=np.float32) * np.float32(norm_jitter)
    elif spec.init in (INIT_NORMAL, INIT_SMALL):
        a = rng.standard_normal(spec.shape, dtype=np.float32) * np.float32(std)
    else:
        raise ValueError(f"unknown init {spec.init!r} for {spec.name}")
    t = torch.from_numpy(a)
    dt = torch.bfloat16 if spec.role != "vector" else vector_dtype
    return t.to(dt)


def random_tensors(specs: Iterable[TensorSpec], seed: int, std: float = 0.02,
                   norm_jitter: float = 0.0, vector_dtype=torch.bfloat16) -> Dict[str, torch.Tensor]:
    return {s.name: random_tensor(s, seed, std, norm_jitter, vector_dtype) for s in specs}


def write_random_model(model_dir, config, seed: int, std: float = 0.02, norm_jitter: float = 0.0,
                       vector_dtype=torch.bfloat16) -> Path:
    """Write ``config.json`` and ``model.safetensors`` for ``config`` (a typed
    configuration of a registered architecture).  Matrices and tables are stored as
    bfloat16, so a float32 run and a bfloat16 run read exactly the same numbers."""
    from ..models import build_model  # late: models import parts which import weights.spec

    model_dir = Path(model_dir)
    model_dir.mkdir(parents=True, exist_ok=True)
    model = build_model(config, torch.float32)
    tensors = random_tensors(model.tensor_specs(), seed, std, norm_jitter, vector_dtype)
    (model_dir / "config.json").write_text(json.dumps(config.to_dict(), indent=2) + "\n")
    write_safetensors(model_dir / "model.safetensors", tensors,
                      metadata={"format": "pt", "seed": seed, "std": std})
    return model_dir
