"""Loading a model's tensors from ``model.safetensors`` by name.

kappai looks tensors up by name and validates every shape against the dimensions the
metadata gave (src/model.c:113-128, validate_model_dims :278-586), naming the tensor
that is missing or wrong.  Here all problems of a file are collected and raised as ONE
error that lists missing tensors, unexpected tensors and wrong shapes.
"""
from __future__ import annotations

import json
from pathlib import Path
from typing import Dict, Iterable, List

import torch

from .safetensors_io import SafetensorsError, SafetensorsFile
from .spec import TensorSpec

COMPUTE_DTYPES = {"bfloat16": torch.bfloat16, "float32": torch.float32}


class WeightsError(ValueError):
    """Raised once per load with everything that is wrong with the file."""

    def __init__(self, path, missing: List[str], unexpected: List[str], wrong: List[str],
                 other: List[str] = ()):
        self.missing, self.unexpected, self.wrong_shape, self.other = (
            list(missing), list(unexpected), list(wrong), list(other))
        lines = [f"{path}: weights do not match the model built from config.json"]
        if self.missing:
            lines.append(f"  missing tensors ({len(self.missing)}): " + ", ".join(self.missing))
        if self.unexpected:
            lines.append(f"  unexpected tensors ({len(self.unexpected)}): "
                         + ", ".join(self.unexpected))
        if self.wrong_shape:
            lines.append(f"  wrong shapes ({len(self.wrong_shape)}): " + "; ".join(self.wrong_shape))
        if self.other:
            lines.append("  " + "; ".join(self.other))
        super().__init__("\n".join(lines))


def parse_dtype(name: str) -> torch.dtype:
    key = {"bf16": "bfloat16", "fp32": "float32"}.get(name, name)
    if key not in COMPUTE_DTYPES:
        raise ValueError(f"dtype must be one of {', '.join(COMPUTE_DTYPES)}; got {name!r}")
    return COMPUTE_DTYPES[key]


def stored_to_runtime(t: torch.Tensor, compute_dtype: torch.dtype) -> torch.Tensor:
    """Dtype rule of the engine: in a bfloat16 run 16-bit floats are kept as bfloat16 and
    a tensor stored in 32 bits stays so; integer tables become int32; in a float32 run
    every float is widened (exactly) to float32."""
    if t.dtype in (torch.int32, torch.int64):
        return t.to(torch.int32)
    if compute_dtype == torch.float32:
        return t.to(torch.float32)
    if t.dtype == torch.float32:
        return t
    return t.to(torch.bfloat16)


def _weight_files(model_dir: Path) -> List[Path]:
    single = model_dir / "model.safetensors"
    if single.is_file():
        return [single]
    index = model_dir / "model.safetensors.index.json"
    if index.is_file():
        names = sorted(set(json.loads(index.read_text())["weight_map"].values()))
        for n in names:        # a model folder is untrusted input: its files lie inside it
            if (not isinstance(n, str) or not n or n in (".", "..") or "/" in n or "\\" in n
                    or Path(n).is_absolute()):
                raise WeightsError(model_dir, [], [], [], [
                    f"{index.name}: weight_map names the file {n!r}; a plain file name inside "
                    "the model folder is needed"])
        return [model_dir / n for n in names]
    raise WeightsError(model_dir, [], [], [], [f"no model.safetensors in {model_dir}"])


def check_and_load(model_dir, specs: Iterable[TensorSpec], compute_dtype: torch.dtype,
                   device) -> Dict[str, torch.Tensor]:
    """Check the file(s) against ``specs`` and return ``{name: tensor on device}``."""
    model_dir = Path(model_dir)
    specs = {s.name: s for s in specs}
    files = []
    try:
        for p in _weight_files(model_dir):
            files.append(SafetensorsFile(p))
    except SafetensorsError as exc:
        raise WeightsError(model_dir, [], [], [], [str(exc)]) from exc
    try:
        where = {}
        for f in files:
            for n in f.names():
                where[n] = f
        missing = sorted(n for n in specs if n not in where)
        unexpected = sorted(n for n in where if n not in specs)
        wrong = []
        for n, s in specs.items():
            if n in where:
                e = where[n].entries[n]
                if tuple(e.shape) != tuple(s.shape):
                    wrong.append(f"{n}: file has {list(e.shape)}, model needs {list(s.shape)}")
                elif e.dtype not in ("BF16", "F16", "F32"):
                    wrong.append(f"{n}: file has dtype {e.dtype}, a float tensor is needed")
        if missing or unexpected or wrong:
            raise WeightsError(files[0].path if len(files) == 1 else model_dir,
                               missing, unexpected, wrong)
        out = {}
        for n in specs:
            out[n] = stored_to_runtime(where[n].read(n), compute_dtype).to(device)
        return out
    finally:
        for f in files:
            f.close()
