"""Loads a model folder (``config.json`` + ``*.safetensors``) into a :class:`Model`.

Weights are bound by tensor name against the names and shapes that the model's parts declare, and
the check is strict: one :class:`CheckpointError` lists every missing tensor, every unexpected
tensor and every wrong shape (reference: src/dli/model/loader.py:67-91). Only safetensors files are
read; a folder that holds only pickle-based ``.bin``/``.pt`` weights is refused (:26-35).

Stored types: a ``matrix`` tensor takes the engine's activation type (bfloat16 when serving,
float32 on the 32-bit path); a tensor whose part asks for ``float32`` stays 32-bit (from bfloat16
storage it is widened exactly); integer tables become int32.
"""

from __future__ import annotations

from pathlib import Path
from typing import Any, Mapping, Optional

import numpy as np
import torch

from .. import architectures  # noqa: F401  (registers the built-in architectures)
from ..config.registry import read_config_json, resolve_architecture
from ..parts.base import Runtime
from ..parts.model import Model
from ..parts.spec import WeightSpec
from .safetensors_io import SafetensorsFile, SafetensorsFormatError, TensorEntry

_LIST_LIMIT = 12


class CheckpointError(ValueError):
    """The model folder cannot be used: format, missing or unexpected tensors, wrong shapes."""


def parse_dtype(name: str | torch.dtype) -> torch.dtype:
    if isinstance(name, torch.dtype):
        if name in (torch.float32, torch.bfloat16):
            return name
        raise ValueError(f"the engine computes in float32 or bfloat16, not {name}")
    table = {"float32": torch.float32, "fp32": torch.float32, "f32": torch.float32,
             "bfloat16": torch.bfloat16, "bf16": torch.bfloat16}
    if name not in table:
        raise ValueError(f"the engine computes in float32 or bfloat16, not {name!r}")
    return table[name]


def safetensor_files(model_dir: Path) -> list[Path]:
    files = sorted(model_dir.glob("*.safetensors"))
    if files:
        return files
    if any(model_dir.glob("*.bin")) or any(model_dir.glob("*.pt")) or any(model_dir.glob("*.pth")):
        raise CheckpointError(
            f"{model_dir} only has pickle-based weights (.bin/.pt); refusing to load them. "
            "Use a safetensors copy of the model.")
    raise CheckpointError(f"no *.safetensors files in {model_dir}")


def _to_torch(entry: TensorEntry) -> torch.Tensor:
    """Host tensor with the file's logical type (bfloat16 bits are re-viewed, not converted)."""
    bits = np.array(entry.bits)  # a private, writable copy of the mapped bytes
    if entry.tag == "BF16":
        return torch.from_numpy(bits.view(np.int16)).view(torch.bfloat16)
    if entry.tag == "BOOL":
        return torch.from_numpy(bits)
    return torch.from_numpy(bits)


def _place(entry: TensorEntry, spec: WeightSpec, rt: Runtime) -> torch.Tensor:
    host = _to_torch(entry)
    if spec.role == "int32":
        if not entry.is_integer:
            raise CheckpointError(f"{entry.name!r} is stored as {entry.tag} but must be an integer table")
        return host.to(device=rt.device, dtype=torch.int32)
    if not entry.is_float:
        raise CheckpointError(f"{entry.name!r} is stored as {entry.tag} but must be floating point")
    target = torch.float32 if spec.role == "float32" else rt.dtype
    dev = host.to(rt.device)
    return dev if dev.dtype == target else dev.to(target)


def _short(names: list[str]) -> str:
    if len(names) <= _LIST_LIMIT:
        return str(names)
    return f"{names[:_LIST_LIMIT]} and {len(names) - _LIST_LIMIT} more"


def build_model(config: Mapping[str, Any], rt: Runtime) -> tuple[Model, Any]:
    """The model (without weights) and typed configuration that a config.json dictionary names."""
    arch = resolve_architecture(config)
    cfg = arch.parse_config(config)
    return Model(arch.build_spec(cfg), rt), cfg


def load_model(model_dir: str | Path, *, dtype: str | torch.dtype = "bfloat16",
               device: str | torch.device = "cuda", decode_weight_copy: bool = True) -> Model:
    """Load ``model_dir`` (``config.json`` chooses the model class through the registry).
    ``decode_weight_copy`` (bfloat16 only): keep each matrix a second time in the order in which
    the decode kernels read it: faster decode steps, twice the weight memory.

    Raises:
        CheckpointError: unusable folder; the message lists missing, unexpected and misshapen tensors.
        UnsupportedModelError / ConfigError: the configuration asks for what is not implemented.
    """
    model_dir = Path(model_dir)
    rt = Runtime(torch.device(device), parse_dtype(dtype), decode_weight_copy=decode_weight_copy)
    raw = read_config_json(model_dir)
    model, cfg = build_model(raw, rt)
    model.config = cfg
    expected = model.weight_specs()

    files: list[SafetensorsFile] = []
    try:
        where: dict[str, SafetensorsFile] = {}
        for path in safetensor_files(model_dir):
            try:
                f = SafetensorsFile(path)
            except SafetensorsFormatError as exc:
                raise CheckpointError(str(exc)) from exc
            files.append(f)
            for name in f.names():
                where[name] = f

        problems: list[str] = []
        # a tied model whose file still carries the alias: accept only an exact copy, then drop it
        for alias, canonical in model.spec.tied_aliases.items():
            if alias in where and alias not in expected:
                if canonical in where:
                    a, c = where[alias].get(alias), where[canonical].get(canonical)
                    same = a.tag == c.tag and a.shape == c.shape and np.array_equal(a.bits, c.bits)
                    if not same:
                        raise CheckpointError(
                            f"tie_word_embeddings=true but {alias} differs from {canonical}")
                del where[alias]

        missing = sorted(n for n, s in expected.items() if n not in where and not s.optional)
        unexpected = sorted(n for n in where if n not in expected)
        bad_shape = sorted(
            f"{n}: file {list(where[n].shape_of(n))}, model {list(s.shape)}"
            for n, s in expected.items() if n in where and where[n].shape_of(n) != tuple(s.shape))
        if missing:
            problems.append(f"missing tensors: {_short(missing)}")
        if unexpected:
            problems.append(f"unexpected tensors: {_short(unexpected)}")
        if bad_shape:
            problems.append(f"shape mismatch: {_short(bad_shape)}")
        if problems:
            raise CheckpointError(f"{model_dir}: " + "; ".join(problems))

        tensors = {n: _place(where[n].get(n), s, rt) for n, s in expected.items() if n in where}
    finally:
        for f in files:
            f.close()
    model.load_weights(tensors)
    return model
