"""Random-weights mode: writes a model folder from a configuration and a seed.

The folder holds ``config.json`` and ``model.safetensors`` and loads like any other. Every tensor
is drawn from its own generator keyed by (seed, tensor name), so a tensor's values do not depend on
which other tensors the model has: matrices and biases ``N(0, std)``, norm weights ``1`` (or
``1 + norm_jitter * N(0, 1)`` so that a norm in the wrong place changes the result). Values are
stored in bfloat16 by default; what the 32-bit path then loads is exactly what serving loads.
"""

from __future__ import annotations

import json
import zlib
from pathlib import Path
from typing import Any, Mapping

import numpy as np
import torch

from .. import architectures  # noqa: F401
from ..config.registry import resolve_architecture
from ..parts.base import Runtime
from ..parts.model import Model
from .safetensors_io import float32_to_bfloat16_bits, write_safetensors

_CHUNK = 1 << 24


def _generator(seed: int, name: str) -> np.random.Generator:
    return np.random.default_rng([int(seed) & 0xFFFFFFFFFFFFFFFF, zlib.crc32(name.encode("utf-8"))])


def random_tensor(name: str, shape: tuple[int, ...], init: str, seed: int, std: float,
                  norm_jitter: float) -> np.ndarray:
    rng = _generator(seed, name)
    if init == "zeros":
        return np.zeros(shape, np.float32)
    if init == "ones":
        return np.ones(shape, np.float32)
    if init == "norm":
        out = np.ones(shape, np.float32)
        if norm_jitter:
            out += np.float32(norm_jitter) * rng.standard_normal(shape, dtype=np.float32)
        return out
    out = np.empty(int(np.prod(shape)), np.float32)
    for lo in range(0, out.size, _CHUNK):  # bounded temporary memory for large tables
        hi = min(out.size, lo + _CHUNK)
        out[lo:hi] = rng.standard_normal(hi - lo, dtype=np.float32)
    out *= np.float32(std)
    return out.reshape(shape)


def _drawn_on_device(name: str, shape: tuple[int, ...], init: str, seed: int, std: float, norm_jitter: float,
                     device: torch.device) -> torch.Tensor:
    """The same distributions as :func:`random_tensor`, drawn by the device's generator (other
    values for the same seed): float32 on ``device``."""
    gen = torch.Generator(device=device)
    gen.manual_seed((int(seed) * 1000003 + zlib.crc32(name.encode("utf-8"))) & 0x7FFFFFFFFFFFFFFF)
    if init == "zeros":
        return torch.zeros(shape, dtype=torch.float32, device=device)
    if init in ("ones", "norm"):
        out = torch.ones(shape, dtype=torch.float32, device=device)
        if init == "norm" and norm_jitter:
            out += norm_jitter * torch.empty(shape, dtype=torch.float32, device=device).normal_(generator=gen)
        return out
    return torch.empty(shape, dtype=torch.float32, device=device).normal_(0.0, std, generator=gen)


def write_random_model(out_dir: str | Path, config: Mapping[str, Any] | Any, *, seed: int = 0,
                       std: float = 0.02, norm_jitter: float = 0.0,
                       storage: str = "bfloat16", device: str | torch.device = "cpu") -> Path:
    """Write ``config.json`` and ``model.safetensors`` for ``config`` (a config.json dictionary,
    or a typed configuration with ``to_hf_dict``) with weights drawn from ``seed``. With a GPU as
    ``device`` the values are drawn there (seconds instead of minutes for a billion weights; the
    values are that generator's, not the host generator's)."""
    raw = dict(config.to_hf_dict()) if hasattr(config, "to_hf_dict") else dict(config)
    if storage not in ("bfloat16", "float32"):
        raise ValueError("storage must be 'bfloat16' or 'float32'")
    arch = resolve_architecture(raw)
    cfg = arch.parse_config(raw)
    model = Model(arch.build_spec(cfg), Runtime(torch.device("cpu"), torch.float32))
    tensors: dict[str, tuple[str, np.ndarray]] = {}
    for name, spec in model.weight_specs().items():
        if spec.role == "int32":
            tensors[name] = ("I32", np.zeros(spec.shape, np.int32))
            continue
        if torch.device(device).type != "cpu":
            t = _drawn_on_device(name, tuple(spec.shape), spec.init, seed, std, norm_jitter, torch.device(device))
            if storage == "bfloat16":
                tensors[name] = ("BF16", t.to(torch.bfloat16).view(torch.int16).cpu().numpy().view(np.uint16))
            else:
                tensors[name] = ("F32", t.cpu().numpy())
            continue
        values = random_tensor(name, tuple(spec.shape), spec.init, seed, std, norm_jitter)
        if storage == "bfloat16":
            tensors[name] = ("BF16", float32_to_bfloat16_bits(values).reshape(spec.shape))
        else:
            tensors[name] = ("F32", values)
    out = Path(out_dir)
    out.mkdir(parents=True, exist_ok=True)
    (out / "config.json").write_text(json.dumps(raw, indent=2) + "\n")
    write_safetensors(out / "model.safetensors", tensors, metadata={"format": "pt"})
    return out
