"""Puts a loaded model together with its cache: manager (metadata), store (device memory) and the
step function. Generation, the scheduler's engine and trace replay all go through this one path."""

from __future__ import annotations

from dataclasses import dataclass
from pathlib import Path
from typing import Optional

import torch

from ..cache.manager import CacheManager
from ..cache.store import CacheStore, bytes_per_page, group_specs, plan_groups
from ..parts.model import Model
from ..weights.loader import load_model
from .step import StepFunction


@dataclass
class EngineCore:
    model: Model
    manager: CacheManager
    store: CacheStore
    step: StepFunction

    @property
    def page_size(self) -> int:
        return self.manager.page_size


def pages_for_budget(model: Model, page_size: int, budget_bytes: int) -> int:
    """How many pages per group fit a byte budget (reference: src/dli/kv/paged_store.py:78-89)."""
    specs = model.cache_specs()
    groups, of_layer = plan_groups(specs)
    per = bytes_per_page(groups, [of_layer.count(g) for g in range(len(groups))], page_size, model.rt.dtype)
    if per == 0:
        return 1
    n = budget_bytes // per
    if n < 1:
        raise ValueError(f"a cache budget of {budget_bytes} bytes holds no page of {per} bytes")
    return int(n)


def build_core(model: Model | str | Path, *, num_pages: int, page_size: int = 16, max_seqs: int = 64,
               dtype: str | torch.dtype = "bfloat16", device: str = "cuda",
               enable_prefix_caching: bool = True, eviction_policy: str = "lru",
               watermark: float = 0.01, confine_to_thread: bool = True) -> EngineCore:
    """``confine_to_thread``: the cache manager refuses changes from any thread but the one that
    built the core (``core.manager.adopt()`` hands it to another)."""
    if not isinstance(model, Model):
        model = load_model(model, dtype=dtype, device=device)
    specs = model.cache_specs()
    store = CacheStore(model.rt, specs, num_pages=num_pages, page_size=page_size, max_seqs=max_seqs)
    manager = CacheManager(
        group_specs(store.groups), num_pages=num_pages, page_size=page_size, max_seqs=max_seqs,
        eviction_policy=eviction_policy, enable_prefix_caching=enable_prefix_caching,
        stateful=store.stateful, watermark=watermark, confine_to_thread=confine_to_thread)
    return EngineCore(model, manager, store, StepFunction(model, manager, store))
