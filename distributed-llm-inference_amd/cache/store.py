"""Device memory of the cache: page pools per group and state arrays per stateful layer.

Layers are grouped by what their mixers declare (:class:`PagedKVSpec`): equal specs share one
group, one block table per request and one pool tensor
``[layers of the group, 2 (keys, values), pages, kv_heads * page_size * head_dim]``
(where a value's size differs from a key's: one tensor ``[layers, 1, pages, ...]`` for the keys
and one for the values, or none if the mixer keeps no values).
Inside a page, keys lie as ``[kv_heads][page_size][head_dim]`` and values as
``[kv_heads][value_dim][page_size]`` (the order in which the attention kernels consume them).
A mixer that declares a :class:`StateSpec` gets an array ``[state slots + 1, *shape]`` instead: one
row per slot that a request can hold, and a last row (``scratch_slot``) that no request holds, for
the padding rows of a replayed graph to write to.
Everything is allocated once and zero-filled (reference: src/dli/kv/paged_store.py:50-52).
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Sequence

import torch

from ..parts.base import PagedKVSpec, Runtime, StateSpec
from .manager import CopyOp, GroupSpec


@dataclass
class LayerCache:
    """What one schedule entry's mixer gets: its pages (with the group whose block tables index
    them) or its state array. ``writable`` is False for an entry that reads another's cache."""

    kind: str  # "paged" or "state"
    group: int = -1
    k_pages: Optional[torch.Tensor] = None  # [pages, kv_heads, page_size, head_dim]
    v_pages: Optional[torch.Tensor] = None  # [pages, kv_heads, value_dim, page_size]; None: keys only
    state: Optional[torch.Tensor] = None    # [slots, *shape]
    writable: bool = True
    window: int = 0

    def reader(self) -> "LayerCache":
        return LayerCache(self.kind, self.group, self.k_pages, self.v_pages, self.state, False, self.window)


def plan_groups(specs: Sequence[Optional[PagedKVSpec | StateSpec]]) -> tuple[list[PagedKVSpec], list[int]]:
    """Distinct paged specs in order of first appearance, and each layer's group (-1: none)."""
    groups: list[PagedKVSpec] = []
    of_layer: list[int] = []
    for s in specs:
        if isinstance(s, PagedKVSpec):
            if s not in groups:
                groups.append(s)
            of_layer.append(groups.index(s))
        else:
            of_layer.append(-1)
    return groups, of_layer


def group_specs(groups: Sequence[PagedKVSpec]) -> list[GroupSpec]:
    return [GroupSpec("window", g.window) if g.window > 0 else GroupSpec() for g in groups] or [GroupSpec()]


def bytes_per_page(groups: Sequence[PagedKVSpec], layers_per_group: Sequence[int], page_size: int,
                   dtype: torch.dtype) -> int:
    """Bytes that one page id costs across all groups and layers, keys and values."""
    item = torch.empty((), dtype=dtype).element_size()
    return sum(n * page_size * g.kv_heads * (g.head_dim + g.v_dim) * item for g, n in zip(groups, layers_per_group))


class CacheStore:
    def __init__(self, rt: Runtime, specs: Sequence[Optional[PagedKVSpec | StateSpec]], *,
                 num_pages: int, page_size: int, max_seqs: int) -> None:
        self.rt = rt
        self.page_size = page_size
        self.num_pages = num_pages
        self.scratch_slot = max_seqs
        self.groups, self._group_of = plan_groups(specs)
        self.layers_per_group = [self._group_of.count(g) for g in range(len(self.groups))]
        # per group: the tensors [layers, 1 or 2, pages, elements] that hold its pages
        self.pools: list[list[torch.Tensor]] = []
        for g, n_layers in zip(self.groups, self.layers_per_group):
            sizes = [g.kv_heads * page_size * g.head_dim, g.kv_heads * page_size * g.v_dim]
            if sizes[0] == sizes[1]:
                shapes = [(n_layers, 2, num_pages, sizes[0])]
            else:
                shapes = [(n_layers, 1, num_pages, n) for n in sizes if n > 0]
            self.pools.append([torch.zeros(shape, device=rt.device, dtype=rt.dtype) for shape in shapes])
        self.layers: list[Optional[LayerCache]] = []
        seen = [0] * len(self.groups)
        for spec, g in zip(specs, self._group_of):
            if isinstance(spec, PagedKVSpec):
                i = seen[g]
                seen[g] += 1
                pools = self.pools[g]
                keys = pools[0][i, 0]
                values = pools[0][i, 1] if pools[0].shape[1] == 2 else (pools[1][i, 0] if len(pools) > 1 else None)
                self.layers.append(LayerCache(
                    "paged", g,
                    keys.view(num_pages, spec.kv_heads, page_size, spec.head_dim),
                    None if values is None else values.view(num_pages, spec.kv_heads, spec.v_dim, page_size),
                    window=spec.window))
            elif isinstance(spec, StateSpec):
                self.layers.append(LayerCache(
                    "state", state=torch.zeros(max_seqs + 1, *spec.shape, device=rt.device, dtype=spec.dtype)))
            else:
                self.layers.append(None)

    @property
    def stateful(self) -> bool:
        return any(c is not None and c.kind == "state" for c in self.layers)

    def bytes_per_page(self) -> int:
        return bytes_per_page(self.groups, self.layers_per_group, self.page_size, self.rt.dtype)

    def copy_pages(self, ops_list: Sequence[CopyOp]) -> None:
        """Do the copy-on-write copies of a step, every layer of each group at once
        (reference: src/dli/kv/paged_store.py:110-118)."""
        if not ops_list:
            return
        from ..kernels import ops

        for g, pools in enumerate(self.pools):
            mine = [o for o in ops_list if o.group == g]
            if not mine:
                continue
            for o in mine:
                if not (0 <= o.src < self.num_pages and 0 <= o.dst < self.num_pages):
                    raise ValueError(f"page copy {o} names a page outside the pool")
            src = torch.tensor([o.src for o in mine], dtype=torch.int32, device=self.rt.device)
            dst = torch.tensor([o.dst for o in mine], dtype=torch.int32, device=self.rt.device)
            for pool in pools:
                ops.copy_pages(pool, src, dst)
