"""One step's batch, as the step function gives it to the model.

A step runs the next tokens of several requests at once: portions of prompts beside single decoded
tokens, cut anywhere. :class:`StepEntry` is one request's share; :class:`StepContext` is the
device-side description of the whole batch that every part reads. The rows of all entries are laid
end to end: entries that bring exactly one token come first (they take the decode kernels), then the
portions, each group in the order given.

Reference: the runner's flattening of scheduled chunks (src/dli/engine/runner.py:53-183) and the
metadata carriers of src/dli/model/kv_cache.py:94-210.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Callable, Hashable, Optional, Sequence

import numpy as np
import torch


def upload(arrays: Sequence[np.ndarray], device: torch.device) -> list[torch.Tensor]:
    """The host arrays as device tensors of the same shapes and types, all views of one buffer
    that one asynchronous copy from pinned memory fills; each starts on a 16-byte boundary. A
    copy from pageable memory would make the host wait for the work already queued on the GPU,
    which then idles while the host catches up with its launches."""
    starts, at = [], 0
    for a in arrays:
        starts.append(at)
        at += -(-a.nbytes // 16) * 16
    host = torch.empty(max(at, 16), dtype=torch.uint8, pin_memory=True)
    flat = host.numpy()
    for a, s0 in zip(arrays, starts):
        flat[s0:s0 + a.nbytes] = np.ascontiguousarray(a).reshape(-1).view(np.uint8)
    buf = host.to(device, non_blocking=True)
    return [buf[s0:s0 + a.nbytes].view(torch.from_numpy(np.empty(0, a.dtype)).dtype).view(a.shape)
            for a, s0 in zip(arrays, starts)]


@dataclass
class StepEntry:
    """``tokens`` continue request ``seq_id`` at absolute position ``start``; ``want`` lists the
    offsets among these tokens whose logits are asked for (possibly none)."""

    seq_id: Hashable
    tokens: Sequence[int]
    start: int
    want: Sequence[int] = ()


@dataclass
class HostBatch:
    """A checked step laid out on the host: single-token entries first, then portions (``order``
    maps the layout's entries to the caller's). What the device-side context is made from, by an
    upload or by a copy into a captured graph's arrays."""

    order: list                   # layout entry -> index in the caller's list
    seq_ids: list
    num_decode: int
    token_ids: np.ndarray         # int64 [tokens]
    positions: np.ndarray         # int32 [tokens]
    q_start: np.ndarray           # int32 [entries + 1]
    kv_len: np.ndarray            # int32 [entries]
    state_slots: np.ndarray       # int32 [entries]
    logit_rows: np.ndarray        # int32 [k], in the caller's order of entries and wants
    slots: list                   # per group: int64 [tokens]
    tables: list                  # per group: int64 [entries, widest table], a row of pages per entry, padded with zeros

    @property
    def num_tokens(self) -> int:
        return int(self.q_start[-1])

    @property
    def num_entries(self) -> int:
        return len(self.order)


@dataclass
class GroupView:
    """Addresses of one cache group for this step."""

    slots: torch.Tensor          # int32 [tokens]: page * page_size + offset where each token's k,v go
    block_tables: torch.Tensor   # int32 [entries, width]: pages of each request, in position order
    table_width: int


@dataclass
class StepContext:
    device: torch.device
    page_size: int
    num_tokens: int
    num_entries: int
    num_decode: int               # leading entries that bring exactly one token
    token_ids: torch.Tensor       # int32 [tokens]
    positions: torch.Tensor       # int32 [tokens], absolute
    q_start: torch.Tensor         # int32 [entries + 1]: first row of each entry
    kv_len: torch.Tensor          # int32 [entries]: keys of the request after this step
    state_slots: torch.Tensor     # int32 [entries]
    logit_rows: torch.Tensor      # int32 [k]: rows whose logits are wanted, in the caller's order
    groups: list[GroupView]
    # host copies (parts may need them to choose kernels and grids)
    q_start_host: np.ndarray = field(default_factory=lambda: np.zeros(1, np.int32))
    kv_len_host: np.ndarray = field(default_factory=lambda: np.zeros(0, np.int32))
    state_slots_host: np.ndarray = field(default_factory=lambda: np.zeros(0, np.int32))
    seq_ids: list = field(default_factory=list)
    # per mixer (``id(mixer)``), what it answered to ``Mixer.decode_plan`` for this step: set only
    # on the context of a recorded step, whose host arrays say nothing about the steps it will replay
    decode_plans: dict = field(default_factory=dict)
    # where the head may leave the first stage of every row's argmax (``parts.base.ArgmaxStage``):
    # offered by a step that chooses every row's token on the device right after the forward pass
    argmax_stage: Any = None
    _tiles: dict = field(default_factory=dict)
    _memo: dict = field(default_factory=dict)

    @property
    def max_kv_len(self) -> int:
        return int(self.kv_len_host.max()) if self.num_entries else 0

    @property
    def max_decode_kv_len(self) -> int:
        return int(self.kv_len_host[:self.num_decode].max()) if self.num_decode else 0

    def entry_rows(self, e: int) -> tuple[int, int]:
        return int(self.q_start_host[e]), int(self.q_start_host[e + 1])

    def begin_forward(self) -> None:
        """Called at the start of every forward pass over this context: forgets what parts derived
        from arrays that may have changed on the device since the last pass (positions move when a
        graph runs several decode steps on one context)."""
        self._memo.clear()

    def memo(self, key: Hashable, make: Callable[[], Any]) -> Any:
        """``make()``, made at the first call with this key in a forward pass and kept until the
        next pass begins: for what several layers derive alike from the step's device arrays."""
        hit = self._memo.get(key)
        if hit is None:
            hit = self._memo[key] = make()
        return hit

    def is_fresh(self, e: int) -> bool:
        """The entry starts its request at position 0 (per-request state must be reset)."""
        q0, q1 = self.entry_rows(e)
        return int(self.kv_len_host[e]) - (q1 - q0) == 0

    def upload(self, arrays: Sequence[np.ndarray]) -> list[torch.Tensor]:
        """The host arrays as device tensors on the step's device (one copy for all of them)."""
        return upload(arrays, self.device)

    def step_lists(self, key: Hashable, make: Callable[[], Any]) -> Any:
        """``make()``, made once per key and kept as long as the context: for lists that depend on
        the step's host arrays alone (which entry brings how many tokens over how many keys),
        such as the tile lists of the attention kernels."""
        hit = self._tiles.get(key)
        if hit is None:
            hit = self._tiles[key] = make()
        return hit

    def q_tiles(self, rows_per_tile: int, first_entry: int = 0,
                last_entry: Optional[int] = None) -> tuple[torch.Tensor, torch.Tensor]:
        """Query tiles ``(entry, first query of the tile)`` of entries ``[first, last)``, by entry
        and then by query, as two int32 device vectors; built once per step and tile height."""
        last = self.num_entries if last_entry is None else last_entry

        def make() -> tuple[torch.Tensor, torch.Tensor]:
            ent: list[int] = []
            q0s: list[int] = []
            for e in range(first_entry, last):
                length = int(self.q_start_host[e + 1] - self.q_start_host[e])
                for q0 in range(0, length, rows_per_tile):
                    ent.append(e)
                    q0s.append(q0)
            return tuple(self.upload([np.asarray(ent, np.int32), np.asarray(q0s, np.int32)]))

        return self.step_lists(("query tiles", rows_per_tile, first_entry, last), make)
