"""The step function: one batch of (request, its next tokens) in, logits at the wanted places out.

It runs only the tokens it is given, as one batch, against the cache that earlier steps left:
each entry's keys and values are written at the slots that the cache manager reserved for them,
every row attends to its own request's pages, and afterwards the tokens are marked computed.
The logits at a position do not depend on how the request's tokens were cut into steps, on what
else is in the batch, or on which pages are used.

Reference: ``ModelRunner.execute`` (src/dli/engine/runner.py:53-183): copy-on-write copies first,
then the flattened batch with single-token rows before portions, one forward pass, logits in the
caller's order, ``mark_computed`` for every chunk.
"""

from __future__ import annotations

from typing import Optional, Sequence

import numpy as np
import torch

from ..cache.manager import RELEASED, CacheManager, CopyOp
from ..cache.store import CacheStore
from ..parts.model import Model
from .batch import GroupView, HostBatch, StepContext, StepEntry, upload


MAX_DECODE_STEPS = 8  # tokens per request that one graph replay may decode


class StepError(ValueError):
    """A batch that the step function refuses (it would read or write outside a request's cache)."""


class StepFunction:
    def __init__(self, model: Model, manager: CacheManager, store: CacheStore) -> None:
        if manager.page_size != store.page_size:
            raise ValueError("cache manager and store disagree on the page size")
        if manager.num_groups != max(1, len(store.groups)):
            raise ValueError("cache manager and store disagree on the number of groups")
        self.model, self.manager, self.store = model, manager, store
        self.rt = model.rt
        self.caches = model.bind_caches(store.layers)
        self.vocab_size = model.spec.vocab_size
        self.steps_run = 0
        self.graphs = None  # DecodeGraphs, when the engine enables graph replay of decode steps
        # the parts that keep something per request, each once: they are asked how they would lay
        # out a decode step before one is recorded (``Mixer.decode_plan``)
        self.plan_owners = list({id(part): part for part in model.cache_owners()
                                 if part is not None and hasattr(part, "decode_plan")}.values())

    def enable_decode_graphs(self, max_batch: int, max_model_len: int) -> None:
        """Replay decode-only steps through HIP graphs (bfloat16 with the matrix-core decode path
        only; other steps run eagerly)."""
        from .decode_graph import DecodeGraphs

        self.graphs = DecodeGraphs(self, max_batch=max_batch,
                                   max_blocks_per_seq=-(-max_model_len // self.manager.page_size))
        if not self.graphs.enabled:
            self.graphs = None

    # ------------------------------------------------------------------ batch building

    def build_context(self, entries: Sequence[StepEntry]) -> StepContext:
        """Check the entries against the cache manager and lay the batch out on the device."""
        return self.upload_context(self.lay_out(entries))

    def lay_out(self, entries: Sequence[StepEntry]) -> HostBatch:
        """Check the entries against the cache manager and lay the batch out in host arrays."""
        mgr, ps = self.manager, self.manager.page_size
        count = len(entries)
        seen = set()
        lengths = []
        for e in entries:
            if e.seq_id in seen:
                raise StepError(f"request {e.seq_id!r} appears twice in one step")
            seen.add(e.seq_id)
            n = len(e.tokens)
            lengths.append(n)
            if n == 0:
                raise StepError(f"request {e.seq_id!r} brings no tokens")
            computed = mgr.num_computed_tokens(e.seq_id)
            if e.start != computed:
                raise StepError(
                    f"request {e.seq_id!r}: portion starts at {e.start} but {computed} tokens are computed")
            if e.start + n > mgr.num_tokens(e.seq_id):
                raise StepError(f"request {e.seq_id!r}: no cache slots reserved up to {e.start + n}")
            for wnt in e.want:
                if not 0 <= int(wnt) < n:
                    raise StepError(f"request {e.seq_id!r}: wanted place {wnt} outside its {n} tokens")

        # single-token entries first, then portions; each kind in the given order
        order = [i for i in range(count) if lengths[i] == 1] + [i for i in range(count) if lengths[i] != 1]
        num_decode = sum(1 for n in lengths if n == 1)
        ordered = [entries[i] for i in order]
        q_start = np.zeros(count + 1, np.int32)
        np.cumsum([lengths[i] for i in order], out=q_start[1:])
        first_row = dict(zip(order, q_start[:-1].tolist()))
        total = int(q_start[-1])
        starts = np.asarray([e.start for e in ordered], np.int64)
        kv_len = (starts + np.asarray([lengths[i] for i in order], np.int64)).astype(np.int32)
        state_slots = np.asarray([mgr.state_slot(e.seq_id) for e in ordered], np.int32)
        token_ids = np.empty(total, np.int64)
        positions = np.empty(total, np.int32)
        # the single tokens at once, the portions one by one
        token_ids[:num_decode] = [e.tokens[0] for e in ordered[:num_decode]]
        positions[:num_decode] = starts[:num_decode]
        for k in range(num_decode, count):
            e, r0, r1 = ordered[k], int(q_start[k]), int(q_start[k + 1])
            token_ids[r0:r1] = e.tokens
            positions[r0:r1] = np.arange(e.start, e.start + r1 - r0)
        if total and (int(token_ids.min()) < 0 or int(token_ids.max()) >= self.vocab_size):
            bad = int(token_ids[(token_ids < 0) | (token_ids >= self.vocab_size)][0])
            raise StepError(f"token id {bad} outside the vocabulary")
        logit_rows = np.asarray(
            [first_row[i] + int(w) for i, e in enumerate(entries) for w in e.want], dtype=np.int32)

        n_groups, limit = mgr.num_groups, self.store.num_pages
        pos64 = positions.astype(np.int64)
        row_entry = np.repeat(np.arange(count), np.diff(q_start)) if total else np.zeros(0, np.int64)
        slots: list[np.ndarray] = []
        tables: list[np.ndarray] = []
        for g in range(n_groups):
            # the block tables of the group as the rows of one array, padded with zeros
            lists = [mgr.table_ref(e.seq_id, g) for e in ordered]
            width = max(map(len, lists), default=1) or 1
            rows = np.zeros((max(count, 1), width), np.int64)
            held = np.zeros(max(count, 1), np.int64)
            for k, t in enumerate(lists):
                rows[k, :len(t)] = t
                held[k] = len(t)
            short = np.flatnonzero(held[:count] * ps < kv_len)
            if short.size:
                raise StepError(f"request {ordered[int(short[0])].seq_id!r}: block table shorter than its keys")
            if rows.size and (int(rows.min()) < RELEASED or int(rows.max()) >= limit):
                raise StepError("a block table names a page outside the pool")
            # a page that the window has passed gives a negative slot, refused here
            where = rows[row_entry, pos64 // ps] * ps + pos64 % ps
            if total and (int(where.min()) < 0 or int(where.max()) >= limit * ps):
                raise StepError("a cache slot lies outside the pool, or in a page that the window has passed")
            rows[rows == RELEASED] = 0  # pages that the window has passed: never read
            slots.append(where)
            tables.append(rows)
        return HostBatch(order=order, seq_ids=[e.seq_id for e in ordered], num_decode=num_decode,
                         token_ids=token_ids, positions=positions, q_start=q_start, kv_len=kv_len,
                         state_slots=state_slots, logit_rows=logit_rows, slots=slots, tables=tables)

    def upload_context(self, batch: HostBatch) -> StepContext:
        """The device-side context of a laid-out step (one copy from pinned memory)."""
        n_groups, total = self.manager.num_groups, batch.num_tokens
        dev = self.rt.device
        # every integer array of the step goes to the device in one copy from pinned memory
        pending: list[np.ndarray] = []

        def to_dev(a: np.ndarray) -> int:
            pending.append(np.ascontiguousarray(a, dtype=np.int32))
            return len(pending) - 1

        group_arrays = [(to_dev(batch.slots[g]), to_dev(batch.tables[g]), batch.tables[g].shape[1])
                        for g in range(n_groups)]
        named = {name: to_dev(a) for name, a in (
            ("token_ids", batch.token_ids), ("positions", batch.positions), ("q_start", batch.q_start),
            ("kv_len", batch.kv_len), ("state_slots", batch.state_slots), ("logit_rows", batch.logit_rows))}
        views = upload(pending, dev)
        groups = [GroupView(views[s_], views[t_], width) for s_, t_, width in group_arrays]
        return StepContext(
            device=dev, page_size=self.manager.page_size, num_tokens=total, num_entries=len(batch.order),
            num_decode=batch.num_decode, groups=groups, q_start_host=batch.q_start, kv_len_host=batch.kv_len,
            state_slots_host=batch.state_slots, seq_ids=batch.seq_ids, **{name: views[i] for name, i in named.items()})

    # ------------------------------------------------------------------ the step

    @property
    def max_decode_steps(self) -> int:
        """Tokens per request that :meth:`run` can decode in one call (``steps``)."""
        return MAX_DECODE_STEPS if self.graphs is not None and self.graphs.enabled else 1

    def run(self, entries: Sequence[StepEntry], copy_ops: Sequence[CopyOp] = (),
            sampling: Optional[Sequence[tuple]] = None, steps: int = 1):
        """Run one step. Returns float32 logits ``[wanted places, vocab]`` on the device, in the
        order of the entries and of each entry's ``want``.

        With ``sampling`` (one ``(temperature, top_k, top_p, seed, draw index)`` for each wanted
        place, temperature 0 meaning greedy) a token is chosen at every wanted place and the list
        of token ids is returned instead.

        ``steps`` > 1 (decode-only batches with ``sampling``, cache room reserved ahead with
        ``CacheManager.reserve_ahead``): every request decodes that many tokens, each sampled
        token being the next input on the device; returns one list of token ids per decoded
        position. The tokens but the last are appended to the requests in the cache manager and
        all positions that were run are marked computed."""
        self.store.copy_pages(copy_ops)  # before any write of this step (runner.py:56)
        if not entries:
            return torch.empty(0, self.vocab_size, device=self.rt.device, dtype=torch.float32)
        if steps > 1:
            return self._run_many(entries, copy_ops, sampling, steps)
        if self.graphs is not None and not copy_ops and self.graphs.can_run(entries):
            for e in entries:  # the same checks as build_context makes
                if e.start != self.manager.num_computed_tokens(e.seq_id):
                    raise StepError(f"request {e.seq_id!r}: portion starts at {e.start} but "
                                    f"{self.manager.num_computed_tokens(e.seq_id)} tokens are computed")
                if e.start + 1 > self.manager.num_tokens(e.seq_id):
                    raise StepError(f"request {e.seq_id!r}: no cache slot reserved at {e.start}")
                if any(int(w) != 0 for w in e.want):
                    raise StepError(f"request {e.seq_id!r}: wanted place outside its one token")
            if len({e.seq_id for e in entries}) != len(entries):
                raise StepError("a request appears twice in one step")
            use_graph_sampler = sampling is not None and all(len(e.want) == 1 for e in entries)
            logits = self.graphs.run(entries, sampling if use_graph_sampler else None)
            if use_graph_sampler:
                tokens, logits = logits, None
        else:
            logits = self.model.forward(self.build_context(entries), self.caches)
        for e in entries:
            self.manager.mark_computed(e.seq_id, e.start + len(e.tokens))
        self.steps_run += 1
        if sampling is None:
            return logits
        if logits is None:
            return tokens
        return self._sample(logits, sampling)

    def _run_many(self, entries: Sequence[StepEntry], copy_ops: Sequence[CopyOp],
                  sampling: Optional[Sequence[tuple]], steps: int) -> list[list[int]]:
        mgr, ps = self.manager, self.manager.page_size
        if steps > self.max_decode_steps:
            raise StepError(f"{steps} tokens per step asked for, {self.max_decode_steps} possible")
        if copy_ops or sampling is None or len(sampling) != len(entries) or any(len(e.tokens) != 1 for e in entries):
            raise StepError("several tokens per step need a decode-only batch that samples every request")
        if len({e.seq_id for e in entries}) != len(entries):
            raise StepError("a request appears twice in one step")
        if not self.graphs.can_run(entries, steps):
            # longer than the graphs were sized for: the same tokens, one step at a time
            rounds, cur = [], list(entries)
            for j in range(steps):
                toks = self.run(cur, (), [(t, k, p, seed, draw + j) for t, k, p, seed, draw in sampling])
                rounds.append(toks)
                if j + 1 < steps:
                    for e, tok in zip(cur, toks):
                        if mgr.append_slots(e.seq_id, [tok]):
                            raise StepError("a page reserved ahead was shared")
                    cur = [StepEntry(e.seq_id, (tok,), e.start + 1, (0,)) for e, tok in zip(cur, toks)]
            return rounds
        for e in entries:
            if e.start != mgr.num_computed_tokens(e.seq_id) or e.start + 1 != mgr.num_tokens(e.seq_id):
                raise StepError(f"request {e.seq_id!r}: its last token must be the only one not computed")
            if tuple(int(w) for w in e.want) != (0,):
                raise StepError(f"request {e.seq_id!r}: the one token's logits must be wanted")
            for g in range(mgr.num_groups):
                if len(mgr.table_ref(e.seq_id, g)) * ps < e.start + steps:
                    raise StepError(f"request {e.seq_id!r}: no cache room reserved for {steps} tokens")
        rounds = self.graphs.run(entries, sampling, steps=steps)
        for i, e in enumerate(entries):
            # all tokens but the last in one call: the pages were reserved, none of them is shared
            if mgr.append_slots(e.seq_id, [rounds[j][i] for j in range(steps - 1)]):
                raise StepError("a page reserved ahead was shared")
            mgr.mark_computed(e.seq_id, e.start + steps)
        self.steps_run += steps
        return rounds

    def _sample(self, logits: torch.Tensor, sampling: Sequence[tuple]) -> list[int]:
        from ..kernels import ops

        rows = logits.shape[0]
        if rows != len(sampling):
            raise StepError("one sampling tuple is needed for each wanted place")
        if rows == 0:
            return []
        dev = logits.device
        temperature, top_p, top_k, seeds, counters = upload(
            [np.asarray([s[0] for s in sampling], np.float32), np.asarray([s[2] for s in sampling], np.float32),
             np.asarray([s[1] for s in sampling], np.int32), np.asarray([s[3] for s in sampling], np.int64),
             np.asarray([s[4] for s in sampling], np.int64)], dev)
        out = torch.empty(rows, dtype=torch.int32, device=dev)
        ops.sample(logits, temperature, top_k, top_p, seeds, counters, out)
        return out.cpu().tolist()
