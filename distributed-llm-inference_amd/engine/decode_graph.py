"""HIP-graph replay of decode steps.

A step in which every request brings exactly one token always launches the same kernels with the
same grids; only the contents of a few small integer arrays change (token ids, positions, cache
slots, lengths, block tables). Such steps are captured once per (batch bucket, key-split factor)
into a HIP graph whose kernels read those arrays from fixed device addresses; a later step copies
its arrays there with one host-to-device copy and replays the graph. That removes the per-kernel
launch cost, which would otherwise exceed the step's memory time at small batches.

A batch smaller than its bucket is padded with rows that have no keys and no cache slot: they
write nothing and their logits are dropped. Capture uses the same model code as eager steps.
No memset node is recorded: buffers that must start at zero are cleared by fill kernels.

The reference replays CUDA graphs of batched decode in fixed buckets the same way
(src/dli/engine/cuda_graph.py:19-21,137-144), padding rows into a scratch block.
"""

from __future__ import annotations

import gc
import weakref

from dataclasses import dataclass
from typing import Optional, Sequence

import numpy as np
import torch

from ..kernels import ops
from ..parts.base import ArgmaxStage
from .batch import GroupView, StepContext, StepEntry
from .table_rows import TableRows


# A recording costs as much time as ten to twenty decode steps; a recorded shape of more rows that
# stands in costs a tenth to a third of a step more. A shape is recorded once it has been asked for
# RECORD_AFTER_STEPS decode steps, at once if nothing recorded can stand in, or if what can has more
# than STAND_IN_ROWS times its rows.
RECORD_AFTER_STEPS = 64
STAND_IN_ROWS = 4

_RECORDERS: "weakref.WeakSet[DecodeGraphs]" = weakref.WeakSet()  # every recorder that has not been collected yet


def _bucket(n: int) -> int:
    b = 1
    while b < n:
        b *= 2
    return b


def _batch_bucket(n: int) -> int:
    """Rows of the graph that serves ``n`` requests: powers of two up to 32, then multiples of 16
    (a product's cost grows with its row tiles of 16: 40 requests run on 48 rows, not 64)."""
    return _bucket(n) if n <= 32 else -(-n // 16) * 16


@dataclass
class _Captured:
    graph: torch.cuda.CUDAGraph
    ctx: StepContext
    host: torch.Tensor      # pinned int32 staging, same layout as dev
    dev: torch.Tensor
    logits: torch.Tensor
    views: dict             # name -> numpy view into host
    width: int              # block-table entries per row
    rows: TableRows         # what the block-table rows hold, so that a replay patches them
    tokens_host: Optional[torch.Tensor] = None  # pinned int32 [steps * b]: sampled tokens (sampling graphs)
    staged: Optional[torch.cuda.Event] = None   # the last copy of host to dev: host is not refilled before it


class DecodeGraphs:
    def __init__(self, step_fn, *, max_batch: int, max_blocks_per_seq: int) -> None:
        self.step_fn = step_fn
        self.rt = step_fn.rt
        self.max_batch = max_batch
        self.max_width = max(1, max_blocks_per_seq)
        self.n_groups = step_fn.manager.num_groups
        self.captured: dict[tuple, _Captured] = {}
        self._asked: dict[tuple, int] = {}   # decode steps that a shape that is not recorded has been asked for
        _RECORDERS.add(self)
        self.replays = 0
        self.enabled = self._supported()

    def _supported(self) -> bool:
        """Graphs are recorded in bfloat16, for models all of whose mixers can be recorded."""
        if self.rt.dtype != torch.bfloat16:
            return False
        return self.step_fn.model.graph_capturable(self.step_fn.store.page_size)

    def can_run(self, entries: Sequence[StepEntry], steps: int = 1) -> bool:
        if not self.enabled or not entries or len(entries) > self.max_batch:
            return False
        ps = self.step_fn.manager.page_size
        return all(len(e.tokens) == 1 and e.start + steps <= self.max_width * ps for e in entries)

    # ------------------------------------------------------------------ capture

    def _layout(self, b: int, width: int) -> tuple[dict, int]:
        fields = [("token_ids", b), ("positions", b), ("q_start", b + 1), ("kv_len", b), ("state_slots", b),
                  ("logit_rows", b)]
        fields += [("temperature", b), ("top_p", b), ("top_k", b), ("seeds", 2 * b), ("counters", 2 * b)]
        for g in range(self.n_groups):
            fields += [(f"slots{g}", b), (f"tables{g}", b * width)]
        offsets, at = {}, 0
        for name, n in fields:
            offsets[name] = (at, n)
            at += -(-n // 4) * 4  # 16-byte aligned starts
        return offsets, at

    def _capture(self, b: int, plans: tuple, width: int, sampled: bool, steps: int = 1) -> _Captured:
        dev_name = self.rt.device
        offsets, total = self._layout(b, width)
        host = torch.zeros(total, dtype=torch.int32).pin_memory()
        dev = torch.zeros(total, dtype=torch.int32, device=dev_name)
        hv = host.numpy()
        views = {name: hv[o:o + n] for name, (o, n) in offsets.items()}
        dv = {name: dev[o:o + n] for name, (o, n) in offsets.items()}
        # a batch of padding rows: no keys, no slot
        views["q_start"][:] = np.arange(b + 1)
        views["logit_rows"][:] = np.arange(b)
        for g in range(self.n_groups):
            views[f"slots{g}"][:] = -1
        views["state_slots"][:] = self.step_fn.store.scratch_slot
        dev.copy_(host)
        groups = [GroupView(dv[f"slots{g}"], dv[f"tables{g}"].view(b, width), width)
                  for g in range(self.n_groups)]
        ctx = StepContext(
            device=dev_name, page_size=self.step_fn.manager.page_size, num_tokens=b, num_entries=b,
            num_decode=b, token_ids=dv["token_ids"], positions=dv["positions"], q_start=dv["q_start"],
            kv_len=dv["kv_len"], state_slots=dv["state_slots"], logit_rows=dv["logit_rows"], groups=groups,
            q_start_host=np.arange(b + 1, dtype=np.int32), kv_len_host=np.zeros(b, np.int32),
            state_slots_host=np.zeros(b, np.int32), seq_ids=[None] * b)
        ctx.decode_plans = {id(part): plan for part, plan in zip(self.step_fn.plan_owners, plans)}
        ctx.all_rows_wanted = True  # logit_rows is the identity here
        model, caches = self.step_fn.model, self.step_fn.caches
        side = torch.cuda.Stream()
        views["temperature"].view(np.float32)[:] = 0.0  # padding rows are greedy
        views["top_p"].view(np.float32)[:] = 1.0
        views["top_k"][:] = -1
        tokens_host = tokens_dev = tokens_all = scratch = None
        if sampled:
            tokens_host = torch.zeros(steps * b, dtype=torch.int32).pin_memory()
            tokens_dev = torch.zeros(b, dtype=torch.int32, device=dev_name)
            tokens_all = torch.zeros(steps, b, dtype=torch.int32, device=dev_name)
            scratch = ops.sample_scratch(b, dev_name)
            stage = ArgmaxStage(scratch)
            ctx.argmax_stage = stage
        ps = self.step_fn.manager.page_size

        def body(steps=steps):
            # `steps` decode steps back to back: after each, the sampled tokens become the next
            # inputs and positions, lengths, slots and draw counters move on, all on the device
            for j in range(steps):
                if sampled:
                    stage.parts = 0  # the head may do the first stage of the argmax and say so
                logits = model.forward(ctx, caches)
                if sampled:
                    ops.sample_and_advance(
                        logits, dv["temperature"].view(torch.float32), dv["top_k"], dv["top_p"].view(torch.float32),
                        dv["seeds"].view(torch.int64), dv["counters"].view(torch.int64), tokens_dev, scratch,
                        stage.parts, tokens_all[j], dv["token_ids"], dv["positions"], dv["kv_len"],
                        [g.slots for g in groups], [g.block_tables for g in groups], ps, advance=j + 1 < steps)
            if sampled:
                tokens_host.copy_(tokens_all.view(-1), non_blocking=True)
            return logits

        # One step outside the capture: what the parts and the libraries set up at their first call
        # with these shapes (buffers that live on, plans of products) must not happen inside it.
        dev.copy_(host)
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            body(1)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        # No cyclic garbage collection while the stream is capturing: a dead cycle that holds
        # device memory or an older graph (an engine that was dropped) would be destroyed in the
        # middle of the capture, and freeing those is not allowed there (the process aborts).
        # Where the process has had other recorders than this one, such cycles are collected here,
        # before the capture, with the device idle (an older graph is then never taken apart while
        # a newer one runs). A process with one engine skips this: the collection takes 30 ms
        # beside a loaded model, three times what the recording itself takes.
        collecting = gc.isenabled()
        if len(_RECORDERS) > 1:
            gc.collect()
        gc.disable()
        try:
            with torch.cuda.graph(graph):
                logits = body()
        finally:
            if collecting:
                gc.enable()
        return _Captured(graph, ctx, host, dev, logits, views, width, TableRows(b, width, self.n_groups), tokens_host)

    def _shape_key(self, requests: int, max_kv: int, sampled: bool, steps: int) -> tuple:
        """The captured shape that serves ``requests`` requests of which the longest will hold
        ``max_kv`` keys: (padded batch, what each part that keeps a cache plans for such a step,
        block-table width, sampled, steps). The parts plan for the requests that are there, not
        for the padded rows, which bring no work (17 requests on a graph of 32 rows: planned for
        32, the attention cut each request's keys into two runs where 17 requests want four, and
        took 38.6 us a layer instead of 29)."""
        b = _batch_bucket(requests)
        width = max(16, _bucket(-(-max_kv // self.step_fn.manager.page_size)))
        plans = tuple(part.decode_plan(requests, max_kv) for part in self.step_fn.plan_owners)
        return (b, plans, width, sampled, steps)

    def _stand_in(self, key: tuple, requests: int) -> Optional[tuple]:
        """The recorded shape with the fewest rows (then with the same plans, then the narrowest
        block table) that can run a step of ``key``'s kind for ``requests`` requests: as many
        tokens a step, sampled alike, rows and table width at least as large. What its parts
        planned may have been planned for another batch: that costs speed, never a result."""
        def order(k):
            return (k[0], k[1] != key[1], k[2])

        best = None
        for other, cap in self.captured.items():
            if (other[3:] == key[3:] and requests <= other[0] <= STAND_IN_ROWS * key[0]
                    and other[2] >= key[2]):
                if best is None or order(other) < order(best[0]):
                    best = (other, cap)
        return best

    def warm_up(self, batches: Sequence[int], max_len: int, *, sampled: bool = True,
                steps: Sequence[int] = (1,)) -> int:
        """Capture now every graph that decode steps of ``batches`` requests with up to ``max_len``
        keys can ask for, so that no capture (two eager forwards and a recording) falls between
        two tokens of a live request later. Returns the number of graphs captured by this call."""
        if not self.enabled:
            return 0
        ps = self.step_fn.manager.page_size
        max_len = min(int(max_len), self.max_width * ps)
        keys = set()
        for n in batches:
            if not 0 < n <= self.max_batch:
                raise ValueError(f"batch {n} outside 1..{self.max_batch}")
            for k in steps:
                # the shape changes only just after the page count passes a power of two and where the
                # key count reaches a multiple of 128 (the unit of the split rule)
                edges = {*range(128, max_len + 1, 128), *(ps * 2 ** i for i in range(32) if ps * 2 ** i <= max_len)}
                for kv in sorted({1, max_len, *edges, *(e + 1 for e in edges if e < max_len)}):
                    keys.add(self._shape_key(n, kv, sampled, k))
        made = 0
        for key in sorted(keys):
            if key not in self.captured:
                self.captured[key] = self._capture(*key)
                made += 1
        return made

    # ------------------------------------------------------------------ replay

    def run(self, entries: Sequence[StepEntry], sampling: Optional[Sequence[tuple]] = None, steps: int = 1):
        """A decode-only step. Without ``sampling``: logits ``[wanted, vocab]`` (a view of the
        graph's output: use it before the next step). With ``sampling``, one
        ``(temperature, top_k, top_p, seed, draw index)`` per entry: the graph samples too and the
        chosen token ids come back as a list; with ``steps`` > 1 the graph runs that many decode
        steps in a row and one list per step comes back (the block tables must already hold the
        pages of all positions that will be written)."""
        mgr = self.step_fn.manager
        n = len(entries)
        sampled = sampling is not None
        if steps > 1 and not sampled:
            raise ValueError("several steps in a row need the sampling parameters")
        key = self._shape_key(n, max(e.start + steps for e in entries), sampled, steps)
        cap = self.captured.get(key)
        if cap is None:
            # A shape that has been asked for little (the tail of a batch, whose requests end one
            # by one) is served by a recorded shape of more rows or a wider block table.
            self._asked[key] = self._asked.get(key, 0) + steps
            stand_in = self._stand_in(key, n) if self._asked[key] < RECORD_AFTER_STEPS else None
            if stand_in is not None:
                key, cap = stand_in
            else:
                cap = self.captured[key] = self._capture(*key)
        b = key[0]
        v = cap.views
        if cap.staged is not None:
            # a caller that used the last logits without waiting for them (a copy on the stream,
            # say) comes back while the copy of the staging buffer may still be queued
            cap.staged.synchronize()
        limit = self.step_fn.store.num_pages
        token_ids, positions, kv_len, state_slots = v["token_ids"], v["positions"], v["kv_len"], v["state_slots"]
        # The step's arrays are filled in bulk (one conversion per array instead of one per number):
        # at large batches this loop is a visible part of the step.
        toks = [int(e.tokens[0]) for e in entries]
        starts = [e.start for e in entries]
        if min(toks) < 0 or max(toks) >= self.step_fn.vocab_size:
            bad = next(e for e, t in zip(entries, toks) if not 0 <= t < self.step_fn.vocab_size)
            raise ValueError(f"request {bad.seq_id!r}: token id {int(bad.tokens[0])} outside the vocabulary")
        token_ids[:n] = toks
        positions[:n] = starts
        np.add(positions[:n], 1, out=kv_len[:n])
        kv_len[n:] = 0
        token_ids[n:] = 0
        positions[n:] = 0
        state_slots[:n] = [mgr.state_slot(e.seq_id) for e in entries]
        state_slots[n:] = self.step_fn.store.scratch_slot
        rows = []
        for i, e in enumerate(entries):
            if e.want:
                rows.extend(i for _ in e.want)
        for g in range(self.n_groups):
            slots = cap.rows.fill(mgr, entries, g, v[f"tables{g}"], limit)
            v[f"slots{g}"][:n] = slots
            v[f"slots{g}"][n:] = -1
        if sampled:
            temp, top_p = v["temperature"].view(np.float32), v["top_p"].view(np.float32)
            seeds, counters = v["seeds"].view(np.int64), v["counters"].view(np.int64)
            temp[n:] = 0.0
            ts, ks, pp, sd, dr = zip(*sampling)
            temp[:n], v["top_k"][:n], top_p[:n], seeds[:n], counters[:n] = ts, ks, pp, sd, dr
        cap.dev.copy_(cap.host, non_blocking=True)
        if not sampled:  # the sampling path waits for the whole replay below
            if cap.staged is None:
                cap.staged = torch.cuda.Event()
            cap.staged.record()
        cap.graph.replay()
        self.replays += 1
        if sampled:
            torch.cuda.current_stream().synchronize()
            if steps == 1:
                return cap.tokens_host[:n].tolist()
            return [row[:n] for row in cap.tokens_host.view(steps, b).tolist()]
        if rows == list(range(n)):
            return cap.logits[:n]
        if not rows:
            return cap.logits[:0]
        return cap.logits[torch.tensor(rows, device=cap.logits.device)]
