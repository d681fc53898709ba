"""Trace replay: feeds given token ids through a model step by step and writes logits.

    trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N

Steps come on standard input, one JSON object a line::

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

All entries of a step run as one batch through the engine's own step function, cache manager and
kernels (this module has no forward pass of its own and samples nothing). For a step in which
something is wanted, ``OUT/<step>.f32`` receives the logits at the wanted places, in the order of
the entries and of ``want``, as little-endian float32 ``[wanted, vocab]``. After every step a line
``done <step>`` is printed and flushed. Requests named in ``end`` give back what they hold after
the step. The cache pool is made for ``--max-tokens`` tokens, so pages are used again.

The reference has no such tool; its nearest relatives are ``PagedSequence.prefill/feed``
(src/dli/generate.py:98-138) and the teacher-forcing runner of src/dli/bench/precision.py:210-230.
"""

from __future__ import annotations

import argparse
import json
import sys
from pathlib import Path
from typing import Any, Optional, Sequence, TextIO

import numpy as np

PAGE_SIZE = 16  # divides the 64 tokens that each request's count is rounded up to


class TraceError(ValueError):
    """A step that cannot be replayed."""


class TraceSession:
    """Replays steps on an engine core: reserves cache for each entry's tokens, runs the step
    function, gives back what ended requests hold. Shared by the command line and by tests."""

    def __init__(self, core: Any) -> None:
        self.core = core
        self.fed: dict[Any, int] = {}

    def step(self, entries: Sequence[dict], end: Sequence[Any] = ()):
        """``entries``: ``{"id", "tokens", "want"}`` dictionaries. Returns float32 logits
        ``[wanted, vocab]`` (device tensor) in the order of the entries and of ``want``."""
        from .engine.batch import StepEntry

        mgr = self.core.manager
        batch, copies = [], []
        for ent in entries:
            rid, tokens = ent.get("id"), [int(t) for t in ent.get("tokens") or []]
            want = [int(w) for w in ent.get("want") or []]
            if rid is None or not tokens:
                raise TraceError("an entry needs an id and at least one token")
            if rid not in self.fed:
                # On a core with content reuse the leading pages may be another request's, already
                # computed: only the rest of the tokens runs, and nothing can be wanted before it.
                skip = mgr.allocate(rid, tokens, respect_watermark=False).num_cached_tokens
                if any(w < skip for w in want):
                    mgr.free(rid)
                    raise TraceError(f"request {rid!r}: logits wanted at a place whose page was reused")
                self.fed[rid] = skip
                tokens, want = tokens[skip:], [w - skip for w in want]
            else:
                copies.extend(mgr.append_slots(rid, tokens))
            batch.append(StepEntry(rid, tokens, self.fed[rid], want))
        logits = self.core.step.run(batch, copies)
        for e in batch:
            self.fed[e.seq_id] += len(e.tokens)
        for rid in end:
            if rid in self.fed:
                mgr.free(rid)
                del self.fed[rid]
        return logits


    def fork(self, parent: Any, child: Any) -> None:
        """``child`` continues from everything ``parent`` has been fed, sharing its pages; the
        first write of either into a shared, partly filled page copies that page first."""
        if self.core.store.stateful:
            raise TraceError("a model with per-request state cannot be forked here")
        if parent not in self.fed or child in self.fed:
            raise TraceError(f"cannot fork {parent!r} into {child!r}")
        self.core.manager.fork(parent, child)
        self.fed[child] = self.fed[parent]


class TraceRunner:
    def __init__(self, model_dir: str | Path, dtype: str, out_dir: str | Path, max_tokens: int,
                 page_size: int = PAGE_SIZE, max_live: int = 64) -> None:
        from .engine.core import build_core

        if max_tokens < 1:
            raise TraceError("--max-tokens must be positive")
        self.out_dir = Path(out_dir)
        self.out_dir.mkdir(parents=True, exist_ok=True)
        num_pages = -(-max_tokens // page_size)
        # No content reuse here: a step must run exactly the tokens it brings.
        core = build_core(model_dir, num_pages=num_pages, page_size=page_size, max_seqs=max_live,
                          dtype=dtype, enable_prefix_caching=False, watermark=0.0)
        core.step.enable_decode_graphs(max_live, num_pages * page_size)  # as serving does
        self.session = TraceSession(core)

    def run_step(self, record: dict) -> Optional[Path]:
        step = record.get("step")
        if not isinstance(step, int):
            raise TraceError(f"a step needs an integer 'step', got {step!r}")
        try:
            logits = self.session.step(record.get("entries") or [], record.get("end") or [])
        except TraceError as exc:
            raise TraceError(f"step {step}: {exc}") from exc
        path = None
        if logits.shape[0] > 0:
            path = self.out_dir / f"{step}.f32"
            logits.cpu().numpy().astype("<f4", copy=False).tofile(path)
        return path

    def replay(self, lines: TextIO, done: TextIO) -> int:
        count = 0
        for line in lines:
            line = line.strip()
            if not line:
                continue
            try:
                record = json.loads(line)
            except json.JSONDecodeError as exc:
                raise TraceError(f"input line {count + 1} is not JSON: {exc}") from exc
            self.run_step(record)
            done.write(f"done {record['step']}\n")
            done.flush()
            count += 1
        return count


def main(argv: Optional[Sequence[str]] = None) -> int:
    p = argparse.ArgumentParser(prog="trace_run", description=__doc__,
                                formatter_class=argparse.RawDescriptionHelpFormatter)
    p.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    p.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    p.add_argument("--out", required=True, help="folder that receives <step>.f32")
    p.add_argument("--max-tokens", type=int, required=True,
                   help="most tokens that live requests hold at any time (each rounded up to 64)")
    p.add_argument("--page-size", type=int, default=PAGE_SIZE,
                   help=f"token slots of a cache page (default {PAGE_SIZE}; the pool is --max-tokens / this)")
    args = p.parse_args(argv)
    try:
        if args.page_size < 1 or 64 % args.page_size:
            raise TraceError("--page-size must divide the 64 tokens that a request's count is rounded up to")
        runner = TraceRunner(args.model, args.dtype, args.out, args.max_tokens, page_size=args.page_size)
        runner.replay(sys.stdin, sys.stdout)
    except Exception as exc:  # one clear line, non-zero exit
        print(f"trace_run: {type(exc).__name__}: {exc}", file=sys.stderr, flush=True)
        return 1
    return 0


if __name__ == "__main__":
    sys.exit(main())
