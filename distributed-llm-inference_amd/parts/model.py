"""A model put together from a :class:`ModelSpec`: embedding, scheduled layers, final norm, head.

The model knows nothing of requests or pages: :meth:`Model.forward` takes a
:class:`dli_amd.engine.batch.StepContext` and one :class:`dli_amd.cache.store.LayerCache` per
schedule entry, runs the tokens of the step once through the schedule, and returns float32 logits
of the wanted rows only (rows are selected before the final norm and the head, which are row-wise;
reference: src/dli/model/llama.py:299-305).
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping, Optional, Sequence

import torch

from ..kernels import ops
from .base import Part, Runtime
from .registry import build_part
from .spec import ModelSpec, WeightSpec

# importing the modules registers the built-in parts
from . import attention, block, embedding, feed_forward, head, norm, position  # noqa: F401,E402


@dataclass
class BuiltLayer:
    block: Part
    parts: dict[str, Part]


class BoundCaches(list):
    """The caches of a model's schedule entries, in schedule order (what :meth:`Model.bind_caches`
    returns and :meth:`Model.forward` takes), with room for what the model derives from them: the
    description of its blocks for the loop in C holds the addresses of these very pages, so it
    lives and dies with this list and not with the model."""

    derived: Any = None             # NativeBlocks, or False where that route does not apply
    derived_for: int = -1           # the model's ``weights_version`` it was made for


def _walk(part: Part):
    yield part
    for sub in part.sub_parts().values():
        yield from _walk(sub)


class Model:
    def __init__(self, spec: ModelSpec, runtime: Runtime) -> None:
        self.spec, self.rt = spec, runtime
        self.embedding = build_part("embedding", spec.embedding, runtime)
        self.layers: list[BuiltLayer] = []
        for ls in spec.layers:
            blk = build_part("block", ls.block, runtime)
            missing = [r for r in blk.roles if r not in ls.parts]
            if missing:
                raise ValueError(f"block {ls.block.kind!r} needs the roles {missing}")
            parts = {role: build_part(family, ps, runtime) for role, (family, ps) in ls.parts.items()}
            self.layers.append(BuiltLayer(blk, parts))
        self.final_norm = build_part("norm", spec.final_norm, runtime)
        self.head = build_part("head", spec.head, runtime)
        self.weights_version = 0   # counts load_weights(): what was derived from older tensors is stale
        self.native_steps = True   # steps with portions: all layers' launches from one call where the blocks allow
        self.native_runs = 0       # how many steps went that way

    # ------------------------------------------------------------------ weights

    def _all_parts(self) -> list[Part]:
        tops: list[Part] = [self.embedding]
        for layer in self.layers:
            tops.append(layer.block)
            tops.extend(layer.parts.values())
        tops += [self.final_norm, self.head]
        out: list[Part] = []
        for t in tops:
            out.extend(_walk(t))
        return out

    def weight_specs(self) -> dict[str, WeightSpec]:
        """Every tensor the model binds, by checkpoint name."""
        out: dict[str, WeightSpec] = {}
        for part in self._all_parts():
            for local, ws in part.weight_specs().items():
                name = part.prefix + local
                if name in out and out[name] != ws:
                    raise ValueError(f"two parts bind {name!r} with different specs")
                out[name] = ws
        return out

    def load_weights(self, tensors: Mapping[str, torch.Tensor]) -> None:
        """Hand every part its tensors (by checkpoint name), tie the head, finalize."""
        for part in self._all_parts():
            local = {}
            for name in part.weight_specs():
                full = part.prefix + name
                if full in tensors:
                    local[name] = tensors[full]
            part.load_weights(local)
        self.head.tie(self.embedding.table())
        for part in self._all_parts():
            part.finalize()
        self.weights_version += 1

    # ------------------------------------------------------------------ cache needs

    def cache_specs(self) -> list[Optional[Any]]:
        """What each schedule entry keeps per request (``None``: nothing of its own)."""
        return [None if owner is None or entry.cache_of is not None else owner.cache_spec()
                for entry, owner in zip(self.spec.schedule, self.cache_owners())]

    def cache_owners(self) -> list[Optional[Part]]:
        """Per schedule entry, the part of its layer that keeps something per request: whichever
        part, in whatever role, answers ``cache_spec()`` with a spec. A schedule entry has one
        cache, so a layer with two such parts is refused."""
        out: list[Optional[Part]] = []
        for entry in self.spec.schedule:
            owners = [(role, part) for role, part in self.layers[entry.layer].parts.items()
                      if callable(getattr(part, "cache_spec", None)) and part.cache_spec() is not None]
            if len(owners) > 1:
                raise ValueError(f"layer {entry.layer}: the parts {[r for r, _ in owners]} each keep a cache; "
                                 f"a schedule entry has one (put them in entries of their own)")
            out.append(owners[0][1] if owners else None)
        return out

    def graph_capturable(self, page_size: int) -> bool:
        """Whether decode steps of this model may be recorded into device graphs: every part of it
        says so (``Part.graph_capturable``; a mixer answers for the parts it owns)."""
        parts = [self.embedding, self.final_norm, self.head]
        for layer in self.layers:
            parts.append(layer.block)
            parts.extend(layer.parts.values())
        return all(p.graph_capturable(page_size) for p in parts)

    def bind_caches(self, layer_caches: Sequence[Any]) -> BoundCaches:
        """Per schedule entry, the cache it uses: its own, or a read-only view of another's."""
        out = BoundCaches()
        for i, entry in enumerate(self.spec.schedule):
            if entry.cache_of is not None:
                src = layer_caches[entry.cache_of]
                out.append(src.reader() if src is not None else None)
            else:
                out.append(layer_caches[i])
        return out

    # ------------------------------------------------------------------ step

    STREAM_ROWS = 64  # steps with at most this many rows, all decoding, take the fused kernels

    def _streams(self, ctx: Any) -> bool:
        # Steps that hold a portion run eagerly, where the host's time per launch decides: the fused
        # kernels would be fewer launches, but issued one by one from Python they take longer than
        # the plain kernels issued from the loop in C (2.1 against 1.7 ms for 64 tokens at the 1B sizes).
        if not 0 < ctx.num_tokens <= self.STREAM_ROWS or ctx.num_decode != ctx.num_entries:
            return False
        if not (self.embedding.streams(ctx) and self.head.streams(ctx) and hasattr(self.final_norm, "fused_params")):
            return False
        return all(hasattr(l.block, "forward_stream") and l.block.streams(ctx, l.parts) for l in self.layers)

    def _forward_stream(self, ctx: Any, caches: Sequence[Any]) -> torch.Tensor:
        stream = self.embedding.forward_stream(ctx.token_ids)
        order = [self.layers[entry.layer] for entry in self.spec.schedule]
        for i, (layer, cache) in enumerate(zip(order, caches)):
            # the norm that the stream meets next: the following entry's first, or the final one
            after = order[i + 1].block.first_norm(order[i + 1].parts) if i + 1 < len(order) else self.final_norm
            layer.block.forward_stream(stream, ctx, cache, layer.parts, following=after)
        if ctx.argmax_stage is not None:  # offered by a step that samples every row on the device
            logits = self.head.forward_stream(stream, self.final_norm, ctx.argmax_stage)
        else:
            logits = self.head.forward_stream(stream, self.final_norm)
        k = ctx.logit_rows.shape[0]
        if getattr(ctx, "all_rows_wanted", False):
            return logits
        out = torch.empty(k, logits.shape[1], device=logits.device, dtype=torch.float32)
        if k:
            ops.gather_rows(logits, ctx.logit_rows, out)
        return out

    def _native_blocks(self, caches: Sequence[Any]):
        """The schedule as one array of block descriptions for the loop in C, made once per bound
        list of caches and set of weights and kept on that list; ``None`` if some block or cache
        is not of the kind that route covers, or the caches are not a :class:`BoundCaches`."""
        if not isinstance(caches, BoundCaches):
            return None
        if caches.derived is None or caches.derived_for != self.weights_version:
            from .native import NativeBlocks

            caches.derived = NativeBlocks.build(self, caches) or False
            caches.derived_for = self.weights_version
        return caches.derived or None

    def forward(self, ctx: Any, caches: Sequence[Any]) -> torch.Tensor:
        """Run the step's tokens through the schedule; float32 logits ``[wanted rows, vocab]``."""
        ctx.begin_forward()
        if self._streams(ctx):
            return self._forward_stream(ctx, caches)
        x = self.embedding.forward(ctx.token_ids)
        delta: Optional[torch.Tensor] = None
        native = self._native_blocks(caches) if self.rt.is_bf16 and self.native_steps and ctx.num_tokens > 0 else None
        if native is not None:
            delta = native.run(x, ctx)      # every layer's launches from one call; None: nothing ran
            self.native_runs += delta is not None
        if delta is None:
            for entry, cache in zip(self.spec.schedule, caches):
                layer = self.layers[entry.layer]
                x, delta = layer.block.forward(x, delta, ctx, cache, layer.parts)
        k = ctx.logit_rows.shape[0]
        if k == 0:
            return torch.empty(0, self.spec.vocab_size, device=self.rt.device, dtype=torch.float32)
        xs = torch.empty(k, x.shape[1], device=x.device, dtype=x.dtype)
        ops.gather_rows(x, ctx.logit_rows, xs)
        ds = None
        if delta is not None:
            ds = torch.empty_like(xs)
            ops.gather_rows(delta, ctx.logit_rows, ds)
        h = self.final_norm.forward(xs, ds)
        return self.head.forward(h)
