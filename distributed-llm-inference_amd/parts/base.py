"""What a part of each family must provide.

Every part is constructed as ``cls(runtime, **params)`` with its sizes and constants as keyword
parameters (nothing is read from a model-wide configuration: a part does not know which model it
is in), declares the tensors it binds (:meth:`Part.weight_specs`, names relative to its prefix) and
receives them in :meth:`Part.load_weights`.

Activations are ``[tokens, width]`` tensors of the runtime's activation type, rows of all requests
of the step laid end to end; what belongs to which request is in the :class:`StepContext`.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Hashable, Mapping, Optional, NamedTuple

import torch

from .spec import WeightSpec


@dataclass
class Runtime:
    """Where and in which type the model computes."""

    device: torch.device
    dtype: torch.dtype  # torch.float32 (true 32-bit path) or torch.bfloat16 (serving)
    # bfloat16 only: keep a second copy of each matrix in the order in which the decode kernels
    # read it (faster decode steps of 5 to 16 rows, twice the weight memory)
    decode_weight_copy: bool = True

    @property
    def is_bf16(self) -> bool:
        return self.dtype == torch.bfloat16

    def empty(self, *shape: int, dtype: Optional[torch.dtype] = None) -> torch.Tensor:
        return torch.empty(*shape, device=self.device, dtype=dtype or self.dtype)


# ------------------------------------------------------------------------------ cache requirements

@dataclass(frozen=True)
class PagedKVSpec:
    """A mixer that keeps keys and values of ``kv_heads x head_dim`` per token in pages.

    ``window`` > 0: only the last ``window`` keys are ever read, so pages that lie wholly before
    the window may be given back while the request still runs. ``value_dim``: the size of a
    value where it differs from a key's (``None``: the same; 0: the mixer keeps keys only, a
    compressed cache for instance, and gets no value pages). Layers with equal specs share one
    group of pages and one block table.
    """

    kv_heads: int
    head_dim: int
    window: int = 0
    value_dim: Optional[int] = None

    def __post_init__(self) -> None:
        if self.kv_heads <= 0 or self.head_dim <= 0 or self.window < 0 or (self.value_dim or 0) < 0:
            raise ValueError(f"{self}: heads and sizes must be positive, window and value_dim not negative")

    @property
    def v_dim(self) -> int:
        return self.head_dim if self.value_dim is None else self.value_dim


@dataclass(frozen=True)
class StateSpec:
    """A mixer that keeps a fixed-size state per request: ``shape`` elements of ``dtype`` in the
    slot that the request holds from admission to its end. The slot is zeroed when a request
    takes it."""

    shape: tuple[int, ...]
    dtype: torch.dtype = torch.float32


@dataclass
class DecodeStream:
    """The residual stream of a step with few rows, in the form the fused decode kernels pass on:
    ``x [rows, hidden]`` already holds every residual sum, and ``ssq [parts, rows]`` holds each
    row's sum of squares in parts, as the kernel that last wrote ``x`` left them (the next
    RMSNorm is computed from them inside the product kernel that consumes ``x``)."""

    x: torch.Tensor
    ssq: torch.Tensor
    # The rows of ``x`` already normalised by ``normed_for`` (a norm's weight address and eps),
    # where the kernel that last wrote ``x`` was told which norm follows and applied it too.
    normed: Optional[torch.Tensor] = None
    normed_for: Optional[tuple] = None

    def wrote(self, ssq: torch.Tensor, normed: Optional[torch.Tensor] = None, norm: Any = None) -> None:
        """``x`` has new values: their sums of squares, and their normalised rows if ``norm`` was
        applied as well. Every part that changes ``x`` says so through this call."""
        self.ssq = ssq
        self.normed = normed
        self.normed_for = norm_key(norm) if normed is not None else None

    def normed_by(self, norm: Any) -> Optional[torch.Tensor]:
        """The rows normalised by this very norm, if the last writer left them."""
        return self.normed if self.normed is not None and self.normed_for == norm_key(norm) else None


def norm_key(norm: Any) -> Optional[tuple]:
    """What identifies a norm for :class:`DecodeStream`: its weight's address and its eps."""
    if norm is None or not hasattr(norm, "fused_params"):
        return None
    w, eps = norm.fused_params()
    return (w.data_ptr(), float(eps))


class Part:
    family: str = ""
    kind: str = ""
    prefix: str = ""

    def __init__(self, runtime: Runtime) -> None:
        self.rt = runtime

    def weight_specs(self) -> dict[str, WeightSpec]:
        """Tensors of this part by local name (the checkpoint name is ``prefix + name``)."""
        return {}

    def native_fields(self) -> Optional[dict]:
        """What the loop in C that issues a whole step's launches (:mod:`dli_amd.parts.native`)
        needs to know of this part: tensors and constants by the names of its argument structure,
        or ``None`` (the default) for a part that this route does not cover; the step then runs
        part by part."""
        return None

    def load_weights(self, tensors: Mapping[str, torch.Tensor]) -> None:
        """Receive the tensors of :meth:`weight_specs`, already on the device and typed by role."""

    def sub_parts(self) -> dict[str, "Part"]:
        """Parts owned by this one (their prefix is relative to the checkpoint root)."""
        return {}

    def finalize(self) -> None:
        """Called once after the weights are loaded: build device tables, fuse tensors."""

    def graph_capturable(self, page_size: int) -> bool:
        """Whether this part's work on a step in which every request brings one token may be
        recorded into a device graph and replayed. True promises that it reads such a step only
        through the context's device arrays (``positions``, ``kv_len``, ``state_slots``, the
        groups' slots and block tables: the host copies are stale in a replay), never waits for
        the device, and tolerates padding rows: rows beyond the live requests have no keys, cache
        slot -1 and the state slot that no request holds (``CacheStore.scratch_slot``), which they
        may overwrite. The default is False, and a model is replayed from graphs only if all its
        parts say True (``Model.graph_capturable``); otherwise its decode steps run eagerly."""
        return False

    def streams(self, ctx: Any) -> bool:
        """Whether this part can run ``ctx``'s step on a :class:`DecodeStream` (its
        ``forward_stream``). Parts that do not implement the fused form return False, and the
        model then runs the step through the plain ``forward`` methods."""
        return False


class Embedding(Part):
    """Token ids to rows: ``forward(ids int32 [n]) -> [n, hidden]``."""

    def forward(self, ids: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError

    def table(self) -> torch.Tensor:
        """The ``[vocab, hidden]`` table, for a head that is tied to it."""
        raise NotImplementedError


class Norm(Part):
    """Row-wise normalisation: ``forward(x) -> y``; ``forward(x, delta)`` first replaces ``x`` by
    ``x + delta`` in place (the residual sum, 32-bit arithmetic) and returns the norm of the sum."""

    def forward(self, x: torch.Tensor, delta: Optional[torch.Tensor] = None) -> torch.Tensor:
        raise NotImplementedError


class RotaryTable(NamedTuple):
    """What a rotary encoding hands to the mixer whose kernels rotate.

    ``inv_freq`` float32 ``[dim/2]``; the first ``dim`` components of every head are rotated.
    ``pairing`` says which components form a rotated pair: ``"half"`` pairs component ``i`` with
    ``i + dim/2`` (reference: src/dli/model/rope.py:63-70); a mixer refuses a pairing that its
    kernels do not implement instead of rotating wrongly."""

    inv_freq: torch.Tensor
    dim: int
    pairing: str = "half"


class PositionEncoding(Part):
    """How positions enter a mixer.

    A rotary encoding exposes :meth:`rotary_table` (a :class:`RotaryTable`); the attention mixer
    then rotates inside its fused cache-write kernel. Any other encoding returns ``None`` there
    and implements :meth:`apply`, which rewrites q and k (``[tokens, heads, head_dim]`` views)
    before keys are cached.
    """

    def rotary_table(self) -> Optional[RotaryTable]:
        return None

    def apply(self, q: torch.Tensor, k: Optional[torch.Tensor], positions: torch.Tensor) -> None:
        """In-place change of q and k for the given absolute positions (default: nothing)."""

    def step_angles(self, ctx: Any, dtype: torch.dtype) -> torch.Tensor:
        """For an encoding with a rotary table: cos and sin of the step's positions,
        ``[tokens, 2, dim/2]`` rounded to ``dtype``, for a product kernel that rotates in its
        epilogue. Made by the first layer that asks in a forward pass and shared by all layers
        whose tables are the same tensor (``StepContext.memo``)."""
        from ..kernels import ops

        table = self.rotary_table().inv_freq
        return ctx.memo(("rotary_angles", table.data_ptr(), dtype),
                        lambda: ops.rope_angles(ctx.positions, table, dtype))


class Mixer(Part):
    """The part of a layer that mixes information between positions.

    ``cache_spec()`` says what it keeps per request (pages of keys/values, a fixed-size state, or
    nothing). ``forward(x, ctx, cache)`` gets the normalised rows, the step's context
    (:class:`dli_amd.engine.batch.StepContext`) and the :class:`dli_amd.cache.store.LayerCache` of
    its schedule entry (``None`` without cache), and returns ``[tokens, hidden]``. It must treat
    each request's rows in order and must not let one request's rows influence another's.
    """

    def cache_spec(self) -> Optional[PagedKVSpec | StateSpec]:
        return None

    def decode_plan(self, requests: int, max_keys: int) -> Hashable:
        """How this mixer would lay out a recorded step in which ``requests`` requests bring one
        token each and the longest holds ``max_keys`` keys: any hashable value (``None``: nothing
        to choose). Whoever records such steps for replay asks every mixer, records one graph per
        distinct answer and hands the answer back as ``ctx.decode_plans[id(mixer)]`` while the
        step is recorded, when the host arrays that the mixer would otherwise choose from are
        not there. Answers should be coarse (few distinct ones over the lengths of a request's
        life), since each is a recording of its own."""
        return None

    def forward(self, x: torch.Tensor, ctx: Any, cache: Any) -> torch.Tensor:
        raise NotImplementedError


class FeedForward(Part):
    """Position-wise part: ``forward(x, ctx) -> [tokens, hidden]``."""

    def forward(self, x: torch.Tensor, ctx: Any) -> torch.Tensor:
        raise NotImplementedError


class Block(Part):
    """Arrangement of a layer's parts: where norms sit and where residual sums are made.

    ``forward(x, delta, ctx, cache, parts) -> (x, delta)``. The residual stream is ``x + delta``
    (``delta`` may be ``None``): a block hands its last output back un-added so that the next norm
    can make the sum and normalise in one kernel (``Norm.forward(x, delta)``). ``parts`` maps the
    roles of the layer's :class:`LayerSpec` to built parts."""

    roles: tuple[str, ...] = ()

    def forward(self, x: torch.Tensor, delta: Optional[torch.Tensor], ctx: Any, cache: Any,
                parts: Mapping[str, Part]) -> tuple[torch.Tensor, Optional[torch.Tensor]]:
        raise NotImplementedError

    def native_fields(self, parts: Mapping[str, Part]) -> Optional[dict]:  # type: ignore[override]
        """This arrangement with its parts' tensors and constants, for the loop in C that issues a
        whole step's launches: a dict with the key ``"kind"`` naming an arrangement that the loop
        implements, or ``None`` (the default) for any other; the step then runs part by part."""
        return None

    def streams(self, ctx: Any, parts: Mapping[str, Part]) -> bool:  # type: ignore[override]
        """Whether this arrangement and its parts can run ``ctx``'s step on a
        :class:`DecodeStream` (``forward_stream(stream, ctx, cache, parts, following=...)``)."""
        return False

    def first_norm(self, parts: Mapping[str, Part]) -> Optional["Norm"]:
        """The norm that this arrangement applies to the stream before anything else, if there is
        one: the block before it may apply it in the kernel that writes the stream (the fused
        decode path passes it on as ``following``)."""
        return None


@dataclass
class ArgmaxStage:
    """What a step's sampler offers the head: ``scratch``, float32 values and int32 indices with
    room for ``[rows, compute units]`` each. A head whose kernel has every logit in a register
    anyway may leave each row's best (value, lowest index) per workgroup there, as
    ``[rows, parts]``, and say how many ``parts`` there are; the sampler then skips the kernel that
    reads all logits once more for that. 0 parts: nothing was left."""

    scratch: tuple
    parts: int = 0


class Head(Part):
    """Rows to logits: ``forward(x [k, hidden]) -> float32 [k, vocab]``. ``tie(table)`` gives a
    tied head the embedding's table. The fused decode form, ``forward_stream(stream, norm,
    argmax=None)``, may fill an :class:`ArgmaxStage`."""

    def tie(self, table: torch.Tensor) -> None:
        raise NotImplementedError

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError
