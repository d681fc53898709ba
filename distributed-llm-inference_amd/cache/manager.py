"""The cache manager: pages of keys and values with a block table per request, in groups.

Device memory for keys and values is cut into pages of ``page_size`` token slots. Layers whose
needs differ form *groups* (:class:`GroupSpec`): a ``full`` group keeps every key of a request; a
``window`` group only ever reads the last ``window`` keys, so pages that the window has passed are
given back while the request still runs. Each group has pages of its own and each request one block
table per group. Beside the pages, every request holds one *state slot* from admission to its end
(:mod:`.state_slots`). This module is metadata only: it never touches a tensor.

The behaviour follows the reference's block manager (src/dli/kv/block_manager.py): pages are taken
one at a time as a request grows; a request's full, computed pages are entered into a content index
(hash chain over the token prefix) and stay reusable after the request ends, until memory is needed
(leaves first); a page shared with a fork is copied before it is written (copy-on-write); an
operation that cannot get its pages raises :class:`NoFreePagesError` before it changes anything.

Content reuse needs the cached pages to be a pure function of the token prefix in *every* group,
and the request to have no other per-request state: it is off for a ``stateful`` model. Every
group keeps a content index of its own, under the same identities (the hash chain over the token
prefix). A prompt's leading pages are served from the indexes only as far as *all* groups can
serve them: a ``full`` group must hold every page of the run, a ``window`` group the pages that the
first computed token's window still reaches (the pages before those start out as released, as
they would be had the request computed the run itself).

Rules of the content index (each prevents a concrete fault; block_manager.py:17-29):
only full pages are entered; only after their keys have been computed; a prompt is never served
wholly from the index (the page with its last token is always computed, since a step must run at
least one token to give logits); in a full group a page is entered only under its own request's
cached parent, and only leaves are reclaimed, so every cached page is reachable from the root (a
window group gives its oldest pages back first, so there a page stands by itself: no parent, any
idle one may be reclaimed, and a lookup asks for each page it needs by name); shared pages are
never written.
"""

from __future__ import annotations

import functools
import threading
from collections import Counter
from dataclasses import dataclass, field
from typing import Hashable, Optional, Sequence

from .page_identity import ROOT_PARENT, PageHash, chain_hashes, page_hash
from .pool import PagePool
from .reclaim import ReclaimOrder
from .state_slots import NoFreeSlotError, StateSlots

SeqId = Hashable
RELEASED = -1  # block-table entry of a page that a window has passed


class NoFreePagesError(RuntimeError):
    """Not enough free or reclaimable pages; nothing was changed."""


class SequenceError(KeyError):
    """Unknown or duplicate request id."""

    def __str__(self) -> str:  # KeyError would print the message's repr, quotes and all
        return str(self.args[0]) if self.args else ""


class WrongThreadError(RuntimeError):
    """A manager that is confined to one thread was changed from another."""


def _confined(method):
    """The manager has no lock: one thread (the engine's loop) makes every change. With
    ``confine_to_thread`` a change from any other thread fails at once instead of corrupting the
    tables some steps later (the reference's block manager checks the same:
    src/dli/kv/block_manager.py:447-449)."""

    @functools.wraps(method)
    def checked(self, *args, **kwargs):
        home = self._home_thread
        if home is not None and threading.get_ident() != home:
            raise WrongThreadError(
                f"CacheManager.{method.__name__} called from thread {threading.get_ident()}, but the manager "
                f"belongs to thread {home} (hand it over with adopt())")
        return method(self, *args, **kwargs)

    return checked


@dataclass(frozen=True)
class GroupSpec:
    """Needs of one group of layers: ``kind`` is ``"full"`` or ``"window"`` (then ``window`` > 0)."""

    kind: str = "full"
    window: int = 0

    def __post_init__(self) -> None:
        if self.kind not in ("full", "window"):
            raise ValueError(f"unknown cache group kind {self.kind!r}")
        if (self.kind == "window") != (self.window > 0):
            raise ValueError("a window group needs window > 0, a full group window == 0")


@dataclass(frozen=True)
class CopyOp:
    """Copy page ``src`` onto page ``dst`` of ``group`` (all its layers) before the next step."""

    src: int
    dst: int
    group: int = 0


@dataclass(frozen=True)
class Allocation:
    """Result of admitting a prompt: its block tables (one per group), how many leading tokens
    already have their keys cached, and its state slot."""

    block_tables: tuple[tuple[int, ...], ...]
    num_cached_tokens: int
    state_slot: int

    @property
    def block_table(self) -> tuple[int, ...]:
        return self.block_tables[0]


@dataclass
class CacheStats:
    num_pages: int = 0
    free_pages: int = 0
    cached_idle_pages: int = 0
    used_pages: int = 0
    prompt_tokens_queried: int = 0
    prompt_tokens_hit: int = 0
    evictions: int = 0
    cow_copies: int = 0
    duplicate_registrations: int = 0
    window_pages_released: int = 0

    @property
    def hit_rate(self) -> float:
        return self.prompt_tokens_hit / self.prompt_tokens_queried if self.prompt_tokens_queried else 0.0


@dataclass
class _Seq:
    tables: list[list[int]]
    num_tokens: int
    num_computed: int
    namespace: bytes
    state_slot: int
    released: list[int]  # per group: leading pages that a window has passed
    page_hashes: list[PageHash] = field(default_factory=list)
    tail_tokens: list[int] = field(default_factory=list)
    num_registered: int = 0
    reserved: int = 0  # tokens that the tables have room for, where that exceeds num_tokens


@dataclass
class _Hits:
    """What the content indexes hold of a prompt: ``pages`` leading pages need no computing;
    group g's table starts with ``first[g]`` released entries, then the cached pages ``found[g]``."""

    pages: int
    first: list[int]
    found: list[list[int]]


class CacheManager:
    """Hands out pages and state slots to requests and keeps the content indexes.

    Args:
        groups: one :class:`GroupSpec` per group of layers (the dense Llama decoder has one).
        num_pages: pages per group (one number for all, or one per group).
        page_size: token slots per page.
        max_seqs: number of state slots, i.e. the most requests that hold cache at once.
        stateful: the model keeps per-request state outside the pages (disables content reuse).
        enable_prefix_caching: content reuse, in all groups or in none.
        watermark: fraction of each group's pages kept back when *admitting* prompts, so running
            requests can still grow (block_manager.py:138-139).
        confine_to_thread: every call that changes the manager must come from the thread that
            made it (or that last called :meth:`adopt`); any other raises :class:`WrongThreadError`.
    """

    def __init__(
        self,
        groups: Sequence[GroupSpec] = (GroupSpec(),),
        *,
        num_pages: int | Sequence[int],
        page_size: int,
        max_seqs: int = 256,
        eviction_policy: str | ReclaimOrder = "lru",
        enable_prefix_caching: bool = True,
        stateful: bool = False,
        watermark: float = 0.01,
        confine_to_thread: bool = False,
    ) -> None:
        self._home_thread: Optional[int] = threading.get_ident() if confine_to_thread else None
        if page_size <= 0:
            raise ValueError("page_size must be positive")
        if not groups:
            raise ValueError("at least one cache group is needed")
        if not 0.0 <= watermark < 1.0:
            raise ValueError("watermark must be in [0, 1)")
        self.groups = tuple(groups)
        counts = [num_pages] * len(self.groups) if isinstance(num_pages, int) else list(num_pages)
        if len(counts) != len(self.groups) or any(c <= 0 for c in counts):
            raise ValueError("num_pages must be positive, one number or one per group")
        self.page_size = page_size
        # a policy given by name is made once per group; an order handed in serves the first group
        self.pools = [PagePool(c, eviction_policy if i == 0 or isinstance(eviction_policy, str) else "lru")
                      for i, c in enumerate(counts)]
        self.slots = StateSlots(max_seqs)
        self.prefix_caching = bool(enable_prefix_caching and not stateful)
        self._reserve = [int(watermark * c) for c in counts]
        self._seqs: dict[SeqId, _Seq] = {}
        self._stats = CacheStats()

    def adopt(self) -> None:
        """The calling thread becomes the one that may change a confined manager."""
        if self._home_thread is not None:
            self._home_thread = threading.get_ident()

    # ------------------------------------------------------------------ queries

    @property
    def num_pages(self) -> int:
        """Pages of the smallest group: what bounds the longest request."""
        return min(p.num_pages for p in self.pools)

    @property
    def num_available_pages(self) -> int:
        return min(p.num_available for p in self.pools)

    @property
    def num_groups(self) -> int:
        return len(self.groups)

    def has_sequence(self, seq_id: SeqId) -> bool:
        return seq_id in self._seqs

    def sequences(self) -> list[SeqId]:
        return list(self._seqs)

    def block_table(self, seq_id: SeqId, group: int = 0) -> tuple[int, ...]:
        """Page ids of the request in ``group``; :data:`RELEASED` where a window has passed."""
        return tuple(self._seq(seq_id).tables[group])

    def table_ref(self, seq_id: SeqId, group: int = 0) -> list[int]:
        """The request's live page list in ``group`` (read only: it changes as the request grows)."""
        return self._seq(seq_id).tables[group]

    def state_slot(self, seq_id: SeqId) -> int:
        return self._seq(seq_id).state_slot

    def num_tokens(self, seq_id: SeqId) -> int:
        return self._seq(seq_id).num_tokens

    def num_computed_tokens(self, seq_id: SeqId) -> int:
        return self._seq(seq_id).num_computed

    def slot_mapping(self, seq_id: SeqId, start: int, end: int, group: int = 0) -> list[int]:
        """Flat cache slot ``page * page_size + offset`` of positions ``[start, end)``."""
        seq = self._seq(seq_id)
        if not 0 <= start <= end <= seq.num_tokens:
            raise ValueError(f"positions [{start}, {end}) outside reserved [0, {seq.num_tokens})")
        ps, table = self.page_size, seq.tables[group]
        out = []
        for p in range(start, end):
            page = table[p // ps]
            if page == RELEASED:
                raise ValueError(f"position {p} lies in a page that the window has passed")
            out.append(page * ps + p % ps)
        return out

    def pages_needed_for_prompt(self, token_ids: Sequence[int], namespace: bytes = b"") -> int:
        hits, _ = self._lookup(token_ids, namespace)
        return self._ceil(len(token_ids)) - hits.pages

    def can_allocate(self, token_ids: Sequence[int], namespace: bytes = b"") -> bool:
        """Whether :meth:`allocate` would succeed with the watermark respected."""
        if self.slots.num_free == 0:
            return False
        hits, _ = self._lookup(token_ids, namespace)
        return self._admissible(len(token_ids), hits, respect_watermark=True)

    def stats(self) -> CacheStats:
        s = self._stats
        free = sum(len(p.free) for p in self.pools)
        idle = sum(p.num_idle for p in self.pools)
        total = sum(p.num_pages for p in self.pools)
        return CacheStats(
            num_pages=total, free_pages=free, cached_idle_pages=idle, used_pages=total - free - idle,
            prompt_tokens_queried=s.prompt_tokens_queried, prompt_tokens_hit=s.prompt_tokens_hit,
            evictions=sum(p.evictions for p in self.pools), cow_copies=s.cow_copies,
            duplicate_registrations=s.duplicate_registrations,
            window_pages_released=s.window_pages_released,
        )

    # ------------------------------------------------------------------ lifecycle

    @_confined
    def allocate(self, seq_id: SeqId, token_ids: Sequence[int], *, namespace: bytes = b"",
                 respect_watermark: bool = True) -> Allocation:
        """Admit a prompt: reuse cached leading pages, take the rest, take a state slot
        (reference: src/dli/kv/block_manager.py:238-284, there for one group and no slots).

        Raises:
            SequenceError: the id is live already.
            NoFreePagesError / NoFreeSlotError: not enough pages or slots (nothing changed).
            ValueError: empty prompt.
        """
        n = len(token_ids)
        if n == 0:
            raise ValueError(f"request {seq_id!r} brings an empty prompt")
        if seq_id in self._seqs:
            raise SequenceError(f"request {seq_id!r} holds cache already")
        if self.slots.num_free == 0:
            raise NoFreeSlotError(f"all {self.slots.num_slots} state slots are taken")
        hits, hashes = self._lookup(token_ids, namespace)
        pages = self._ceil(n)
        if not self._admissible(n, hits, respect_watermark=respect_watermark):
            raise NoFreePagesError(
                f"request {seq_id!r} needs {pages - hits.pages} more pages for its {n} tokens; "
                f"{self.num_available_pages} can be had ({max(self._reserve)} kept back)")
        # Everything below succeeds: the checks above have counted the pages.
        tables = [self._fill_table(pool, hits.first[g], hits.found[g], pages) for g, pool in enumerate(self.pools)]
        seq = _Seq(tables=tables, num_tokens=n, num_computed=hits.pages * self.page_size, namespace=namespace,
                   state_slot=self.slots.take(), released=list(hits.first))
        if self.prefix_caching:
            seq.page_hashes, seq.num_registered = hashes, hits.pages
            seq.tail_tokens = list(token_ids[len(hashes) * self.page_size:])
        self._stats.prompt_tokens_queried += n
        self._stats.prompt_tokens_hit += seq.num_computed
        self._seqs[seq_id] = seq
        return Allocation(tuple(map(tuple, tables)), seq.num_computed, seq.state_slot)

    @staticmethod
    def _fill_table(pool: PagePool, first: int, hits: Sequence[int], pages: int) -> list[int]:
        """A new request's table in one group: ``first`` entries for pages that the window has
        passed already, the cached pages that its prompt matched, then fresh ones up to ``pages``.
        The matched pages are taken hold of first, so that none of them can be reclaimed to make
        room for the fresh ones."""
        for page in hits:
            pool.incref(page)
            pool.order.found(page)
        return [*([RELEASED] * first), *hits, *(pool.take() for _ in range(pages - first - len(hits)))]

    @_confined
    def append_slots(self, seq_id: SeqId, token_ids: Sequence[int]) -> list[CopyOp]:
        """Reserve slots for tokens appended to the request; returns the page copies that must be
        done on the device before the next write (copy-on-write of a shared partial page)."""
        seq = self._seq(seq_id)
        ps, pos, n = self.page_size, seq.num_tokens, len(token_ids)
        have = self._ceil(max(seq.num_tokens, seq.reserved))  # pages in place, some reserved ahead
        needed = max(0, self._ceil(pos + n) - have)
        cows = []
        for g, pool in enumerate(self.pools):
            # the partly filled page that the first new token goes into (pages behind it may be
            # reserved ahead: those are never shared)
            last = seq.tables[g][pos // ps] if pos % ps != 0 else RELEASED
            cow = last != RELEASED and pool.ref[last] > 1
            cows.append(cow)
            if needed + cow > pool.num_available:
                raise NoFreePagesError(f"append needs {needed + cow} pages in group {g}")
        ops: list[CopyOp] = []
        for g, pool in enumerate(self.pools):
            table = seq.tables[g]
            if cows[g]:
                old = table[pos // ps]
                new = pool.take()
                ops.append(CopyOp(src=old, dst=new, group=g))
                table[pos // ps] = new
                pool.decref(old)
                self._stats.cow_copies += 1
            for _ in range(needed):
                table.append(pool.take())
        seq.num_tokens += n
        if seq.reserved <= seq.num_tokens:
            seq.reserved = 0
        if self.prefix_caching:
            seq.tail_tokens.extend(token_ids)
        return ops

    @_confined
    def reserve_ahead(self, seq_id: SeqId, extra_tokens: int) -> None:
        """Make room for ``extra_tokens`` more tokens than the request has, without naming them:
        the pages they will need are taken now, :meth:`append_slots` uses them later. For steps
        that decode several tokens on the device before the host sees any of them.

        Raises:
            NoFreePagesError: not enough pages (nothing changed).
        """
        seq = self._seq(seq_id)
        if extra_tokens <= 0:
            return
        target = seq.num_tokens + extra_tokens
        have = self._ceil(max(seq.num_tokens, seq.reserved))
        needed = self._ceil(target) - have
        if needed > 0:
            for g, pool in enumerate(self.pools):
                if needed > pool.num_available:
                    raise NoFreePagesError(f"reserving ahead needs {needed} pages in group {g}")
            for g, pool in enumerate(self.pools):
                for _ in range(needed):
                    seq.tables[g].append(pool.take())
        seq.reserved = max(seq.reserved, target)

    @_confined
    def mark_computed(self, seq_id: SeqId, num_computed_tokens: int) -> None:
        """Record that the keys of the first ``num_computed_tokens`` tokens are written.

        Newly full pages enter the content index; pages that a window has passed are given back.
        """
        seq = self._seq(seq_id)
        if not seq.num_computed <= num_computed_tokens <= seq.num_tokens:
            raise ValueError(
                f"computed must be in [{seq.num_computed}, {seq.num_tokens}], got {num_computed_tokens}")
        seq.num_computed = num_computed_tokens
        if self.prefix_caching:
            self._register_full_pages(seq)
        for g, spec in enumerate(self.groups):
            if spec.kind == "window":
                self._release_passed(seq, g, spec.window)

    @_confined
    def fork(self, parent_id: SeqId, child_id: SeqId) -> int:
        """Create ``child_id`` sharing every page of the parent; returns the child's state slot
        (copying the parent's state into it is the caller's business)."""
        parent = self._seq(parent_id)
        if child_id in self._seqs:
            raise SequenceError(f"sequence {child_id!r} already allocated")
        slot = self.slots.take()
        held = self._ceil(parent.num_tokens)  # pages reserved ahead stay the parent's alone
        for g, pool in enumerate(self.pools):
            for page in parent.tables[g][:held]:
                if page != RELEASED:
                    pool.incref(page)
        self._seqs[child_id] = _Seq(
            tables=[list(t[:held]) for t in parent.tables], num_tokens=parent.num_tokens,
            num_computed=parent.num_computed, namespace=parent.namespace, state_slot=slot,
            released=list(parent.released), page_hashes=list(parent.page_hashes),
            tail_tokens=list(parent.tail_tokens), num_registered=parent.num_registered)
        return slot

    @_confined
    def free(self, seq_id: SeqId) -> None:
        """Give back everything a finished, aborted or preempted request holds. Cached pages stay
        revivable; the others return to the free list."""
        seq = self._seqs.pop(seq_id, None)
        if seq is None:
            raise SequenceError(f"unknown sequence {seq_id!r}")
        for g, pool in enumerate(self.pools):
            for page in reversed(seq.tables[g]):  # deepest first, as leaves are reclaimed first
                if page != RELEASED:
                    pool.decref(page)
        self.slots.give_back(seq.state_slot)

    @_confined
    def reset_prefix_cache(self) -> int:
        """Reclaim every idle cached page; returns how many."""
        return sum(p.evict_all_idle() for p in self.pools)

    # ------------------------------------------------------------------ verification

    def check_invariants(self) -> None:
        """Verify that no page or slot is lost, held twice or freed twice (AssertionError if so)."""
        for g, pool in enumerate(self.pools):
            expected: Counter = Counter()
            for seq in self._seqs.values():
                table = seq.tables[g]
                assert len(table) == self._ceil(max(seq.num_tokens, seq.reserved)), "table size != ceil(tokens/page)"
                assert 0 <= seq.num_computed <= seq.num_tokens, "computed outside [0, tokens]"
                assert all(p == RELEASED for p in table[:seq.released[g]]), "released prefix holds a page"
                assert all(p != RELEASED for p in table[seq.released[g]:]), "a live page is missing"
                expected.update(p for p in table if p != RELEASED)
            pool.check(expected)
        self.slots.check([s.state_slot for s in self._seqs.values()])

    # ------------------------------------------------------------------ internals

    def _ceil(self, n: int) -> int:
        return -(-n // self.page_size)

    def _seq(self, seq_id: SeqId) -> _Seq:
        try:
            return self._seqs[seq_id]
        except KeyError:
            raise SequenceError(f"unknown sequence {seq_id!r}") from None

    def _first_needed_page(self, g: int, computed_pages: int) -> int:
        """The first page of group ``g`` that a request with ``computed_pages`` full pages computed
        still reads: its next query sits at the first position after them."""
        spec = self.groups[g]
        if spec.kind != "window":
            return 0
        return max(0, computed_pages * self.page_size - spec.window + 1) // self.page_size

    def _lookup(self, token_ids: Sequence[int], namespace: bytes) -> tuple[_Hits, list[PageHash]]:
        """The longest run of leading full pages that every group can serve from its index,
        never the page with the last token."""
        none = _Hits(0, [0] * len(self.pools), [[] for _ in self.pools])
        if not self.prefix_caching:
            return none, []
        eligible = (len(token_ids) - 1) // self.page_size * self.page_size
        hashes = chain_hashes(namespace, token_ids[:eligible], self.page_size)
        run = len(hashes)   # full groups: the run ends at the first page that one of them lacks
        for g, pool in enumerate(self.pools):
            if self.groups[g].kind == "full":
                run = next((i for i, h in enumerate(hashes[:run]) if h not in pool.by_identity), run)
        while run > 0:      # window groups: the pages that the window at the run's end reaches
            short = False
            for g, pool in enumerate(self.pools):
                if self.groups[g].kind == "window":
                    short = short or any(hashes[i] not in pool.by_identity
                                         for i in range(self._first_needed_page(g, run), run))
            if not short:
                break
            run -= 1
        if run == 0:
            return none, hashes
        first = [self._first_needed_page(g, run) for g in range(len(self.pools))]
        found = [[pool.by_identity[h] for h in hashes[first[g]:run]] for g, pool in enumerate(self.pools)]
        return _Hits(run, first, found), hashes

    def _admissible(self, n_tokens: int, hits: _Hits, *, respect_watermark: bool) -> bool:
        fresh = self._ceil(n_tokens) - hits.pages
        for g, pool in enumerate(self.pools):
            reserve = self._reserve[g] if respect_watermark else 0
            revived = sum(1 for p in hits.found[g] if pool.ref[p] == 0)  # idle hits stop being reclaimable
            if pool.num_available - revived - fresh < reserve:
                return False
        return True

    def _register_full_pages(self, seq: _Seq) -> None:
        ps = self.page_size
        full_computed = seq.num_computed // ps
        while seq.num_registered < full_computed:
            i = seq.num_registered
            while len(seq.page_hashes) <= i:  # identities of newly completed pages, from the tail
                parent_hash = seq.page_hashes[-1] if seq.page_hashes else ROOT_PARENT
                seq.page_hashes.append(page_hash(seq.namespace, parent_hash, seq.tail_tokens[:ps]))
                del seq.tail_tokens[:ps]
            for g, pool in enumerate(self.pools):
                table = seq.tables[g]
                if table[i] == RELEASED:
                    continue
                chained = self.groups[g].kind == "full" and i > 0
                outcome = pool.register(table[i], seq.page_hashes[i], seq.page_hashes[i - 1] if chained else None,
                                        table[i - 1] if chained else None, i)
                if outcome == "duplicate":
                    self._stats.duplicate_registrations += 1
            seq.num_registered += 1

    def _release_passed(self, seq: _Seq, g: int, window: int) -> None:
        # The next query sits at position num_computed or later and sees keys
        # j >= position - window + 1; a page whose last key lies before that is never read again.
        first_needed = seq.num_computed - window + 1
        table, pool = seq.tables[g], self.pools[g]
        while seq.released[g] < len(table) and (seq.released[g] + 1) * self.page_size <= first_needed:
            page = table[seq.released[g]]
            table[seq.released[g]] = RELEASED
            pool.decref(page)
            seq.released[g] += 1
            self._stats.window_pages_released += 1
