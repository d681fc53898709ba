"""The cache: page and slot bookkeeping (:mod:`.manager`) and device memory (:mod:`.store`)."""

from .manager import (
    RELEASED, Allocation, CacheManager, CacheStats, CopyOp, GroupSpec, NoFreePagesError, SequenceError,
    WrongThreadError,
)
from .page_identity import ROOT_PARENT, chain_hashes, page_hash
from .reclaim import OldestFirst, ReclaimOrder, ReusedLast, make_order
from .state_slots import NoFreeSlotError, StateSlots

__all__ = [
    "RELEASED", "Allocation", "CacheManager", "CacheStats", "CopyOp", "GroupSpec",
    "NoFreePagesError", "NoFreeSlotError", "OldestFirst", "ROOT_PARENT", "ReclaimOrder", "ReusedLast",
    "SequenceError", "StateSlots", "WrongThreadError", "chain_hashes", "make_order", "page_hash",
]
