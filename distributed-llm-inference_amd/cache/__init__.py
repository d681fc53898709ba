"""The cache: page and slot bookkeeping (:mod:`.manager`) and device memory (:mod:`.store`)."""

from .manager import (
    RELEASED, Allocation, CacheManager, CacheStats, CopyOp, GroupSpec, NoFreePagesError, SequenceError,
)
from .page_identity import ROOT_PARENT, chain_hashes, page_hash
from .reclaim import CostAwarePolicy, LRUPolicy, make_policy
from .state_slots import NoFreeSlotError, StateSlots

__all__ = [
    "RELEASED", "Allocation", "CacheManager", "CacheStats", "CopyOp", "CostAwarePolicy", "GroupSpec",
    "LRUPolicy", "NoFreePagesError", "NoFreeSlotError", "ROOT_PARENT", "SequenceError", "StateSlots",
    "chain_hashes", "make_policy", "page_hash",
]
