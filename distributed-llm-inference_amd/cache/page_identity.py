"""Content identities of full cache pages, as a hash chain over the token prefix.

What a page holds depends on every token before it, so a page's identity chains its parent's:
``h_i = SHA256(u32le(len(ns)) || ns || h_{i-1} || int64le(tokens of page i))`` with 32 zero bytes
as the root's parent (reference: src/dli/kv/hashing.py:29-61). Two pages with equal identities hold
equal keys and values and may be shared. The namespace is length-prefixed so that ``b"ab"`` with
some tokens can never alias ``b"a"`` with others; tokens are 64-bit so no vocabulary truncates.
"""

from __future__ import annotations

import hashlib
import struct
from typing import Sequence

PageHash = bytes
ROOT_PARENT: PageHash = bytes(32)


def page_hash(namespace: bytes, parent: PageHash, tokens: Sequence[int]) -> PageHash:
    h = hashlib.sha256()
    h.update(struct.pack("<I", len(namespace)))
    h.update(namespace)
    h.update(parent)
    h.update(struct.pack(f"<{len(tokens)}q", *tokens))
    return h.digest()


def chain_hashes(namespace: bytes, tokens: Sequence[int], page_size: int,
                 parent: PageHash = ROOT_PARENT) -> list[PageHash]:
    """Identities of every *full* page of ``tokens``; a partial last page has none."""
    out: list[PageHash] = []
    for start in range(0, len(tokens) - page_size + 1, page_size):
        parent = page_hash(namespace, parent, tokens[start:start + page_size])
        out.append(parent)
    return out
