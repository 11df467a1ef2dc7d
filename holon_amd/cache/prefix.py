"""Reuse of cached pages across requests that start with the same tokens. core/holon/core/prefix.py:1-24 (the
hash chain, the tree of entries, eviction of idle leaves), core/holon/core/state.py:180-224, :433-462 (adopt, publish).

A *block* is one page of tokens in every paged group. Block i of a request is keyed by a hash of block i-1's key and
block i's tokens, rooted in a namespace, so a key names the whole prefix up to the block's end; a match also compares
the entry's tokens and parent, so a colliding hash is a miss. The index keeps one reference on every page of every
entry.

A request holds exactly the pages of the chain it follows: the blocks it adopted when admitted, and the blocks it
published since (a block someone else published first replaces the request's own copy). Whoever holds a block
therefore holds every block before it, and an entry whose pages only the index holds has only such entries below it:
they can always be freed, leaves first, least recently used first.
"""
from __future__ import annotations

import collections
import dataclasses
import hashlib

import numpy as np

from .pool import PagePool


@dataclasses.dataclass(eq=False)
class CachedBlock:
    key: bytes
    parent: bytes | None
    tokens: tuple[int, ...]
    pages: tuple[int, ...]                # one page per group
    children: int = 0
    tick: int = 0                         # when it was last matched or stored


class PrefixIndex:
    def __init__(self, namespace: bytes, block: int, pools: list[PagePool]) -> None:
        self.namespace, self.block, self.pools = namespace, block, pools
        self.entries: collections.OrderedDict[bytes, CachedBlock] = collections.OrderedDict()   # least recent first
        self._tick = 0
        self.hits = self.evictions = 0

    def key(self, prev: bytes | None, tokens) -> bytes:
        h = hashlib.blake2b(self.namespace if prev is None else prev, digest_size=16)
        h.update(np.asarray(tokens, dtype=np.int64).tobytes())
        return h.digest()

    def _touch(self, e: CachedBlock) -> None:
        self._tick += 1
        e.tick = self._tick
        self.entries.move_to_end(e.key)

    def match(self, tokens: list[int], max_blocks: int) -> list[CachedBlock]:
        """The cached blocks that `tokens` starts with, at most `max_blocks` of them."""
        out: list[CachedBlock] = []
        prev = None
        for i in range(max_blocks):
            mine = tuple(tokens[i * self.block: (i + 1) * self.block])
            e = self.entries.get(self.key(prev, mine))
            if e is None or e.parent != prev or e.tokens != mine:
                break
            out.append(e)
            prev = e.key
        for e in out:
            self._touch(e)
        self.hits += len(out)
        return out

    def get(self, key: bytes) -> CachedBlock | None:
        return self.entries.get(key)

    def store(self, key: bytes, parent: bytes | None, tokens: tuple[int, ...], pages: tuple[int, ...]) -> CachedBlock:
        """A new entry over pages that its publisher holds; the index takes a reference of its own on each."""
        for pool, page in zip(self.pools, pages):
            pool.incref(page)
        e = CachedBlock(key, parent, tokens, pages)
        self.entries[key] = e
        if parent is not None:
            self.entries[parent].children += 1
        self._touch(e)
        return e

    def touch(self, e: CachedBlock) -> None:
        self._touch(e)

    # -- eviction -------------------------------------------------------------------------------------------------
    def _idle(self, e: CachedBlock) -> bool:
        """Only the index holds it (the groups' pages of a block are taken and given back together)."""
        return self.pools[0].refs(e.pages[0]) == 1

    def idle_pages(self) -> int:
        """Pages per group that only the index holds: what eviction can free."""
        return sum(1 for e in self.entries.values() if self._idle(e))

    def is_cached(self, gid: int) -> set[int]:
        return {e.pages[gid] for e in self.entries.values()}

    def _drop(self, e: CachedBlock) -> None:
        del self.entries[e.key]
        if e.parent is not None:
            self.entries[e.parent].children -= 1
        for pool, page in zip(self.pools, e.pages):
            pool.decref(page)
        self.evictions += 1

    def evict(self, blocks: int) -> int:
        """Free up to `blocks` idle entries, least recently used leaves first; an entry whose last child goes becomes
        a leaf and goes with it when it is older than what the scan has reached. Returns how many went."""
        victims: list[CachedBlock] = []
        taken: set[bytes] = set()
        fewer: dict[bytes, int] = {}                  # children that go, by parent
        for e in self.entries.values():
            if len(victims) >= blocks:
                break
            reached = e.tick
            while (e is not None and len(victims) < blocks and e.key not in taken
                   and e.children == fewer.get(e.key, 0) and self._idle(e)):
                victims.append(e)
                taken.add(e.key)
                parent = self.entries[e.parent] if e.parent is not None else None
                if parent is not None:
                    fewer[parent.key] = fewer.get(parent.key, 0) + 1
                e = parent if parent is not None and parent.tick <= reached else None
        for e in victims:
            self._drop(e)
        return len(victims)

    def flush(self) -> None:
        """Forget everything; requests keep the pages they hold."""
        for e in list(self.entries.values()):
            for pool, page in zip(self.pools, e.pages):
                pool.decref(page)
        self.entries.clear()
