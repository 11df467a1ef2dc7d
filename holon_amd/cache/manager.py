"""The cache manager: slots, paged groups with block tables, and fixed-size per-request state.

A request is given a *slot* when it is admitted: its row in every block table and in every fixed-size state tensor.
State that grows lives in pages. Paged states of equal page geometry (values per token, window, dtype), whichever runs
declare them and however many one run declares, form a *group*: one page pool, one block table, one storage tensor
`[members, pages, page_size * elems]` with a member for every (run, state name) of the group. Page id p means row p
of every member. Groups with different needs (all tokens, a window of them, another width) have pools and tables of
their own; a windowed group gives pages back as soon as the window has passed them, a finished request gives back
everything.

With a prefix index (`enable_prefix`) full pages of tokens are shared between requests that start alike: `adopt` gives
a new request the cached pages of its longest known prefix, `publish` hands the pages a request has filled to the
index, and `reserve` evicts cached pages nobody uses when the pool runs short.

core/holon/core/state.py:124-554 (`StateManager`: admit/reserve/release, `BlockTable`), core/holon/core/assembly.py:
140-189 (grouping by declaration), std/holon_std/state/paged/kind.py:10-19 (pages needed).
"""
from __future__ import annotations

import dataclasses

import numpy as np
import torch

from ..parts.base import PagedState, SlotState
from ..model import SitePages
from .pool import PagePool
from .prefix import PrefixIndex


@dataclasses.dataclass
class PagedGroup:
    gid: int
    decl: PagedState                              # with name ignored: elems, window, dtype decide the group
    sites: list[int]                              # the runs with a state in this group (a run once)
    members: list[tuple[int, str]]                # (run, state name) of every row of `storage`
    pool: PagePool
    storage: torch.Tensor                         # [len(members), num_pages, page_size * elems]
    table: np.ndarray                             # [max_seqs + 1, max_pages] int32, null page where nothing is held
    table_dev: torch.Tensor
    first: list[int]                              # per slot: first page index still held
    count: list[int]                              # per slot: page indices [first, count) are held
    dirty: set[int] = dataclasses.field(default_factory=set)


class CacheManager:
    """`sites`: the model's run entries (`holon_amd.model.Site`), filled here with their storage; `decls[i]`: what
    run i keeps. `tokens`: capacity of every paged pool, in tokens."""

    def __init__(self, sites: list, decls: list[list[PagedState | SlotState]], *, page_size: int, max_seqs: int,
                 max_model_len: int, tokens: int, device: torch.device, dtype: torch.dtype) -> None:
        self.page_size, self.max_seqs, self.max_model_len = page_size, max_seqs, max_model_len
        self.device, self.dtype = device, dtype
        self.max_pages = -(-max_model_len // page_size)
        self.padding_slot = max_seqs                              # a row of null pages, for rows that compute nothing
        self.groups: list[PagedGroup] = []
        self.slot_states: list[tuple[int, SlotState, torch.Tensor]] = []
        self._free_slots = list(range(max_seqs - 1, -1, -1))
        self._live: set[int] = set()
        self.computed = [0] * (max_seqs + 1)
        self._capacity = [0] * (max_seqs + 1)          # tokens each slot's pages hold (kept beside the groups' counts)
        self.prefix: PrefixIndex | None = None
        self.chain: list[list[bytes] | None] = [None] * (max_seqs + 1)   # per slot: keys of the blocks it follows
        self.tokens_saved = 0
        num_pages = -(-tokens // page_size) + 1
        if tokens < 1:
            raise ValueError("the cache needs room for at least one token")
        keyed: dict[tuple, list[tuple[int, str]]] = {}
        for site, site_decls in zip(sites, decls, strict=True):
            names = [d.name for d in site_decls]
            if len(set(names)) != len(names):
                raise ValueError(f"run {site.run} declares two states of one name: {names}")
            for d in site_decls:
                if isinstance(d, PagedState):
                    key = (d.elems, d.window, d.dtype or dtype)
                    keyed.setdefault(key, []).append((site.run, d.name))
                elif isinstance(d, SlotState):
                    t = torch.zeros((max_seqs + 1, *d.shape), dtype=d.dtype or dtype, device=device)
                    site.slot_state[d.name] = t
                    self.slot_states.append((site.run, d, t))
                else:
                    raise TypeError(f"run {site.run}: unknown state declaration {d!r}")
        for gid, ((elems, window, gdtype), members) in enumerate(keyed.items()):
            pool = PagePool(num_pages)
            storage = torch.zeros((len(members), num_pages, page_size * elems), dtype=gdtype, device=device)
            table = np.full((max_seqs + 1, self.max_pages), pool.null, dtype=np.int32)
            runs = sorted({run for run, _ in members})
            group = PagedGroup(gid, PagedState("", elems, window, gdtype), runs, members, pool, storage, table,
                               torch.from_numpy(table.copy()).to(device), [0] * (max_seqs + 1), [0] * (max_seqs + 1))
            self.groups.append(group)
            for at, (run, name) in enumerate(members):
                sites[run].paged[name] = SitePages(gid, storage[at])
        for site, site_decls in zip(sites, decls):                # `group`, `pages`: the first paged state declared
            first = next((d.name for d in site_decls if isinstance(d, PagedState)), None)
            if first is not None:
                site.group, site.pages = site.paged[first].group, site.paged[first].pages
        for site in sites:                                        # runs that read another run's cache
            if site.owner is not None:
                owner = sites[site.owner]
                site.group, site.pages, site.paged, site.slot_state = owner.group, owner.pages, owner.paged, \
                    owner.slot_state

    # -- slots ----------------------------------------------------------------------------------------------------
    @property
    def free_slots(self) -> int:
        return len(self._free_slots)

    def admit(self) -> int | None:
        """A slot for a new request (its fixed-size state zeroed), or None when all are taken."""
        if not self._free_slots:
            return None
        slot = self._free_slots.pop()
        self._live.add(slot)
        self.computed[slot] = 0
        self.chain[slot] = [] if self.prefix is not None else None
        for _, _, t in self.slot_states:
            t[slot].zero_()
        return slot

    def release(self, slot: int) -> None:
        """Give back everything the request holds."""
        if slot not in self._live:
            raise RuntimeError(f"slot {slot} released twice (or never admitted)")
        for g in self.groups:
            for i in range(g.first[slot], g.count[slot]):
                g.pool.decref(int(g.table[slot, i]))
            g.table[slot, : g.count[slot]] = g.pool.null
            g.first[slot] = g.count[slot] = 0
            g.dirty.add(slot)
        self._live.remove(slot)
        self.computed[slot] = self._capacity[slot] = 0
        self.chain[slot] = None
        self._free_slots.append(slot)

    # -- shared prefixes ------------------------------------------------------------------------------------------
    def enable_prefix(self, namespace: bytes) -> bool:
        """Share full pages between requests that start with the same tokens. Only state that a page holds whole can
        be shared: with a windowed group (whose early pages go) or fixed-size state (which no page restores) nothing
        is, and this returns False."""
        if self._live:
            raise RuntimeError("the prefix index is set up before requests are admitted")
        if not self.groups or self.slot_states or any(g.decl.window > 0 for g in self.groups):
            return False
        self.prefix = PrefixIndex(namespace, self.page_size, [g.pool for g in self.groups])
        return True

    def adopt(self, slot: int, tokens: list[int]) -> int:
        """Give a freshly admitted request the cached pages of the longest prefix of `tokens` that the index knows,
        always leaving one token to compute. Returns the tokens it now holds (core/holon/core/state.py:180-224)."""
        if self.prefix is None:
            return 0
        if self.computed[slot] or any(g.count[slot] for g in self.groups):
            raise RuntimeError(f"slot {slot} already holds tokens")
        blocks = self.prefix.match(tokens, (len(tokens) - 1) // self.page_size)
        for gid, g in enumerate(self.groups):
            for i, e in enumerate(blocks):
                g.pool.incref(e.pages[gid])
                g.table[slot, i] = e.pages[gid]
            g.count[slot] = len(blocks)
            g.dirty.add(slot)
        self.chain[slot] = [e.key for e in blocks]
        self.computed[slot] = self._capacity[slot] = len(blocks) * self.page_size
        self.tokens_saved += self.computed[slot]
        return self.computed[slot]

    def publish(self, slot: int, tokens: list[int]) -> None:
        """Hand the pages that the request has filled since the last call to the index. Where another request stored
        the same block first, the request takes that page for its own copy, which is given back
        (core/holon/core/state.py:433-462)."""
        chain = self.chain[slot]
        if self.prefix is None or chain is None:
            return
        P, idx = self.page_size, self.prefix
        for i in range(len(chain), min(self.computed[slot], len(tokens)) // P):
            prev = chain[-1] if chain else None
            block = tuple(tokens[i * P: (i + 1) * P])
            key = idx.key(prev, block)
            mine = tuple(int(g.table[slot, i]) for g in self.groups)
            e = idx.get(key)
            if e is None:
                idx.store(key, prev, block, mine)
            elif e.parent == prev and e.tokens == block:
                if e.pages != mine:
                    for g, theirs, own in zip(self.groups, e.pages, mine):
                        g.pool.incref(theirs)
                        g.table[slot, i] = theirs
                        g.pool.decref(own)
                        g.dirty.add(slot)
                idx.touch(e)
            else:                                     # two prefixes under one key: this request shares nothing further
                self.chain[slot] = None
                return
            chain.append(key)

    def flush_prefix(self) -> None:
        """Forget every cached block (after the weights changed, say); live requests keep their pages but publish
        nothing further."""
        if self.prefix is not None:
            self.prefix.flush()
            for slot in self._live:
                self.chain[slot] = None

    # -- pages ----------------------------------------------------------------------------------------------------
    def pages_needed(self, slot: int, total: int) -> list[int]:
        """Per group, the pages a request needs beyond what it holds to keep `total` tokens."""
        want = -(-total // self.page_size)
        return [max(0, want - g.count[slot]) for g in self.groups]

    def reserve(self, slot: int, total: int) -> bool:
        """Make room for the request's tokens 0 .. total-1 in every group, or take nothing and return False."""
        if slot not in self._live:
            raise RuntimeError(f"slot {slot} is not admitted")
        if total > self.max_model_len:
            raise ValueError(f"{total} tokens exceed max_model_len {self.max_model_len}")
        need = self.pages_needed(slot, total)
        short = max((n - g.pool.free for n, g in zip(need, self.groups)), default=0)
        if short > 0:                   # cached pages nobody uses make room, a few more than needed at a time
            if self.prefix is None:
                return False
            self.prefix.evict(max(short, self.groups[0].pool.usable // 64))
            if any(n > g.pool.free for n, g in zip(need, self.groups)):
                return False
        for n, g in zip(need, self.groups):
            if n:
                pages = g.pool.alloc(n)
                g.table[slot, g.count[slot]: g.count[slot] + n] = pages
                g.count[slot] += n
                g.dirty.add(slot)
        self._capacity[slot] = min(g.count[slot] for g in self.groups) * self.page_size if self.groups \
            else self.max_model_len
        return True

    def capacity(self, slot: int) -> int:
        """Tokens the request's pages hold (the smallest over groups)."""
        if not self.groups:
            return self.max_model_len
        return self._capacity[slot]

    def advance(self, slot: int, computed: int) -> None:
        """The request now has `computed` tokens in the cache: pages a window has passed are given back."""
        self.computed[slot] = computed
        for g in self.groups:
            w = g.decl.window
            if w <= 0:
                continue
            keep_from = max(0, computed - w + 1) // self.page_size      # the next query reads keys from computed-w+1
            keep_from = min(keep_from, g.count[slot])
            if keep_from > g.first[slot]:
                for i in range(g.first[slot], keep_from):
                    g.pool.decref(int(g.table[slot, i]))
                g.table[slot, g.first[slot]: keep_from] = g.pool.null
                g.first[slot] = keep_from
                g.dirty.add(slot)

    def could_fit(self, slot: int | None, total: int, victims: list[int]) -> bool:
        """Whether releasing the requests in `victims` (slots) would let `slot` (None: a new request) keep `total`
        tokens (core/holon/core/state.py:478-497)."""
        want = -(-total // self.page_size)
        for gid, g in enumerate(self.groups):
            have = g.count[slot] if slot is not None else 0
            if self.prefix is None:
                freed = sum(g.count[v] - g.first[v] for v in victims)
            else:                       # a page comes free when only the index, or nobody, would still hold it
                dropped: dict[int, int] = {}
                for v in victims:
                    for p in g.table[v, g.first[v]: g.count[v]].tolist():
                        dropped[p] = dropped.get(p, 0) + 1
                cached = self.prefix.is_cached(gid)
                freed = sum(1 for p in cached if g.pool.refs(p) - dropped.get(p, 0) == 1)
                freed += sum(1 for p, n in dropped.items() if p not in cached and g.pool.refs(p) == n)
            if want - have > g.pool.free + freed:
                return False
        return True

    def victims_needed(self, slot: int, total: int, order: list[int]) -> int | None:
        """How many of the requests in `order` (slots, the first to give way first) must give back what they hold
        before `slot` can keep `total` tokens: the shortest start of `order` that makes room. None when not even all
        of them would."""
        if not self.could_fit(slot, total, order):
            return None
        lo, hi = 0, len(order)                    # room grows with every request that gives way
        while lo < hi:
            mid = (lo + hi) // 2
            if self.could_fit(slot, total, order[:mid]):
                hi = mid
            else:
                lo = mid + 1
        return lo

    def fits_alone(self, total: int) -> bool:
        """Whether an empty cache holds one request of `total` tokens."""
        return all(-(-total // self.page_size) <= g.pool.usable for g in self.groups)

    # -- per-step views -------------------------------------------------------------------------------------------
    def take_dirty(self) -> list[tuple[PagedGroup, np.ndarray, np.ndarray]]:
        """The block-table rows that changed since the last call, per group: (group, row numbers [n] int32, their new
        contents [n, max_pages] int32). The caller brings them to the device with the step's other inputs and puts
        them into `group.table_dev` (core/holon/core/state.py:51-58, 525-532: dirty rows ride the step's upload)."""
        out = []
        for g in self.groups:
            if g.dirty:
                rows = np.fromiter(sorted(g.dirty), dtype=np.int32, count=len(g.dirty))
                out.append((g, rows, g.table[rows]))
                g.dirty.clear()
        return out

    def upload(self) -> None:
        """Copy the block-table rows that changed to the device, by themselves (for callers outside a step)."""
        for g, rows, contents in self.take_dirty():
            idx = torch.from_numpy(rows.astype(np.int64)).to(self.device)
            g.table_dev.index_copy_(0, idx, torch.from_numpy(contents).to(self.device))

    def write_targets(self, gid: int, slots: np.ndarray, positions: np.ndarray) -> tuple[np.ndarray, np.ndarray]:
        """(page, offset) of each token's position in its request's pages (core/holon/core/state.py:541-554)."""
        g = self.groups[gid]
        return g.table[slots, positions // self.page_size].astype(np.int32), \
            (positions % self.page_size).astype(np.int32)

    # -- accounting -----------------------------------------------------------------------------------------------
    def nbytes(self) -> int:
        total = sum(g.storage.numel() * g.storage.element_size() for g in self.groups)
        return total + sum(t.numel() * t.element_size() for _, _, t in self.slot_states)

    def check(self) -> None:
        """Every page is free or held exactly as often as its count says; no table points at a page it does not hold."""
        for g in self.groups:
            held: dict[int, int] = {}
            for slot in range(self.max_seqs + 1):
                row = g.table[slot]
                inside = row[g.first[slot]: g.count[slot]]
                outside = np.concatenate((row[: g.first[slot]], row[g.count[slot]:]))
                if slot not in self._live and g.count[slot]:
                    raise AssertionError(f"group {g.gid}: free slot {slot} holds pages")
                if (outside != g.pool.null).any() or (inside == g.pool.null).any():
                    raise AssertionError(f"group {g.gid}: slot {slot}'s table does not match what it holds")
                for p in inside.tolist():
                    held[p] = held.get(p, 0) + 1
            if self.prefix is not None:
                for e in self.prefix.entries.values():
                    held[e.pages[g.gid]] = held.get(e.pages[g.gid], 0) + 1
                    if e.parent is not None and e.parent not in self.prefix.entries:
                        raise AssertionError(f"cached block {e.key.hex()} outlived the block before it")
            free = set(g.pool._free)
            if len(free) != len(g.pool._free):
                raise AssertionError(f"group {g.gid}: a page is in the free list twice")
            for p in range(g.pool.usable):
                if held.get(p, 0) != g.pool.refs(p) or ((p in free) != (g.pool.refs(p) == 0)):
                    raise AssertionError(f"group {g.gid}: page {p} held {held.get(p, 0)}x, count {g.pool.refs(p)}, "
                                         f"free {p in free}")
            if g.pool.free + len(held) != g.pool.usable:
                raise AssertionError(f"group {g.gid}: {g.pool.usable - g.pool.free - len(held)} pages lost")
