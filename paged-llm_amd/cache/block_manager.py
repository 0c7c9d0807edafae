"""Which page holds which positions of which request: host-side bookkeeping, no tensors.

Behaviour follows pagedllm/block_manager.py:48-243 (reference-counted pages, a free list in
least-recently-freed order, a hash index of full pages for prefix reuse, copy-on-write after a
fork, all-or-nothing allocation), extended in two directions the reference does not have:

* **Groups.**  Layers whose mixers keep different things per token (all keys; only a window of
  them; another page shape) form groups.  Each group has its own pool of pages and each request
  has one block table per group.  A windowed group gives a page back as soon as every position
  in it lies outside the window of all queries still to come.
* **State slots.**  Mixers with state of fixed size per request get one slot id per live
  request from ``StateSlotPool``; the slot is handed out with the first pages and returned with
  the last.  A model without such mixers has slot size zero, and the pool only counts.

A table entry ``NO_PAGE`` (-1) marks a page that a window has passed; kernels never read it.
"""

from __future__ import annotations

import hashlib
import struct
from collections import OrderedDict
import itertools
from dataclasses import dataclass, field

NO_PAGE = -1


@dataclass(frozen=True)
class GroupSpec:
    name: str
    kind: str = "full"        # "full" | "window"
    window: int = 0           # positions kept, for kind "window"

    def __post_init__(self):
        if self.kind not in ("full", "window"):
            raise ValueError(f"unknown cache group kind {self.kind!r}")
        if self.kind == "window" and self.window <= 0:
            raise ValueError("a windowed group needs window > 0")


@dataclass(frozen=True)
class PageCopy:
    """A page copy the step function must do before the next forward pass."""
    src: int
    dst: int


def chain_digest(prev: bytes | None, tokens: list[int]) -> bytes:
    """Digest of a full page's tokens chained to its predecessor's, the same in every process
    (the reference chains Python's process-local ``hash``, pagedllm/block_manager.py:43-45)."""
    h = hashlib.blake2b(digest_size=16)
    h.update(prev or b"\0" * 16)
    h.update(struct.pack(f"<{len(tokens)}q", *tokens))
    return h.digest()


class PagePool:
    """Pages of one group: reference counts, the free list, the hash index."""

    def __init__(self, num_pages: int, keep_hashes: bool):
        if num_pages <= 0:
            raise ValueError("a page pool needs at least one page")
        self.num_pages = num_pages
        self.keep_hashes = keep_hashes
        self.refs = [0] * num_pages
        self.digest: list[bytes | None] = [None] * num_pages
        # Free pages, least recently freed first; that end is handed out (and evicted) first.
        self.free: OrderedDict[int, None] = OrderedDict((i, None) for i in range(num_pages))
        self.by_digest: dict[bytes, int] = {}

    @property
    def num_free(self) -> int:
        return len(self.free)

    def take(self) -> int:
        """A fresh page with one reference; its old content stops being findable."""
        page, _ = self.free.popitem(last=False)
        assert self.refs[page] == 0, f"page {page} on the free list with {self.refs[page]} references"
        self._forget(page)
        self.refs[page] = 1
        return page

    def _forget(self, page: int) -> None:
        d = self.digest[page]
        if d is not None:
            if self.by_digest.get(d) == page:
                del self.by_digest[d]
            self.digest[page] = None

    def share(self, page: int) -> None:
        """One more holder of a page (a free page with findable content is revived)."""
        if self.refs[page] == 0:
            del self.free[page]
        self.refs[page] += 1

    def drop(self, page: int) -> None:
        assert self.refs[page] > 0, f"double free of page {page}"
        self.refs[page] -= 1
        if self.refs[page] == 0:
            if not self.keep_hashes:
                self._forget(page)
            self.free[page] = None

    def remember(self, page: int, d: bytes) -> bool:
        """Index a full page by its digest; False if another page already holds that content."""
        if d in self.by_digest:
            return self.by_digest[d] == page
        self.digest[page] = d
        self.by_digest[d] = page
        return True

    def find(self, d: bytes) -> int | None:
        return self.by_digest.get(d)


class StateSlotPool:
    """Ids of fixed-size per-request state slots."""

    def __init__(self, num_slots: int):
        self.num_slots = num_slots
        self._free = list(range(num_slots - 1, -1, -1))
        self._held: set[int] = set()

    @property
    def num_free(self) -> int:
        return len(self._free)

    def acquire(self) -> int | None:
        if not self._free:
            return None
        s = self._free.pop()
        self._held.add(s)
        return s

    def release(self, slot: int) -> None:
        assert slot in self._held, f"state slot {slot} released twice"
        self._held.remove(slot)
        self._free.append(slot)


@dataclass
class _Holding:
    """What one request holds."""
    tables: dict[str, list[int]]
    state_slot: int | None = None
    version: int = 0          # a new number whenever any table changes (never reused by another holding)
    digests: list = field(default_factory=list)   # chained digests of the request's first full pages, worked out ahead


class CacheManager:
    def __init__(self, groups: list[GroupSpec], num_pages: int | dict[str, int], block_size: int,
                 enable_prefix_caching: bool = True, num_state_slots: int = 0):
        if not groups:
            groups = []
        if block_size <= 0 or block_size & (block_size - 1):
            raise ValueError("block_size must be a power of two")
        self.groups = {g.name: g for g in groups}
        self.block_size = block_size
        # A windowed group forgets early pages, so a cached prefix cannot be re-entered; and a state of fixed
        # size exists only as of the last token run, so a request that skipped a cached prefix would start
        # from a state that never saw it.  Prefix reuse is off in both cases.
        self.prefix_caching = (enable_prefix_caching and bool(groups) and all(g.kind == "full" for g in groups)
                               and num_state_slots == 0)
        self.pools: dict[str, PagePool] = {}
        for g in groups:
            n = num_pages[g.name] if isinstance(num_pages, dict) else num_pages
            self.pools[g.name] = PagePool(n, keep_hashes=self.prefix_caching)
        self.slots = StateSlotPool(num_state_slots)
        self.uses_state = num_state_slots > 0
        self._held: dict[object, _Holding] = {}
        self._versions = itertools.count(1)
        self._pending: dict[str, list[PageCopy]] = {g.name: [] for g in groups}
        self._pending_state: list[PageCopy] = []         # state slots to copy (after a fork), as (src, dst)
        self.num_cache_queries = 0
        self.num_cache_hits = 0

    # ------------------------------------------------------------------ introspection
    def num_free_pages(self, group: str | None = None) -> int:
        if group is None:
            return min((p.num_free for p in self.pools.values()), default=0)
        return self.pools[group].num_free

    def num_pages(self, group: str | None = None) -> int:
        if group is None:
            return min((p.num_pages for p in self.pools.values()), default=0)
        return self.pools[group].num_pages

    def num_cached_pages(self, group: str | None = None) -> int:
        if group is None:
            return min((len(p.by_digest) for p in self.pools.values()), default=0)
        return len(self.pools[group].by_digest)

    def usage(self) -> float:
        return max((1.0 - p.num_free / p.num_pages for p in self.pools.values()), default=0.0)

    def pages_for(self, num_tokens: int) -> int:
        return (num_tokens + self.block_size - 1) // self.block_size

    def holds(self, request) -> bool:
        return request in self._held

    def block_table(self, request, group: str) -> list[int]:
        return self._held[request].tables[group]

    def step_fields(self, request) -> tuple:
        """(block tables by group, state slot, table version) of ``request`` with one look-up, for whoever builds a
        step's entries for hundreds of requests.  The tables are the manager's own lists: read them, do not keep them."""
        h = self._held[request]
        return h.tables, h.state_slot, h.version

    def table_version(self, request) -> int:
        """A number that changes whenever any block table of ``request`` does (a page appended, copied
        for a write, or given back by a window), and that no other state of any request shares: who
        has read the tables at this number need not read them again."""
        return self._held[request].version

    def state_slot(self, request) -> int | None:
        h = self._held.get(request)
        return None if h is None else h.state_slot

    def slot_mapping(self, request, group: str, start: int, count: int) -> list[int]:
        """Flat slot (page * block_size + offset) of each position in [start, start + count)."""
        table, bs = self._held[request].tables[group], self.block_size
        return [table[t // bs] * bs + t % bs for t in range(start, start + count)]

    # ------------------------------------------------------------------ prefix reuse
    def find_cached_prefix(self, tokens: list[int]) -> tuple[dict[str, list[int]], int]:
        """Longest prefix of ``tokens``, in whole pages, whose pages are still findable in every
        group.  The page holding the last token is never returned, so at least one token is
        computed and there are logits to sample from (pagedllm/block_manager.py:111-133).
        Takes no references."""
        if not self.prefix_caching:
            return {g: [] for g in self.groups}, 0
        self.num_cache_queries += 1
        bs = self.block_size
        full = (len(tokens) - 1) // bs
        hits: dict[str, list[int]] = {g: [] for g in self.groups}
        prev = None
        n = 0
        for i in range(full):
            d = chain_digest(prev, tokens[i * bs:(i + 1) * bs])
            found = {g: pool.find(d) for g, pool in self.pools.items()}
            if any(p is None for p in found.values()):
                break
            for g, p in found.items():
                hits[g].append(p)
            prev = d
            n += 1
        if n:
            self.num_cache_hits += 1
        return hits, n * bs

    def note_computed(self, request, tokens: list[int], before: int, after: int) -> None:
        """Positions [before, after) of ``tokens`` now sit in the cache: index the pages that
        became full (pagedllm/block_manager.py:135-158)."""
        if not self.prefix_caching or request not in self._held:
            return
        bs = self.block_size
        first, last = before // bs, after // bs
        if first == last:
            return
        hold = self._held[request]
        ready = hold.digests
        for g, pool in self.pools.items():
            table = hold.tables[g]
            prev = pool.digest[table[first - 1]] if first > 0 else None
            for i in range(first, last):
                page = table[i]
                if pool.digest[page] is None:
                    if prev is None and i > 0:
                        break                      # predecessor not indexed: the chain cannot go on
                    if i < len(ready) and (i == 0 or ready[i - 1] == prev):
                        d = ready[i]               # worked out while the step ran, on the same chain
                    else:
                        d = chain_digest(prev, tokens[i * bs:(i + 1) * bs])
                    if not pool.remember(page, d):
                        break                      # same content already indexed under another page
                prev = pool.digest[page]

    def digests_ahead(self, request, tokens: list[int], after: int) -> None:
        """The digests under which ``note_computed`` will index the full pages of ``tokens[:after]``, worked out
        ahead of it: they depend on the tokens alone, so whoever launched a step that computes a long prompt portion
        can have them made while the GPU runs, and the step's end only has to index them."""
        hold = self._held.get(request) if self.prefix_caching else None
        if hold is None:
            return
        bs, ready = self.block_size, hold.digests
        prev = ready[-1] if ready else None
        for i in range(len(ready), after // bs):
            prev = chain_digest(prev, tokens[i * bs:(i + 1) * bs])
            ready.append(prev)

    # ------------------------------------------------------------------ allocation
    def _first_needed_page(self, g: GroupSpec, num_computed: int) -> int:
        """Pages below this index are out of the window of every query at position >= num_computed."""
        if g.kind != "window":
            return 0
        first_key = num_computed - g.window + 1
        return max(0, first_key) // self.block_size

    def _nothing_to_do(self, hold: _Holding, num_computed: int, num_new: int, total_pages: int) -> bool:
        """The usual decode step: the pages are there, the one written to is the request's alone, and
        no window has moved past a page."""
        bs = self.block_size
        idx = num_computed // bs
        for name, g in self.groups.items():
            table = hold.tables[name]
            if g.kind != "full" or len(table) < total_pages:
                return False
            if num_new > 0 and num_computed % bs != 0 and self.pools[name].refs[table[idx]] > 1:
                return False
        return True

    def allocate(self, request, num_computed: int, num_new: int,
                 cached: dict[str, list[int]] | None = None) -> bool:
        """Make ``request`` hold pages for positions [0, num_computed + num_new) in every group
        (less what a window has passed).  ``cached`` are the pages ``find_cached_prefix`` returned;
        they are shared, and ``num_computed`` must then already count them.

        Either everything succeeds, or nothing changes and False is returned
        (pagedllm/block_manager.py:161-217)."""
        bs = self.block_size
        hold = self._held.get(request)
        new_request = hold is None
        total_pages = self.pages_for(num_computed + num_new)
        if hold is not None and not cached and self._nothing_to_do(hold, num_computed, num_new, total_pages):
            return True
        cached = cached or {}
        plan = {}
        for name, g in self.groups.items():
            pool = self.pools[name]
            table = [] if new_request else hold.tables[name]
            hits = cached.get(name, []) if new_request or not table else []
            have = len(table) + len(hits)
            need = max(0, total_pages - have)
            # Copy-on-write: the write starts inside a page that someone else also holds.
            cow_index = None
            if num_new > 0 and num_computed % bs != 0:
                idx = num_computed // bs
                if idx < have:
                    page = (table + hits)[idx]
                    if page != NO_PAGE and pool.refs[page] + (1 if idx >= len(table) else 0) > 1:
                        cow_index = idx
            # Pages a window has passed come back before the new ones are taken.
            first_needed = self._first_needed_page(g, num_computed)
            releasable = [i for i in range(min(first_needed, len(table))) if table[i] != NO_PAGE
                          and pool.refs[table[i]] == 1]
            revive = sum(1 for p in hits if pool.refs[p] == 0)
            available = pool.num_free - revive + len(releasable)
            if need + (1 if cow_index is not None else 0) > available:
                return False
            plan[name] = (hits, need, cow_index, first_needed)
        if new_request and self.uses_state and self.slots.num_free == 0:
            return False

        if new_request:
            hold = _Holding(tables={name: [] for name in self.groups})
            if self.uses_state:
                hold.state_slot = self.slots.acquire()
            self._held[request] = hold
        changed = new_request
        for name, (hits, need, cow_index, first_needed) in plan.items():
            pool, table = self.pools[name], hold.tables[name]
            changed = changed or bool(hits) or need > 0 or cow_index is not None
            for i in range(min(first_needed, len(table))):
                if table[i] != NO_PAGE:
                    pool.drop(table[i])
                    table[i] = NO_PAGE
                    changed = True
            for p in hits:
                pool.share(p)
            table.extend(hits)
            for i in range(need):
                # A page that lies wholly before the window is never written or read.
                table.append(pool.take() if len(table) >= first_needed else NO_PAGE)
            if cow_index is not None:
                shared = table[cow_index]
                fresh = pool.take()
                self._pending[name].append(PageCopy(shared, fresh))
                pool.drop(shared)
                table[cow_index] = fresh
        if changed:
            hold.version = next(self._versions)
        return True

    def fork(self, parent, child) -> None:
        """``child`` shares every page of ``parent`` (pagedllm/block_manager.py:225-231)."""
        assert child not in self._held, "child already holds pages"
        src = self._held[parent]
        hold = _Holding(tables={})
        for name, table in src.tables.items():
            for p in table:
                if p != NO_PAGE:
                    self.pools[name].share(p)
            hold.tables[name] = list(table)
        if self.uses_state:
            hold.state_slot = self.slots.acquire()
            if hold.state_slot is None:
                for name, table in hold.tables.items():
                    for p in table:
                        if p != NO_PAGE:
                            self.pools[name].drop(p)
                raise RuntimeError("no free state slot for a fork")
            self._pending_state.append(PageCopy(src.state_slot, hold.state_slot))
        hold.version = next(self._versions)
        self._held[child] = hold

    def free(self, request) -> None:
        """Give everything back; the deepest page first, so that the root of a shared prefix is
        the last to be evicted (pagedllm/block_manager.py:219-223)."""
        hold = self._held.pop(request, None)
        if hold is None:
            return
        for name, table in hold.tables.items():
            pool = self.pools[name]
            for p in reversed(table):
                if p != NO_PAGE:
                    pool.drop(p)
        if hold.state_slot is not None:
            self.slots.release(hold.state_slot)

    def take_pending_copies(self) -> dict[str, list[PageCopy]]:
        out = {g: ops for g, ops in self._pending.items() if ops}
        self._pending = {g: [] for g in self.groups}
        return out

    def take_pending_state_copies(self) -> list[PageCopy]:
        """State slots whose content the step function must copy before the next forward pass
        (a forked request starts from its parent's state)."""
        out, self._pending_state = self._pending_state, []
        return out

    # ------------------------------------------------------------------ self-check (tests)
    def check_invariants(self) -> None:
        """No page lost, none held by more or fewer than its count says, none both free and held."""
        for name, pool in self.pools.items():
            counted = [0] * pool.num_pages
            for hold in self._held.values():
                for p in hold.tables[name]:
                    if p != NO_PAGE:
                        counted[p] += 1
            for p in range(pool.num_pages):
                assert counted[p] == pool.refs[p], f"group {name}: page {p} has {pool.refs[p]} references, {counted[p]} holders"
                assert (p in pool.free) == (pool.refs[p] == 0), f"group {name}: page {p} free-list state disagrees with its count"
            assert len(pool.free) + sum(1 for r in pool.refs if r > 0) == pool.num_pages, f"group {name}: a page is lost"
            for d, p in pool.by_digest.items():
                assert pool.digest[p] == d
        held_slots = [h.state_slot for h in self._held.values() if h.state_slot is not None]
        assert len(held_slots) == len(set(held_slots)), "a state slot is held twice"
        assert len(held_slots) + self.slots.num_free == self.slots.num_slots or not self.uses_state, "a state slot is lost"
