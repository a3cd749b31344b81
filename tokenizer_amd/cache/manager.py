"""The cache manager: pages for keys and values, a block table per request and group, state slots.

Layers whose mixers ask for the same kind of cache (`CacheNeed.page_key`) form a *group*.  A
group has its own allocator and pool of pages; a request has one block table per group, and
all layers of a group use the same page ids in their own pool tensors.  A "window" group gives
pages back once every later query is past them.  Beside the pages, each live request holds
one *slot* for per-request state of fixed size (used by mixers that declare a `state_shape`).

This class only does bookkeeping on the host; the tensors live in `CachePools`.
"""
from __future__ import annotations

import dataclasses

from ..parts.spec import CacheNeed
from .allocator import PageAllocator, pages_for_len


class OutOfPages(RuntimeError):
    """The pool cannot hold what a request needs now (the scheduler preempts or waits)."""


@dataclasses.dataclass
class CacheGroup:
    need: CacheNeed
    layers: list[int]            # layer indices whose cache lives in this group
    allocator: PageAllocator


@dataclasses.dataclass
class RequestCache:
    seq_len: int = 0
    tables: list[list[int]] = dataclasses.field(default_factory=list)   # per group; -1 = page given back
    slot: int = -1


def plan_groups(needs: list[CacheNeed]) -> tuple[list[tuple[CacheNeed, list[int]]], list[int | None]]:
    """Group the layers by what they need.  Returns the groups and, per layer, its group index."""
    groups: list[tuple[CacheNeed, list[int]]] = []
    keys: dict[tuple, int] = {}
    group_of: list[int | None] = []
    for layer, need in enumerate(needs):
        if need.kind == "none":
            group_of.append(None)
            continue
        if need.kind not in ("full", "window"):
            raise ValueError(f"layer {layer} asks for an unknown cache kind {need.kind!r}")
        if need.kind == "window" and (need.window is None or need.window < 0):
            raise ValueError(f"layer {layer} asks for a window cache without a window")
        key = need.page_key()
        if key not in keys:
            keys[key] = len(groups)
            groups.append((need, []))
        groups[keys[key]][1].append(layer)
        group_of.append(keys[key])
    return groups, group_of


class CacheManager:
    def __init__(self, needs: list[CacheNeed], num_pages: int, page_size: int = 16, max_requests: int = 8,
                 prefix_cache: bool = False):
        planned, self.group_of_layer = plan_groups(needs)
        self.page_size = page_size
        self.num_pages = num_pages
        self.groups = [CacheGroup(need, layers, PageAllocator(num_pages, page_size)) for need, layers in planned]
        self.max_requests = max_requests
        self._free_slots = list(range(max_requests - 1, -1, -1))
        self.requests: dict[object, RequestCache] = {}
        # Sharing a prefix needs every group to keep all positions (a window group drops pages).
        self.prefix_cache = prefix_cache and all(g.need.kind == "full" for g in self.groups)
        self.state_layers = [i for i, need in enumerate(needs) if need.state_shape is not None]

    # ------------------------------------------------------------------ requests
    def add_request(self, rid) -> RequestCache:
        if rid in self.requests:
            raise KeyError(f"request {rid!r} is already live")
        if not self._free_slots:
            raise OutOfPages(f"all {self.max_requests} request slots are taken")
        entry = RequestCache(0, [[] for _ in self.groups], self._free_slots.pop())
        self.requests[rid] = entry
        return entry

    def has_request(self, rid) -> bool:
        return rid in self.requests

    def seq_len(self, rid) -> int:
        return self.requests[rid].seq_len

    def slot(self, rid) -> int:
        return self.requests[rid].slot

    def table(self, rid, group: int) -> list[int]:
        return self.requests[rid].tables[group]

    def free_slot_count(self) -> int:
        return len(self._free_slots)

    # --------------------------------------------------------------------- pages
    def first_needed_position(self, group: int, seq_len: int) -> int:
        """Lowest key position any query at or past `seq_len` still reads in this group."""
        need = self.groups[group].need
        if need.kind == "window":
            return max(0, seq_len - need.window)
        return 0

    def pages_missing(self, rid, new_len: int) -> list[int]:
        """Pages each group lacks for the request to hold `new_len` tokens."""
        entry = self.requests[rid]
        return [max(0, pages_for_len(new_len, self.page_size) - len(table)) for table in entry.tables]

    def can_reserve(self, rid, new_len: int) -> bool:
        return all(group.allocator.available() >= missing
                   for group, missing in zip(self.groups, self.pages_missing(rid, new_len)))

    def reserve(self, rid, new_len: int) -> bool:
        """Give the request pages for `new_len` tokens in every group, or change nothing."""
        missing = self.pages_missing(rid, new_len)
        if not all(group.allocator.available() >= count for group, count in zip(self.groups, missing)):
            return False
        entry = self.requests[rid]
        for group, table, count in zip(self.groups, entry.tables, missing):
            table.extend(group.allocator.alloc_n(count))
        return True

    def advance(self, rid, new_len: int) -> None:
        """The request now holds `new_len` tokens; window groups give back pages no query reads again."""
        entry = self.requests[rid]
        if new_len < entry.seq_len:
            raise ValueError("a request's length never shrinks")
        if any(pages_for_len(new_len, self.page_size) > len(table) for table in entry.tables):
            raise ValueError(f"request {rid!r} holds too few pages for {new_len} tokens")
        entry.seq_len = new_len
        for index, (group, table) in enumerate(zip(self.groups, entry.tables)):
            if group.need.kind != "window":
                continue
            first = self.first_needed_position(index, new_len)
            for page_index in range(first // self.page_size):
                if table[page_index] >= 0:
                    group.allocator.free_page(table[page_index])
                    table[page_index] = -1

    def release(self, rid) -> None:
        """End a request: every page and its slot go back."""
        entry = self.requests.pop(rid)
        for group, table in zip(self.groups, entry.tables):
            for page in table:
                if page >= 0:
                    group.allocator.free_page(page)
        self._free_slots.append(entry.slot)

    # -------------------------------------------------------------- prefix cache
    def attach_shared_prefix(self, rid, tokens) -> int:
        """Take already computed full pages for the start of `tokens`; returns how many tokens they hold.

        The last token is left out of the lookup so that the page it lands in stays private
        (qwen-server/src/engine.rs:490-495,519-527).  Only for a request that holds nothing yet.
        """
        entry = self.requests[rid]
        if not self.prefix_cache or entry.seq_len or any(entry.tables):
            return 0
        lookup = tokens[:-1] if len(tokens) else tokens
        marks = [group.allocator.peak_mark() for group in self.groups]
        taken = [group.allocator.take_shared_prefix(lookup) for group in self.groups]
        count = min(len(pages) for pages in taken) if taken else 0
        for group, pages, mark in zip(self.groups, taken, marks):
            for page in pages[count:]:
                group.allocator.free_page(page)
            if len(pages) > count:
                group.allocator.rewind_peaks(mark)
        for table, pages in zip(entry.tables, taken):
            table.extend(pages[:count])
        entry.seq_len = count * self.page_size
        return entry.seq_len

    def detach(self, rid) -> None:
        """Give back everything a request holds but keep it known (used when an admission is rolled back)."""
        entry = self.requests[rid]
        for group, table in zip(self.groups, entry.tables):
            for page in table:
                if page >= 0:
                    group.allocator.free_page(page)
            table.clear()
        entry.seq_len = 0

    def publish(self, rid, tokens) -> None:
        """Make the full, written pages of `tokens` findable by later requests."""
        if not self.prefix_cache:
            return
        entry = self.requests[rid]
        written = tokens[:entry.seq_len]
        for group, table in zip(self.groups, entry.tables):
            group.allocator.publish_prompt_pages(written, table)

    # ------------------------------------------------------------------ checking
    def check_invariants(self) -> None:
        """No page lost, held twice or freed twice; slots likewise."""
        for index, group in enumerate(self.groups):
            group.allocator.check_invariants()
            held: dict[int, int] = {}
            for entry in self.requests.values():
                for page in entry.tables[index]:
                    if page >= 0:
                        held[page] = held.get(page, 0) + 1
            for page in range(group.allocator.capacity()):
                assert group.allocator.refcount(page) == held.get(page, 0), \
                    f"group {index} page {page}: count {group.allocator.refcount(page)}, held {held.get(page, 0)}"
            assert (group.allocator.free_count() + group.allocator.cached_count()
                    + group.allocator.live_count() == group.allocator.capacity())
        slots = [entry.slot for entry in self.requests.values()]
        assert len(set(slots)) == len(slots), "a slot is held twice"
        assert sorted(slots + self._free_slots) == list(range(self.max_requests)), "a slot was lost"
