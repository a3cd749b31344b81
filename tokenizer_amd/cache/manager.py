"""The cache manager: pages for keys and values, a block table per request and group, state slots.

Layers whose mixers ask for the same kind of cache (`CacheNeed.page_key`) form a *group*.  A
group has its own allocator and pool of pages; a request has one block table per group, and
all layers of a group use the same page ids in their own pool tensors.  A "window" group gives
pages back once every later query is past them.  Beside the pages, each live request holds
one *slot* for per-request state of fixed size (used by mixers that declare a `state_shape`).

This class only does bookkeeping on the host; the tensors live in `CachePools`.  The bookkeeping itself
(tables, reservation, window release, prefix sharing, slots, and the packing of a step's batch description)
is C++ (`csrc/host/cache_core.cpp`); this class binds it and keeps the Python-side names of requests.
"""
from __future__ import annotations

import ctypes
import dataclasses

import numpy as np

from .. import host as _host
from ..parts.spec import CacheNeed
from .allocator import PageAllocator


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


def _window_of_window_kind(need: CacheNeed) -> int:
    if need.window is None or need.window < 0:
        raise ValueError("a window cache needs a window")
    return int(need.window)


# What a kind of cache keeps, as the one number the bookkeeping works with: None = the keys and values of
# every position; w >= 0 = a query reads at most w positions behind itself, and pages wholly behind every
# later query are given back.  A mixer with another name for its need (or another way to derive the window
# from its `CacheNeed`) adds its kind here; kind "none" asks for no pages at all.
CACHE_KINDS: dict[str, "callable"] = {
    "full": lambda need: None,
    "window": _window_of_window_kind,
}


def retention_window(need: CacheNeed) -> int | None:
    """The window behind which a group of this need gives pages back (None: never)."""
    try:
        rule = CACHE_KINDS[need.kind]
    except KeyError:
        raise ValueError(f"unknown cache kind {need.kind!r}; known: none, {', '.join(sorted(CACHE_KINDS))}") from None
    return rule(need)


def plan_groups(needs: list[CacheNeed]) -> tuple[list[tuple[CacheNeed, list[int]]], list[int | None]]:
    """Group the layers by what they need.  Returns the groups and, per layer, its group index."""
    groups: list[tuple[CacheNeed, list[int]]] = []
    keys: dict[tuple, int] = {}
    group_of: list[int | None] = []
    for layer, need in enumerate(needs):
        if need.kind == "none":
            group_of.append(None)
            continue
        try:
            retention_window(need)
        except ValueError as err:
            raise ValueError(f"layer {layer}: {err}") from None
        key = need.page_key()
        if key not in keys:
            keys[key] = len(groups)
            groups.append((need, []))
        groups[keys[key]][1].append(layer)
        group_of.append(keys[key])
    return groups, group_of


_FIRST_NAMED = 1 << 62      # handles of requests whose id is not a small non-negative integer


def _is_handle(rid) -> bool:
    return isinstance(rid, int) and not isinstance(rid, bool) and 0 <= rid < _FIRST_NAMED


class _Requests:
    """The live requests, looked up by the caller's request id: `requests[rid]` is a snapshot
    (`RequestCache`) of what the request holds now."""

    def __init__(self, manager: "CacheManager"):
        self._manager = manager

    def __contains__(self, rid) -> bool:
        return self._manager.has_request(rid)

    def __len__(self) -> int:
        return self._manager._lib.ta_cache_n_requests(self._manager._core)

    def __iter__(self):
        manager = self._manager
        out = (ctypes.c_int64 * max(1, len(self)))()
        count = manager._lib.ta_cache_request_ids(manager._core, out)
        names = {handle: rid for rid, handle in manager._ids.items()}
        return iter([names.get(handle, handle) for handle in out[:count]])

    def __getitem__(self, rid) -> RequestCache:
        manager = self._manager
        handle = manager._handle_of(rid)
        tables = [manager.table(rid, g) for g in range(len(manager.groups))]
        return RequestCache(manager._lib.ta_cache_seq_len(manager._core, handle), tables,
                            manager._lib.ta_cache_slot(manager._core, handle))

    def values(self):
        return [self[rid] for rid in self]


class _CoreOwner:
    """Deletes the C++ core when the last Python object that points into it has gone (the manager itself, the
    allocators of its groups, a scheduler built on it)."""

    def __init__(self, lib, core):
        self._lib, self._core = lib, core

    def __del__(self):
        if self._core:
            self._lib.ta_cache_delete(self._core)
            self._core = None


class CacheManager:
    def __init__(self, needs: list[CacheNeed], num_pages: int, page_size: int = 16, max_requests: int = 8,
                 prefix_cache: bool = False):
        planned, self.group_of_layer = plan_groups(needs)
        self.page_size = page_size
        self.num_pages = num_pages
        self.max_requests = max_requests
        self._lib = _host.lib()
        kept = [retention_window(need) for need, _ in planned]
        windows = (ctypes.c_int32 * max(1, len(planned)))(*[-1 if w is None else w for w in kept])
        self.state_layers = [i for i, need in enumerate(needs) if need.state_shape is not None]
        self._core = self._lib.ta_cache_new(len(planned), windows, num_pages, page_size, max_requests,
                                            1 if prefix_cache else 0, len(self.state_layers))
        if not self._core:
            raise ValueError("num_pages and max_requests must not be negative and page_size must be positive")
        self._core_owner = _CoreOwner(self._lib, self._core)
        self.groups = [CacheGroup(need, layers, PageAllocator(num_pages, page_size,
                                                              _borrowed=self._lib.ta_cache_allocator(self._core, g),
                                                              _owner=self._core_owner))
                       for g, (need, layers) in enumerate(planned)]
        # Sharing a prefix needs every group to keep all positions (a window group drops pages) and no layer
        # that keeps state of its own in the request's slot (it would never see an attached prefix's tokens).
        self.prefix_cache = bool(self._lib.ta_cache_prefix_enabled(self._core))
        # A request id that is a small non-negative integer is its own handle in the core (so the scheduler core,
        # which numbers its sequences, and this class speak of the same requests); any other id gets one here.
        self._ids: dict[object, int] = {}
        self._next_handle = _FIRST_NAMED
        self.requests = _Requests(self)

    def _handle_of(self, rid) -> int:
        """The core's handle of a live request; KeyError for one that is not live."""
        if _is_handle(rid):
            if not self._lib.ta_cache_has_request(self._core, rid):
                raise KeyError(rid)
            return rid
        return self._ids[rid]

    # ------------------------------------------------------------------ requests
    def add_request(self, rid) -> RequestCache:
        if self.has_request(rid):
            raise KeyError(f"request {rid!r} is already live")
        handle = rid if _is_handle(rid) else self._next_handle
        slot = self._lib.ta_cache_add_request(self._core, handle)
        if slot < 0:
            raise OutOfPages(f"all {self.max_requests} request slots are taken")
        if not _is_handle(rid):
            self._next_handle += 1
            self._ids[rid] = handle
        return RequestCache(0, [[] for _ in self.groups], slot)

    def has_request(self, rid) -> bool:
        if _is_handle(rid):
            return bool(self._lib.ta_cache_has_request(self._core, rid))
        return rid in self._ids

    def seq_len(self, rid) -> int:
        return self._lib.ta_cache_seq_len(self._core, self._handle_of(rid))

    def slot(self, rid) -> int:
        return self._lib.ta_cache_slot(self._core, self._handle_of(rid))

    def table(self, rid, group: int) -> list[int]:
        handle = self._handle_of(rid)
        length = self._lib.ta_cache_table_len(self._core, handle, group)
        out = (ctypes.c_int32 * max(1, length))()
        self._lib.ta_cache_table(self._core, handle, group, out)
        return list(out[:length])

    def free_slot_count(self) -> int:
        return self._lib.ta_cache_free_slots(self._core)

    # --------------------------------------------------------------------- pages
    def first_needed_position(self, group: int, seq_len: int) -> int:
        """Lowest key position any query at or past `seq_len` still reads in this group."""
        return self._lib.ta_cache_first_needed_position(self._core, group, seq_len)

    def pages_missing(self, rid, new_len: int) -> list[int]:
        """Pages each group lacks for the request to hold `new_len` tokens."""
        out = (ctypes.c_int32 * max(1, len(self.groups)))()
        self._lib.ta_cache_pages_missing(self._core, self._handle_of(rid), new_len, out)
        return list(out[:len(self.groups)])

    def can_reserve(self, rid, new_len: int) -> bool:
        return self._lib.ta_cache_can_reserve(self._core, self._handle_of(rid), new_len) == 1

    def reserve(self, rid, new_len: int) -> bool:
        """Give the request pages for `new_len` tokens in every group, or change nothing."""
        return self._lib.ta_cache_reserve(self._core, self._handle_of(rid), new_len) == 1

    def advance(self, rid, new_len: int) -> None:
        """The request now holds `new_len` tokens; window groups give back pages no query reads again."""
        status = self._lib.ta_cache_advance(self._core, self._handle_of(rid), new_len)
        if status == -4:
            raise ValueError("a request's length never shrinks")
        if status == -5:
            raise ValueError(f"request {rid!r} holds too few pages for {new_len} tokens")

    def release(self, rid) -> None:
        """End a request: every page and its slot go back."""
        handle = self._handle_of(rid)
        self._ids.pop(rid, None)
        self._lib.ta_cache_release(self._core, handle)

    # -------------------------------------------------------------- prefix cache
    def attach_shared_prefix(self, rid, tokens) -> int:
        """Take already computed full pages for the start of `tokens`; returns how many tokens they hold.

        The last token is left out of the lookup so that the page it lands in stays private
        (qwen-server/src/engine.rs:490-495,519-527).  Only for a request that holds nothing yet.
        """
        keep, pointer = _host.token_array(tokens)
        return self._lib.ta_cache_attach_shared_prefix(self._core, self._handle_of(rid), pointer, len(keep))

    def detach(self, rid) -> None:
        """Give back everything a request holds but keep it known (used when an admission is rolled back)."""
        self._lib.ta_cache_detach(self._core, self._handle_of(rid))

    def publish(self, rid, tokens) -> None:
        """Make the full, written pages of `tokens` findable by later requests."""
        if not self.prefix_cache:
            return
        keep, pointer = _host.token_array(tokens)
        self._lib.ta_cache_publish(self._core, self._handle_of(rid), pointer, len(keep))

    # ------------------------------------------------------------------- packing
    def pack_batch(self, rids, token_lists, want_lists, out: np.ndarray, table_width: int | None = None,
                   padded: tuple | None = None):
        """Write one step's batch description into the int32 array `out` (see `engine/batch.py` for the
        order of its parts).  `padded`: five counts (tokens, entries, wanted places, tiles of sixteen prompt
        tokens, single rows) up to which the description is filled with parts that do nothing.  Returns (total
        length, the parts' lengths, the table width per group, and per entry its first row, token count, first
        position and state slot)."""
        n = len(rids)
        ids = np.array([rid if _is_handle(rid) else self._ids[rid] for rid in rids], dtype=np.int64)
        n_tokens = np.array([len(t) for t in token_lists], dtype=np.int32)
        n_want = np.array([len(w) for w in want_lists], dtype=np.int32)
        # (One conversion per entry: a generator over every token costs a prompt of 2,048 tokens 0.1 ms.)
        arrays = [np.asarray(ts, dtype=np.int32) for ts in token_lists]
        tokens = arrays[0] if len(arrays) == 1 else np.concatenate(arrays) if arrays else np.zeros(0, np.int32)
        tokens = np.ascontiguousarray(tokens)
        want = np.fromiter((w for ws in want_lists for w in ws), dtype=np.int32, count=int(n_want.sum()))
        n_groups = len(self.groups)
        sizes = np.zeros(9 + 2 * n_groups, dtype=np.int64)
        widths = np.zeros(max(1, n_groups), dtype=np.int32)
        info = np.zeros(max(1, 4 * n), dtype=np.int32)
        as_i32 = lambda a: a.ctypes.data_as(ctypes.POINTER(ctypes.c_int32))
        as_i64 = lambda a: a.ctypes.data_as(ctypes.POINTER(ctypes.c_int64))
        fill = None if padded is None else np.asarray(padded, dtype=np.int64)
        total = self._lib.ta_cache_pack_batch(self._core, n, as_i64(ids), as_i32(n_tokens), as_i32(tokens),
                                              as_i32(n_want), as_i32(want),
                                              -1 if table_width is None else table_width,
                                              None if fill is None else as_i64(fill), as_i32(out), out.size,
                                              as_i64(sizes), as_i32(widths), as_i32(info))
        if total == -9:
            raise ValueError("an entry without tokens, or counts to fill up to that are smaller than the batch's")
        if total == -3:
            raise KeyError("a request of the batch is not live")
        if total == -5:
            raise RuntimeError("a request holds too few pages for its new tokens (they are reserved before a step)")
        if total == -6:
            raise RuntimeError("a request writes a position into a page it gave back")
        if total == -7:
            raise ValueError("a block table is wider than the fixed width")
        if total == -8:
            raise ValueError("the packed batch does not fit the buffers it should land in")
        if total < 0:
            raise RuntimeError(f"the batch could not be packed (status {total})")
        return int(total), sizes.tolist(), widths[:n_groups].tolist(), info[:4 * n].reshape(n, 4).tolist()

    def packed_size(self, token_counts, want_counts, table_widths, padded: tuple | None = None) -> int:
        """Length of the packed description of a batch with these token and want counts and table widths (filled up
        to the counts of `padded`, if given)."""
        if padded is not None:
            tokens, n, wanted, tiles, single = padded
        else:
            n, tokens, wanted = len(token_counts), sum(token_counts), sum(want_counts)
            tiles = sum(-(-c // 16) for c in token_counts if c != 1)
            single = sum(1 for c in token_counts if c == 1)
        return (3 * tokens + (n + 1) + 2 * n + wanted + 2 * tiles + single
                + sum(tokens + n * w for w in table_widths))

    # ------------------------------------------------------------------ checking
    def check_invariants(self) -> None:
        """No page lost, held twice or freed twice; slots likewise."""
        assert self._lib.ta_cache_check(self._core) == 0, _host.message()
