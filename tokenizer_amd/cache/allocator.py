"""Page allocator: free stack, reference counts, prefix index and a list of cached pages.

The allocator itself is C++ (`csrc/host/page_allocator.cpp`); this class binds it.  Behaviour follows
qwen-infer/src/paged.rs:125-519.  Page ids are 0..n-1 and the first allocation returns 0; the page freed
last is handed out next.  A page published under the hash of its tokens stays out of the free stack when
its count falls to zero, so a later request with the same prefix can take it; `alloc` evicts such pages,
oldest first, only after the free stack is empty.
"""
from __future__ import annotations

import ctypes
import enum

from .. import host as _host


class AllocError(Exception):
    pass


class DoubleFree(AllocError):
    def __init__(self, page: int):
        super().__init__(f"double free of page {page}")
        self.page = page


class UnknownPage(AllocError):
    def __init__(self, page: int):
        super().__init__(f"page {page} was not issued by this allocator")
        self.page = page


class NotFull(AllocError):
    def __init__(self, page: int, length: int, page_size: int):
        super().__init__(f"page {page} needs {page_size} tokens to publish, got {length}")


class Release(enum.Enum):
    SHARED = "shared"    # another holder remains
    CACHED = "cached"    # count is zero, the page stays findable by its prefix
    FREED = "freed"      # back on the free stack


_RELEASES = (Release.SHARED, Release.CACHED, Release.FREED)
_CAPACITY, _FREE, _CACHED, _AVAILABLE, _LIVE, _OCCUPIED, _REFCOUNT, _ALL_ZERO, _PEAK_LIVE, _PEAK_OCCUPIED = range(10)


def prefix_page_hash(parent: int, tokens) -> int:
    """Chained hash of one full page of token ids (qwen-infer/src/paged.rs:93-100)."""
    keep, pointer = _host.token_array(tokens)
    return int(_host.lib().ta_prefix_page_hash(parent, pointer, len(keep)))


_tokens = _host.token_array


class PageAllocator:
    def __init__(self, num_pages: int, page_size: int = 16, _borrowed=None, _owner=None):
        self._lib = _host.lib()
        if _borrowed is not None:                 # an allocator that lives inside a cache manager's core
            self._handle, self._owned = _borrowed, False
            self._owner = _owner                  # whose core it is: kept alive as long as this object
        else:
            if num_pages < 0 or page_size <= 0:
                raise ValueError("num_pages must not be negative and page_size must be positive")
            self._handle, self._owned = self._lib.ta_alloc_new(num_pages, page_size), True
        self.page_size = page_size

    def __del__(self):
        if getattr(self, "_owned", False) and self._handle:
            self._lib.ta_alloc_delete(self._handle)
            self._handle = None

    def _get(self, what: int, arg: int = 0) -> int:
        return self._lib.ta_alloc_get(self._handle, what, arg)

    def _raise(self, status: int, page: int, length: int = 0) -> None:
        if status == -1:
            raise DoubleFree(page)
        if status == -2:
            raise UnknownPage(page)
        if status == -3:
            raise NotFull(page, length, self.page_size)

    # ------------------------------------------------------------------ counters
    def capacity(self) -> int:
        return self._get(_CAPACITY)

    def free_count(self) -> int:
        return self._get(_FREE)

    def cached_count(self) -> int:
        return self._get(_CACHED)

    def available(self) -> int:
        """Pages an allocation can draw on: the free stack plus cached pages."""
        return self._get(_AVAILABLE)

    def live_count(self) -> int:
        return self._get(_LIVE)

    def occupied(self) -> int:
        return self._get(_OCCUPIED)

    def refcount(self, page: int) -> int | None:
        count = self._get(_REFCOUNT, page)
        return None if count < 0 else count

    def all_refcounts_zero(self) -> bool:
        return bool(self._get(_ALL_ZERO))

    @property
    def peak_live(self) -> int:
        return self._get(_PEAK_LIVE)

    @property
    def peak_occupied(self) -> int:
        return self._get(_PEAK_OCCUPIED)

    def peak_mark(self) -> tuple[int, int]:
        return self.peak_live, self.peak_occupied

    def rewind_peaks(self, mark: tuple[int, int]) -> None:
        self._lib.ta_alloc_rewind_peaks(self._handle, mark[0], mark[1])

    # ---------------------------------------------------------------- alloc/free
    def alloc(self) -> int | None:
        page = self._lib.ta_alloc_alloc(self._handle)
        return None if page < 0 else page

    def alloc_n(self, n: int) -> list[int] | None:
        """`n` pages or none at all."""
        out = (ctypes.c_int32 * max(1, n))()
        if not self._lib.ta_alloc_alloc_n(self._handle, n, out):
            return None
        return list(out[:n])

    def free_page(self, page: int) -> Release:
        how = ctypes.c_int32(0)
        self._raise(self._lib.ta_alloc_free(self._handle, page, ctypes.byref(how)), page)
        return _RELEASES[how.value]

    def incref(self, page: int) -> None:
        self._raise(self._lib.ta_alloc_incref(self._handle, page), page)

    # -------------------------------------------------------------- prefix index
    def publish_full_page(self, parent_hash: int, tokens, page: int) -> None:
        keep, pointer = _tokens(tokens)
        self._raise(self._lib.ta_alloc_publish_full_page(self._handle, parent_hash, pointer, len(keep), page),
                    page, len(keep))

    def find_full_page(self, parent_hash: int, parent_page: int | None, tokens) -> int | None:
        keep, pointer = _tokens(tokens)
        page = self._lib.ta_alloc_find_full_page(self._handle, parent_hash, -1 if parent_page is None else parent_page,
                                                 pointer, len(keep))
        return None if page < 0 else page

    def take_shared_prefix(self, tokens) -> list[int]:
        """Published full pages of `tokens`, in order, each with one more holder; stops at the first miss."""
        keep, pointer = _tokens(tokens)
        out = (ctypes.c_int32 * max(1, len(keep) // self.page_size))()
        count = self._lib.ta_alloc_take_shared_prefix(self._handle, pointer, len(keep), out)
        return list(out[:count])

    def publish_prompt_pages(self, tokens, pages) -> None:
        """Index every full page of `tokens`; pages[i] holds tokens [i*size, (i+1)*size)."""
        keep, pointer = _tokens(tokens)
        held, page_pointer = _host.int_array(list(pages))
        self._lib.ta_alloc_publish_prompt_pages(self._handle, pointer, len(keep), page_pointer, len(held))

    def _publish_at(self, value: int, parent_hash: int, parent_page: int | None, tokens, page: int) -> bool:
        """Index `page` under a given hash value (what publishing does after hashing)."""
        keep, pointer = _tokens(tokens)
        return bool(self._lib.ta_alloc_publish_at(self._handle, value, parent_hash,
                                                  -1 if parent_page is None else parent_page, pointer, len(keep), page))

    def _find_at(self, value: int, parent_hash: int, parent_page: int | None, tokens) -> int | None:
        keep, pointer = _tokens(tokens)
        page = self._lib.ta_alloc_find_at(self._handle, value, parent_hash, -1 if parent_page is None else parent_page,
                                          pointer, len(keep))
        return None if page < 0 else page

    def reclaim_cached(self) -> None:
        self._lib.ta_alloc_reclaim_cached(self._handle)

    # ------------------------------------------------------------------- checking
    def check_invariants(self) -> None:
        """Every page is in exactly one place: free, cached (count 0, indexed) or live (count > 0)."""
        assert self._lib.ta_alloc_check(self._handle) == 0, _host.message()


def pages_for_len(length: int, page_size: int) -> int:
    return -(-length // page_size)
