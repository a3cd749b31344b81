"""A plain Python page allocator: the model that the C++ allocator of the package is compared with.

Free stack, reference counts, prefix index and a list of cached pages.

Behaviour follows qwen-infer/src/paged.rs:125-519.  Page ids are 0..n-1 and the first
allocation returns 0; the page freed last is handed out next.  A page published under the
hash of its tokens stays out of the free stack when its count falls to zero, so a later
request with the same prefix can take it; `alloc` evicts such pages, oldest first, only
after the free stack is empty.
"""
from __future__ import annotations

import collections
import dataclasses
import enum

_MASK = (1 << 64) - 1


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


def prefix_page_hash(parent: int, tokens) -> int:
    """Chained hash of one full page of token ids (qwen-infer/src/paged.rs:93-100)."""
    value = 0xCBF29CE484222325 ^ parent
    for token in tokens:
        value ^= int(token) & 0xFFFFFFFF
        value = (value * 0x100000001B3) & _MASK
    return value


@dataclasses.dataclass
class _PrefixEntry:
    page: int
    parent_hash: int
    parent_page: int | None
    tokens: tuple[int, ...]


class PageAllocator:
    def __init__(self, num_pages: int, page_size: int = 16):
        if num_pages < 0 or page_size <= 0:
            raise ValueError("num_pages must not be negative and page_size must be positive")
        self.page_size = page_size
        self._capacity = num_pages
        self._free = list(range(num_pages - 1, -1, -1))
        self._refcount = [0] * num_pages
        self._hash_of: list[int | None] = [None] * num_pages
        self._cached: "collections.OrderedDict[int, None]" = collections.OrderedDict()  # oldest first
        self._index: dict[int, _PrefixEntry] = {}
        self._live = 0
        self.peak_live = 0
        self.peak_occupied = 0

    # ------------------------------------------------------------------ counters
    def capacity(self) -> int:
        return self._capacity

    def free_count(self) -> int:
        return len(self._free)

    def cached_count(self) -> int:
        return len(self._cached)

    def available(self) -> int:
        """Pages an allocation can draw on: the free stack plus cached pages."""
        return len(self._free) + len(self._cached)

    def live_count(self) -> int:
        return self._live

    def occupied(self) -> int:
        return self._live + len(self._cached)

    def refcount(self, page: int) -> int | None:
        return self._refcount[page] if 0 <= page < self._capacity else None

    def all_refcounts_zero(self) -> bool:
        return not any(self._refcount)

    def peak_mark(self) -> tuple[int, int]:
        return self.peak_live, self.peak_occupied

    def rewind_peaks(self, mark: tuple[int, int]) -> None:
        self.peak_live = max(mark[0], self._live)
        self.peak_occupied = max(mark[1], self.occupied())

    def _note_peaks(self) -> None:
        self.peak_live = max(self.peak_live, self._live)
        self.peak_occupied = max(self.peak_occupied, self.occupied())

    # ---------------------------------------------------------------- alloc/free
    def alloc(self) -> int | None:
        if self._free:
            page = self._free.pop()
        elif self._cached:
            page, _ = self._cached.popitem(last=False)
            self._unindex(page)
        else:
            return None
        self._refcount[page] = 1
        self._live += 1
        self._note_peaks()
        return page

    def alloc_n(self, n: int) -> list[int] | None:
        """`n` pages or none at all."""
        if self.available() < n:
            return None
        return [self.alloc() for _ in range(n)]

    def free_page(self, page: int) -> Release:
        if not 0 <= page < self._capacity:
            raise UnknownPage(page)
        if self._refcount[page] == 0:
            raise DoubleFree(page)
        self._refcount[page] -= 1
        if self._refcount[page] > 0:
            return Release.SHARED
        self._live -= 1
        if self._hash_of[page] is not None:
            self._cached[page] = None
            self._note_peaks()
            return Release.CACHED
        self._free.append(page)
        self._note_peaks()
        return Release.FREED

    def incref(self, page: int) -> None:
        if not 0 <= page < self._capacity:
            raise UnknownPage(page)
        if self._refcount[page] == 0:
            if page not in self._cached:
                raise DoubleFree(page)
            del self._cached[page]
            self._refcount[page] = 1
            self._live += 1
            self._note_peaks()
            return
        self._refcount[page] += 1

    # -------------------------------------------------------------- prefix index
    def publish_full_page(self, parent_hash: int, tokens, page: int) -> None:
        if len(tokens) != self.page_size:
            raise NotFull(page, len(tokens), self.page_size)
        if not 0 <= page < self._capacity or self._refcount[page] == 0:
            raise UnknownPage(page)
        self._publish_at(prefix_page_hash(parent_hash, tokens), parent_hash, None, tuple(tokens), page)

    def find_full_page(self, parent_hash: int, parent_page: int | None, tokens) -> int | None:
        if len(tokens) != self.page_size:
            return None
        return self._find_at(prefix_page_hash(parent_hash, tokens), parent_hash, parent_page, tuple(tokens))

    def take_shared_prefix(self, tokens) -> list[int]:
        """Published full pages of `tokens`, in order, each with one more holder; stops at the first miss."""
        parent_hash, parent_page, shared, offset = 0, None, [], 0
        size = self.page_size
        while offset + size <= len(tokens):
            chunk = tuple(tokens[offset:offset + size])
            page = self.find_full_page(parent_hash, parent_page, chunk)
            if page is None:
                break
            try:
                self.incref(page)
            except AllocError:
                break
            shared.append(page)
            parent_hash = prefix_page_hash(parent_hash, chunk)
            parent_page = page
            offset += size
        return shared

    def publish_prompt_pages(self, tokens, pages) -> None:
        """Index every full page of `tokens`; pages[i] holds tokens [i*size, (i+1)*size)."""
        size = self.page_size
        parent_hash, parent_page = 0, None
        for index in range(len(tokens) // size):
            if index >= len(pages):
                break
            chunk = tuple(tokens[index * size:(index + 1) * size])
            page = pages[index]
            value = prefix_page_hash(parent_hash, chunk)
            if not 0 <= page < self._capacity or self._refcount[page] == 0:
                break
            self._publish_at(value, parent_hash, parent_page, chunk, page)
            if self._find_at(value, parent_hash, parent_page, chunk) != page:
                break
            parent_hash, parent_page = value, page

    def reclaim_cached(self) -> None:
        while self._cached:
            page, _ = self._cached.popitem(last=False)
            self._unindex(page)
            self._free.append(page)

    def _publish_at(self, value, parent_hash, parent_page, tokens, page) -> bool:
        existing = self._index.get(value)
        if existing is not None:
            return (existing.page == page and existing.parent_hash == parent_hash
                    and existing.parent_page == parent_page and existing.tokens == tokens)
        if self._hash_of[page] is not None:
            return False
        self._index[value] = _PrefixEntry(page, parent_hash, parent_page, tokens)
        self._hash_of[page] = value
        return True

    def _find_at(self, value, parent_hash, parent_page, tokens) -> int | None:
        entry = self._index.get(value)
        if entry and entry.parent_hash == parent_hash and entry.parent_page == parent_page and entry.tokens == tokens:
            return entry.page
        return None

    def _unindex(self, page: int) -> None:
        value = self._hash_of[page]
        self._hash_of[page] = None
        if value is not None and value in self._index and self._index[value].page == page:
            del self._index[value]

    # ------------------------------------------------------------------- checking
    def check_invariants(self) -> None:
        """Every page is in exactly one place: free, cached (count 0, indexed) or live (count > 0)."""
        seen = collections.Counter(self._free)
        assert all(count == 1 for count in seen.values()), "a page is on the free stack twice"
        for page in range(self._capacity):
            places = (page in seen) + (page in self._cached) + (self._refcount[page] > 0)
            assert places == 1, f"page {page} is in {places} places"
            if page in self._cached:
                assert self._hash_of[page] is not None
        assert self._live == sum(1 for count in self._refcount if count > 0)


def pages_for_len(length: int, page_size: int) -> int:
    return -(-length // page_size)
