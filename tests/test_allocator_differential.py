"""The C++ page allocator against a plain Python model of it (tests/plain/page_allocator_plain.py), under
random sequences of every operation: after each one, every observable of the two must agree."""
import random

import pytest

from plain import page_allocator_plain as model
from tokenizer_amd.cache import allocator as native

P = 4


def observe(alloc):
    return (alloc.capacity(), alloc.free_count(), alloc.cached_count(), alloc.available(), alloc.live_count(),
            alloc.occupied(), [alloc.refcount(page) for page in range(alloc.capacity())], alloc.all_refcounts_zero(),
            alloc.peak_live, alloc.peak_occupied)


def call(alloc, errors, name, *args):
    """The result of an operation, or the name of the error it raised."""
    try:
        result = getattr(alloc, name)(*args)
    except errors.AllocError as err:
        return type(err).__name__
    return getattr(result, "value", result)        # Release members compare by value


@pytest.mark.parametrize("seed", range(12))
def test_random_operations_agree_with_the_plain_model(seed):
    rng = random.Random(seed)
    capacity = rng.choice([1, 3, 6, 10])
    a, b = native.PageAllocator(capacity, P), model.PageAllocator(capacity, P)
    prompts = [[rng.randrange(3) for _ in range(rng.choice([P, 2 * P, 3 * P, 3 * P + 2]))] for _ in range(4)]
    held: list[list[int]] = []                     # page lists of "requests" that hold pages
    for _ in range(400):
        op = rng.choice(["alloc", "alloc_n", "free", "free", "incref", "publish_prompt", "take_prefix", "publish_one",
                         "find", "reclaim", "double_free", "unknown", "rewind"])
        if op == "alloc":
            got = call(a, native, "alloc"), call(b, model, "alloc")
            if got[0] is not None:
                held.append([got[0]])
        elif op == "alloc_n":
            n = rng.randint(0, 4)
            got = call(a, native, "alloc_n", n), call(b, model, "alloc_n", n)
            if got[0]:
                held.append(list(got[0]))
        elif op == "free" and held:
            pages = held.pop(rng.randrange(len(held)))
            got = [call(a, native, "free_page", p) for p in pages], [call(b, model, "free_page", p) for p in pages]
        elif op == "incref" and held:
            page = rng.choice(rng.choice(held))
            got = call(a, native, "incref", page), call(b, model, "incref", page)
            held.append([page])
        elif op == "publish_prompt" and held:
            pages, prompt = rng.choice(held), rng.choice(prompts)
            got = call(a, native, "publish_prompt_pages", prompt, pages), call(b, model, "publish_prompt_pages", prompt, pages)
        elif op == "take_prefix":
            prompt = rng.choice(prompts)
            got = call(a, native, "take_shared_prefix", prompt), call(b, model, "take_shared_prefix", prompt)
            if got[0]:
                held.append(list(got[0]))
        elif op == "publish_one" and held:
            page, tokens = rng.choice(rng.choice(held)), rng.choice(prompts)[:rng.choice([P, P - 1])]
            parent = rng.choice([0, model.prefix_page_hash(0, prompts[0][:P])])
            got = (call(a, native, "publish_full_page", parent, tokens, page),
                   call(b, model, "publish_full_page", parent, tokens, page))
        elif op == "find":
            tokens, parent_page = rng.choice(prompts)[:P], rng.choice([None, 0, capacity - 1])
            parent = rng.choice([0, model.prefix_page_hash(0, prompts[1][:P])])
            got = (call(a, native, "find_full_page", parent, parent_page, tokens),
                   call(b, model, "find_full_page", parent, parent_page, tokens))
        elif op == "reclaim":
            got = call(a, native, "reclaim_cached"), call(b, model, "reclaim_cached")
        elif op == "double_free":
            page = rng.randrange(capacity)
            if any(page in pages for pages in held):
                continue
            got = call(a, native, "free_page", page), call(b, model, "free_page", page)
        elif op == "unknown":
            page = rng.choice([-1, capacity, capacity + 5])
            got = (call(a, native, "free_page", page), call(a, native, "incref", page)), \
                  (call(b, model, "free_page", page), call(b, model, "incref", page))
        elif op == "rewind":
            mark = (rng.randint(0, capacity), rng.randint(0, capacity))
            got = call(a, native, "rewind_peaks", mark), call(b, model, "rewind_peaks", mark)
        else:
            continue
        assert got[0] == got[1], (op, got)
        assert observe(a) == observe(b), op
        a.check_invariants()
        b.check_invariants()
    assert native.prefix_page_hash(7, [1, 2, 0xFFFFFFFF, 5]) == model.prefix_page_hash(7, [1, 2, 0xFFFFFFFF, 5])
