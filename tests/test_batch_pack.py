"""The packed batch description (written by the C++ cache core) against its definition, spelled out here
in plain Python: order and contents of the parts, tiles, rows of single tokens, slots and block tables."""
import random

import numpy as np
import pytest
import torch

from tokenizer_amd.cache import CacheManager
from tokenizer_amd.engine.batch import StepEntry, build_context, filled_counts
from tokenizer_amd.parts.spec import CacheNeed


def needs():
    return [CacheNeed("full", 2, 16), CacheNeed("window", 2, 16, window=20), CacheNeed("none"), CacheNeed("full", 2, 16)]


def expected_parts(manager, entries, table_width, filled=None):
    """The parts of a step's description; `filled`: the counts (tokens, entries, wanted places, tiles, single rows) it
    is filled up to with parts that do nothing."""
    page = manager.page_size
    token_ids, positions, entry_of, cu_q, first, state, want, tiles, single = [], [], [], [0], [], [], [], [], []
    for e, entry in enumerate(entries):
        start, count, row0 = manager.seq_len(entry.rid), len(entry.tokens), len(token_ids)
        token_ids += entry.tokens
        positions += range(start, start + count)
        entry_of += [e] * count
        want += [row0 + w for w in entry.want]
        cu_q.append(row0 + count)
        first.append(start)
        state.append(manager.slot(entry.rid))
        if count == 1:
            single.append(row0)
        else:
            for offset in range(0, count, 16):
                tiles += [e, offset]
    real_tokens, real_entries = len(token_ids), len(entries)
    more_tokens = more_entries = 0
    if filled is not None:
        n_tokens, n_entries, n_want, n_tiles, n_single = filled
        more_tokens, more_entries = n_tokens - real_tokens, n_entries - real_entries
        token_ids += [0] * more_tokens                            # a token of no request: id 0 at position 0,
        positions += [0] * more_tokens
        entry_of += [-1] * more_tokens                            # no entry
        cu_q += [real_tokens] * more_entries                      # an entry without rows
        first += [0] * more_entries
        state += [0] * more_entries
        want += [0] * (n_want - len(want))                        # a wanted place nobody looks at: row 0
        tiles += [real_entries, 0] * (n_tiles - len(tiles) // 2)  # a tile in the first entry without rows
        single += [-1] * (n_single - len(single))                 # no row
    parts = [token_ids, positions, entry_of, cu_q, first, state, want, tiles, single]
    for g in range(len(manager.groups)):
        tables = [manager.table(entry.rid, g) for entry in entries]
        width = table_width if table_width is not None else max([1] + [len(t) for t in tables])
        slots = []
        for entry, table in zip(entries, tables):
            start = manager.seq_len(entry.rid)
            slots += [table[p // page] * page + p % page for p in range(start, start + len(entry.tokens))]
        slots += [-1] * more_tokens                               # and no slot
        flat = []
        for table in tables:
            flat += table[:width] + [-1] * (width - len(table))     # pages held beyond a fixed width are left out
        flat += [-1] * (width * more_entries)
        parts += [slots, flat]
    return parts


@pytest.mark.parametrize("seed", range(6))
@pytest.mark.parametrize("table_width", [None, 12])
@pytest.mark.parametrize("fill", [False, True])
def test_packed_batch_matches_its_definition(seed, table_width, fill):
    rng = random.Random(seed)
    manager = CacheManager(needs(), num_pages=40, page_size=16, max_requests=5)
    rids = ["a", 7, ("t", 1), 12345678901]                    # names, small integers and large ones alike
    lengths = {}
    for rid in rids:
        manager.add_request(rid)
        held = rng.choice([0, 0, 3, 16, 37, 50])
        if held:
            assert manager.reserve(rid, held)
            manager.advance(rid, held)                         # the window group gives pages back here
        lengths[rid] = held
    entries = []
    for rid in rng.sample(rids, rng.randint(1, len(rids))):
        count = rng.choice([1, 1, 2, 15, 16, 17, 40])
        tokens = [rng.randrange(1000) for _ in range(count)]
        want = sorted(rng.sample(range(count), rng.randint(0, min(3, count))))
        assert manager.reserve(rid, lengths[rid] + count)
        entries.append(StepEntry(rid, tokens, want))
    ctx = build_context(entries, manager, "cpu", table_width=table_width, fill=fill)
    filled = filled_counts([len(e.tokens) for e in entries], [len(e.want) for e in entries]) if fill else None
    parts = expected_parts(manager, entries, table_width, filled)
    if fill:
        assert (ctx.n_tokens, ctx.n_entries) == filled[:2] and ctx.n_wanted == sum(len(e.want) for e in entries)
    got = [ctx.token_ids, ctx.positions, ctx.entry_of_token, ctx.cu_q, ctx.first_position, ctx.state_slots,
           ctx.want_rows, ctx.q_tiles.reshape(-1), ctx.decode_rows]
    for g in range(len(manager.groups)):
        got += [ctx.slots[g], ctx.block_tables[g].reshape(-1)]
    assert len(got) == len(parts)
    for index, (have, want) in enumerate(zip(got, parts)):
        assert have.dtype == torch.int32 and have.tolist() == list(want), index
    assert [(i.rid, i.q_start, i.q_len, i.position, i.slot) for i in ctx.entries] == \
        [(e.rid, parts[3][k], len(e.tokens), manager.seq_len(e.rid), manager.slot(e.rid)) for k, e in enumerate(entries)]
    assert ctx.max_q_len == max(len(e.tokens) for e in entries)
    assert ctx.max_position == max(manager.seq_len(e.rid) + len(e.tokens) - 1 for e in entries)
    manager.check_invariants()


@pytest.mark.parametrize("seed", range(8))
def test_the_next_decode_steps_description_is_what_packing_it_again_gives(seed):
    """A step of single tokens, every request then one token further, packed again: the same as what
    `next_decode_description` makes of the first description (the token ids aside), which is what the device is
    left with when a decode graph ends with `Ops.argmax_next_step`.  Where a request needs a page it does not hold
    yet, or a window gives one back, the two differ, and the engine uploads."""
    from tokenizer_amd.engine.engine import next_decode_description
    rng = random.Random(seed)
    manager = CacheManager(needs(), num_pages=60, page_size=16, max_requests=6)
    n_groups, width = len(manager.groups), 8
    rids = list(range(rng.randint(1, 6)))
    for rid in rids:
        manager.add_request(rid)
        held = rng.choice([1, 3, 15, 16, 31, 47, 60])
        assert manager.reserve(rid, held + 1)
        manager.advance(rid, held)

    def packed():
        entries = [StepEntry(rid, [rng.randrange(1000)], [0]) for rid in rids]
        return build_context(entries, manager, "cpu", table_width=width)

    def flat(ctx):
        parts = [ctx.token_ids, ctx.positions, ctx.entry_of_token, ctx.cu_q, ctx.first_position, ctx.state_slots,
                 ctx.want_rows, ctx.q_tiles.reshape(-1), ctx.decode_rows]
        for g in range(n_groups):
            parts += [ctx.slots[g], ctx.block_tables[g].reshape(-1)]
        return np.concatenate([part.numpy() for part in parts])

    for _ in range(20):
        before = flat(packed())
        tables = [[list(manager.table(rid, g)) for rid in rids] for g in range(n_groups)]
        for rid in rids:
            manager.advance(rid, manager.seq_len(rid) + 1)          # the step ran
            assert manager.reserve(rid, manager.seq_len(rid) + 1)   # pages for the next one
        predicted = next_decode_description(before, len(rids), 16, width, n_groups)
        again = flat(packed())
        same_tables = tables == [[list(manager.table(rid, g)) for rid in rids] for g in range(n_groups)]
        n = len(rids)
        assert np.array_equal(predicted[n:], again[n:]) == same_tables
        if not same_tables:
            # A new page or one given back: everything but the tables and the slots that hang on them still agrees.
            assert np.array_equal(predicted[n:8 * n + 1], again[n:8 * n + 1])
    manager.check_invariants()


def test_a_fixed_width_leaves_out_pages_beyond_the_steps_last_token():
    """A prompt's pages are reserved whole while its first portions run: the request's table is then wider than a
    step's fixed width needs to be, and only the pages up to the step's last token are written."""
    manager = CacheManager([CacheNeed("full", 2, 16)], num_pages=40, page_size=16, max_requests=2)
    manager.add_request("a")
    assert manager.reserve("a", 200)                               # thirteen pages
    entry = StepEntry("a", list(range(32)), [31])
    ctx = build_context([entry], manager, "cpu", table_width=4)
    assert ctx.block_tables[0].tolist() == [manager.table("a", 0)[:4]]
    manager.advance("a", 32)
    ctx = build_context([StepEntry("a", list(range(32)), [31])], manager, "cpu", table_width=4)
    assert ctx.block_tables[0].tolist() == [manager.table("a", 0)[:4]] and ctx.positions.tolist() == list(range(32, 64))
    manager.advance("a", 64)
    with pytest.raises(ValueError, match="wider"):                 # tokens 64..95 need a fifth and a sixth page
        build_context([StepEntry("a", list(range(32)), [31])], manager, "cpu", table_width=4)


def test_packing_refuses_what_does_not_fit():
    manager = CacheManager(needs(), num_pages=40, page_size=16, max_requests=3)
    manager.add_request("a")
    assert manager.reserve("a", 40)
    entry = StepEntry("a", list(range(40)), [39])
    with pytest.raises(ValueError, match="wider"):
        build_context([entry], manager, "cpu", table_width=2)
    with pytest.raises(KeyError):
        build_context([StepEntry("nobody", [1], [0])], manager, "cpu")
    host = torch.zeros(10, dtype=torch.int32)
    with pytest.raises(ValueError, match="fit"):
        build_context([entry], manager, "cpu", into=(host, host.clone()))
    # A window group has given the first pages back: writing there again is refused.
    manager.advance("a", 40)
    manager.add_request("b")
    assert manager.reserve("b", 64)
    manager.advance("b", 64)
    out = np.zeros(4096, dtype=np.int32)
    with pytest.raises(RuntimeError, match="too few pages"):
        manager.pack_batch(["b"], [[5]], [[0]], out)                                   # position 64 has no page yet
    assert manager.reserve("b", 65)
    total, sizes, widths, info = manager.pack_batch(["b"], [[5]], [[0]], out)
    assert sizes[0] == 1 and info == [[0, 1, 64, manager.slot("b")]]
    assert manager.table("b", 1)[:2] == [-1, -1]                                       # behind the window of 20


def test_the_counts_a_step_is_filled_up_to():
    """Steps of single tokens stay as they are; any other step is rounded up to counts that steps which differ a
    little share: always room for one entry without rows (where a tile that does nothing lies), tokens in steps of 8
    up to 64 (where the kernels change with the row count) and of 64 beyond."""
    assert filled_counts([1, 1, 1], [1, 1, 1]) == (3, 3, 3, 0, 3)
    assert filled_counts([1], [0]) == (1, 1, 0, 0, 1)
    assert filled_counts([5], [5]) == (8, 4, 8, 5, 0)
    assert filled_counts([2, 1], [0, 1]) == (8, 12, 8, 5, 8)
    assert filled_counts([137, 1, 1, 1], [1, 1, 1, 1]) == (192, 12, 8, 16, 8)
    assert filled_counts([140] + [1] * 3, [0] + [1] * 3) == filled_counts([131, 20] + [1] * 5, [1, 0] + [1] * 5)
    assert filled_counts([448] + [1] * 64, [1] * 65) == filled_counts([430, 9, 11] + [1] * 62, [1, 1, 1] + [1] * 62) \
        == (512, 68, 72, 36, 64)
    # Filled counts are never below the real ones, whatever the batch.
    rng = random.Random(1)
    for _ in range(300):
        counts = [rng.choice([1, 1, 1, 2, 15, 16, 17, 64, 300]) for _ in range(rng.randint(1, 70))]
        wants = [rng.randint(0, min(3, c)) for c in counts]
        tokens, entries, wanted, tiles, single = filled_counts(counts, wants)
        real_tiles = sum(-(-c // 16) for c in counts if c != 1)
        real_single = sum(1 for c in counts if c == 1)
        assert tokens >= sum(counts) and wanted >= sum(wants) and tiles >= real_tiles and single >= real_single
        assert entries >= len(counts) and (entries > len(counts) or real_single == len(counts))


def test_counts_below_the_batchs_are_refused():
    manager = CacheManager([CacheNeed("full", 2, 16)], num_pages=8, page_size=16, max_requests=2)
    manager.add_request("a")
    assert manager.reserve("a", 20)
    out = np.zeros(4096, dtype=np.int32)
    for too_small in ((19, 2, 0, 4, 0), (24, 1, 0, 4, 0), (24, 2, 0, 1, 0)):      # (more tiles than real ones need an entry more)
        with pytest.raises(ValueError, match="smaller"):
            manager.pack_batch(["a"], [list(range(20))], [[]], out, None, too_small)
    total, sizes, _, _ = manager.pack_batch(["a"], [list(range(20))], [[]], out, None, (24, 2, 8, 4, 0))
    assert sizes[:9] == [24, 24, 24, 3, 2, 2, 8, 8, 0]
