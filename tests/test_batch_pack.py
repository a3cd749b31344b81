"""The packed batch description (written by the C++ cache core) against its definition, spelled out here
in plain Python: order and contents of the parts, tiles, rows of single tokens, slots and block tables."""
import random

import numpy as np
import pytest
import torch

from tokenizer_amd.cache import CacheManager
from tokenizer_amd.engine.batch import StepEntry, build_context
from tokenizer_amd.parts.spec import CacheNeed


def needs():
    return [CacheNeed("full", 2, 16), CacheNeed("window", 2, 16, window=20), CacheNeed("none"), CacheNeed("full", 2, 16)]


def expected_parts(manager, entries, table_width):
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
    parts = [token_ids, positions, entry_of, cu_q, first, state, want, tiles, single]
    for g in range(len(manager.groups)):
        tables = [manager.table(entry.rid, g) for entry in entries]
        width = table_width if table_width is not None else max([1] + [len(t) for t in tables])
        slots = []
        for entry, table in zip(entries, tables):
            start = manager.seq_len(entry.rid)
            slots += [table[p // page] * page + p % page for p in range(start, start + len(entry.tokens))]
        flat = []
        for table in tables:
            flat += table[:width] + [-1] * (width - len(table))     # pages held beyond a fixed width are left out
        parts += [slots, flat]
    return parts


@pytest.mark.parametrize("seed", range(6))
@pytest.mark.parametrize("table_width", [None, 12])
def test_packed_batch_matches_its_definition(seed, table_width):
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
    ctx = build_context(entries, manager, "cpu", table_width=table_width)
    parts = expected_parts(manager, entries, table_width)
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
