"""One step's batch: the tokens of every entry flattened on one axis, with the tables kernels need."""
from __future__ import annotations

import dataclasses

import torch


@dataclasses.dataclass
class StepEntry:
    """A request's next tokens in this step and the places among them whose logits are wanted."""
    rid: object
    tokens: list[int]
    want: list[int] = dataclasses.field(default_factory=list)
    token_array: object = dataclasses.field(default=None, repr=False, compare=False)   # `tokens` as an array, once made

    def packed_tokens(self):
        return self.tokens if self.token_array is None else self.token_array


@dataclasses.dataclass
class EntryInfo:
    """Host-side view of one entry, for parts that loop over requests."""
    rid: object
    q_start: int        # first row of the entry on the token axis
    q_len: int
    position: int       # absolute position of its first token (tokens the request held before)
    slot: int           # state slot of the request


def round_up(value: int, step: int) -> int:
    return -(-value // step) * step


def filled_counts(token_counts: list[int], want_counts: list[int]) -> tuple[int, int, int, int, int]:
    """The counts a step's description is filled up to (tokens, entries, wanted places, tiles of sixteen prompt
    tokens, single rows), from the tokens and wanted places of its entries.

    Steps that are nothing but single tokens are left as they are.  Every other step is rounded up a little, with
    parts that do nothing (`CacheManager.pack_batch`): the sizes of a step's launches and the layout of its tables
    depend on these five counts alone, so the mixed steps of a busy server, whose portions and numbers of decoding
    requests differ a little from step to step, fall into a few shapes that come again and again, and a shape that
    comes again replays a captured graph.  Eager steps are filled up in the same way, so a step computes the same,
    bit for bit, whether it is replayed or not.  The steps of the rounding are small where the kernels change with
    the row count (up to 64 rows) and four prompt tiles beyond."""
    tokens, entries, wanted = sum(token_counts), len(token_counts), sum(want_counts)
    single = sum(1 for count in token_counts if count == 1)
    tiles = sum(-(-count // 16) for count in token_counts if count != 1)
    if single == entries:
        return tokens, entries, wanted, tiles, single
    filled_single = round_up(single, 8)
    filled_tokens = round_up(tokens, 8) if tokens <= 64 else round_up(tokens, 64)
    # Entries: the single rows' and, in steps of four, the portions' and one more (a tile that does nothing needs an
    # entry without rows to lie in).  Tiles: as many as that many portions of that many tokens can have at most,
    # whatever their lengths are (a tile that does nothing costs a workgroup that ends at once).
    portions = round_up(entries - single + 1, 4)
    filled_tiles = -(-filled_tokens // 16) + portions
    return filled_tokens, filled_single + portions, round_up(wanted, 8), filled_tiles, filled_single


@dataclasses.dataclass
class StepContext:
    """Everything a part may read about the batch.  Device tensors are int32.  A step's description may be filled up
    with parts that do nothing (`filled_counts`): `n_tokens` and `n_entries` then count those too (they size the
    launches), `entries` lists the real entries only, a token past the real ones has `entry_of_token` -1, position 0
    and slot -1, a single row past the real ones is -1, and the first `n_wanted` of `want_rows` are the real ones."""
    n_tokens: int
    n_entries: int
    token_ids: torch.Tensor          # [T]
    positions: torch.Tensor          # [T] absolute position of each token
    entry_of_token: torch.Tensor     # [T]
    cu_q: torch.Tensor               # [E + 1] first row of each entry, then T
    first_position: torch.Tensor     # [E]
    state_slots: torch.Tensor        # [E]
    want_rows: torch.Tensor          # [W] rows whose logits are wanted
    block_tables: list[torch.Tensor]  # per group [E, P_g]
    slots: list[torch.Tensor]        # per group [T]: page * page_size + offset of each token
    q_tiles: torch.Tensor            # [n_tiles, 2]: (entry, offset) of every 16-token tile of the multi-token entries
    decode_rows: torch.Tensor        # [n_single] rows of the entries that bring one token
    entries: list[EntryInfo]         # host copy
    max_q_len: int
    max_position: int                # largest position in the batch
    page_size: int
    n_wanted: int = -1               # wanted places of the real entries (the leading rows of the step's logits)


def build_context(entries: list[StepEntry], manager, device, table_width: int | None = None,
                  into: tuple | None = None, fill: bool = False) -> StepContext:
    """Lay the entries out on one token axis and gather their tables from the cache manager.

    Pages for the new tokens must already be reserved.  `table_width` fixes the width of every block
    table (wider than needed, padded with -1); `into` = (pinned host tensor, device tensor) of exactly
    the packed size makes the upload land in existing memory, which a captured graph reads.  `fill`: the
    description is filled up to `filled_counts` with parts that do nothing (the engine's steps do; whoever calls a
    part with rows of its own making does not).
    """
    page_size = manager.page_size
    n_groups = len(manager.groups)
    rids = [entry.rid for entry in entries]
    token_lists = [entry.packed_tokens() for entry in entries]
    want_lists = [entry.want for entry in entries]
    padded = filled_counts([len(t) for t in token_lists], [len(w) for w in want_lists]) if fill else None
    if into is not None:
        host, dev = into
    else:
        # The packing itself is the cache manager's (C++); what is needed here is the buffer's size.
        widths = [table_width if table_width is not None else
                  max([1] + [len(manager.table(rid, g)) for rid in rids]) for g in range(n_groups)]
        size = manager.packed_size([len(t) for t in token_lists], [len(w) for w in want_lists], widths, padded)
        host = torch.empty(size, dtype=torch.int32)
        if torch.device(device).type == "cuda":
            host = host.pin_memory()
    total, sizes, widths, info = manager.pack_batch(rids, token_lists, want_lists, host.numpy(), table_width, padded)
    if total != host.numel():
        raise ValueError("the packed batch does not fit the buffers it should land in")
    if into is not None:
        dev.copy_(host, non_blocking=True)
    else:
        dev = host.to(device, non_blocking=True)
    infos = [EntryInfo(rid, row, count, start, slot) for rid, (row, count, start, slot) in zip(rids, info)]
    n_tokens, n_entries = sizes[0], sizes[4]
    views, offset = [], 0
    for size in sizes:
        views.append(dev[offset:offset + size])
        offset += size
    block_tables = [views[10 + 2 * g].reshape(n_entries, widths[g]) for g in range(n_groups)]
    return StepContext(
        n_tokens=n_tokens, n_entries=n_entries, token_ids=views[0], positions=views[1], entry_of_token=views[2],
        cu_q=views[3], first_position=views[4], state_slots=views[5], want_rows=views[6],
        block_tables=block_tables, slots=[views[9 + 2 * g] for g in range(n_groups)],
        q_tiles=views[7].reshape(-1, 2), decode_rows=views[8], entries=infos,
        max_q_len=max((i.q_len for i in infos), default=0),
        max_position=max((i.position + i.q_len - 1 for i in infos), default=0), page_size=page_size,
        n_wanted=sum(len(w) for w in want_lists))
