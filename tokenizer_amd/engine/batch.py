"""One step's batch: the tokens of every entry flattened on one axis, with the tables kernels need."""
from __future__ import annotations

import dataclasses

import numpy as np
import torch


@dataclasses.dataclass
class StepEntry:
    """A request's next tokens in this step and the places among them whose logits are wanted."""
    rid: object
    tokens: list[int]
    want: list[int] = dataclasses.field(default_factory=list)


@dataclasses.dataclass
class EntryInfo:
    """Host-side view of one entry, for parts that loop over requests."""
    rid: object
    q_start: int        # first row of the entry on the token axis
    q_len: int
    position: int       # absolute position of its first token (tokens the request held before)
    slot: int           # state slot of the request


@dataclasses.dataclass
class StepContext:
    """Everything a part may read about the batch.  Device tensors are int32."""
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


def build_context(entries: list[StepEntry], manager, device, table_width: int | None = None,
                  into: tuple | None = None) -> StepContext:
    """Lay the entries out on one token axis and gather their tables from the cache manager.

    Pages for the new tokens must already be reserved.  `table_width` fixes the width of every block
    table (wider than needed, padded with -1); `into` = (pinned host tensor, device tensor) of exactly
    the packed size makes the upload land in existing memory, which a captured graph reads.
    """
    page_size = manager.page_size
    n_groups = len(manager.groups)
    token_ids, positions, entry_of_token, want_rows = [], [], [], []
    cu_q, first_position, state_slots, infos = [0], [], [], []
    slots = [[] for _ in range(n_groups)]
    tables = [[] for _ in range(n_groups)]
    for index, entry in enumerate(entries):
        start = manager.seq_len(entry.rid)
        count = len(entry.tokens)
        row0 = len(token_ids)
        token_ids.extend(entry.tokens)
        positions.extend(range(start, start + count))
        entry_of_token.extend([index] * count)
        want_rows.extend(row0 + w for w in entry.want)
        cu_q.append(row0 + count)
        first_position.append(start)
        state_slots.append(manager.slot(entry.rid))
        infos.append(EntryInfo(entry.rid, row0, count, start, manager.slot(entry.rid)))
        for g in range(n_groups):
            table = manager.table(entry.rid, g)
            tables[g].append(table)
            for p in range(start, start + count):
                page = table[p // page_size]
                if page < 0:
                    raise RuntimeError(f"request {entry.rid!r} writes position {p} into a page it gave back")
                slots[g].append(page * page_size + p % page_size)
    q_tiles, decode_rows = [], []
    for index, info in enumerate(infos):
        if info.q_len == 1:
            decode_rows.append(info.q_start)
        else:
            for offset in range(0, info.q_len, 16):
                q_tiles.extend((index, offset))
    n_tokens, n_entries = len(token_ids), len(entries)
    widths = [max(1, max((len(t) for t in tables[g]), default=1)) for g in range(n_groups)]
    if table_width is not None:
        if any(width > table_width for width in widths):
            raise ValueError("a block table is wider than the fixed width")
        widths = [table_width] * n_groups
    parts = [token_ids, positions, entry_of_token, cu_q, first_position, state_slots, want_rows, q_tiles,
             decode_rows]
    for g in range(n_groups):
        parts.append(slots[g])
        flat = np.full((n_entries, widths[g]), -1, dtype=np.int32)
        for row, table in enumerate(tables[g]):
            flat[row, :len(table)] = table
        parts.append(flat.reshape(-1))
    sizes = [len(p) for p in parts]
    packed = np.concatenate([np.asarray(p, dtype=np.int32).reshape(-1) for p in parts]) if sum(sizes) else \
        np.zeros(0, dtype=np.int32)
    if into is not None:
        host, dev = into
        if host.numel() != packed.size:
            raise ValueError("the packed batch does not fit the buffers it should land in")
        host.numpy()[:] = packed
        dev.copy_(host, non_blocking=True)
    else:
        host = torch.from_numpy(packed)
        if torch.device(device).type == "cuda":
            host = host.pin_memory()
        dev = host.to(device, non_blocking=True)
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
        max_position=max((i.position + i.q_len - 1 for i in infos), default=0), page_size=page_size)
