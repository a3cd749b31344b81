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
    rids = [entry.rid for entry in entries]
    token_lists = [entry.packed_tokens() for entry in entries]
    want_lists = [entry.want for entry in entries]
    if into is not None:
        host, dev = into
    else:
        # The packing itself is the cache manager's (C++); what is needed here is the buffer's size.
        widths = [table_width if table_width is not None else
                  max([1] + [len(manager.table(rid, g)) for rid in rids]) for g in range(n_groups)]
        size = manager.packed_size([len(t) for t in token_lists], [len(w) for w in want_lists], widths)
        host = torch.empty(size, dtype=torch.int32)
        if torch.device(device).type == "cuda":
            host = host.pin_memory()
    total, sizes, widths, info = manager.pack_batch(rids, token_lists, want_lists, host.numpy(), table_width)
    if total != host.numel():
        raise ValueError("the packed batch does not fit the buffers it should land in")
    if into is not None:
        dev.copy_(host, non_blocking=True)
    else:
        dev = host.to(device, non_blocking=True)
    infos = [EntryInfo(rid, row, count, start, slot) for rid, (row, count, start, slot) in zip(rids, info)]
    n_tokens, n_entries = sizes[0], len(entries)
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
