"""Device memory of the cache: pages of keys and values per group, and per-request state slots."""
from __future__ import annotations

import torch

from .manager import CacheManager

_STATE_DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16, "int32": torch.int32}


class CachePools:
    """For group g: `pages[g]` of shape [layers in g, 2, num_pages, n_kv, page_size * d] (keys at 0, values
    at 1) in the compute dtype.  Inside a page keys are laid out [page_size, d] and values transposed,
    [d, page_size] (the layout the matrix-core attention kernels read).  For a layer with fixed-size
    state: `states[layer]` of shape [max_requests, *state_shape]."""

    def __init__(self, manager: CacheManager, needs, dtype: torch.dtype, device):
        self.manager = manager
        self.pages = []
        for group in manager.groups:
            need = group.need
            per_layer = manager.num_pages * need.n_kv_heads * manager.page_size * need.head_dim
            if per_layer >= 2 ** 31:
                # The attention kernels count a layer's keys (and its values) with 32 bits.
                raise ValueError(f"{manager.num_pages} pages of {manager.page_size} tokens are {per_layer} key elements "
                                 f"a layer; the kernels address fewer than 2^31 (at most "
                                 f"{(2 ** 31 - 1) // (need.n_kv_heads * manager.page_size * need.head_dim)} pages here)")
            self.pages.append(torch.zeros((len(group.layers), 2, manager.num_pages, need.n_kv_heads,
                                           manager.page_size * need.head_dim), dtype=dtype, device=device))
        self.states = {}
        for layer, need in enumerate(needs):
            if need.state_shape is not None:
                self.states[layer] = torch.zeros((manager.max_requests, *need.state_shape),
                                                 dtype=_STATE_DTYPES[need.state_dtype], device=device)

    def layer_pages(self, layer: int):
        """(keys [num_pages, n_kv, page_size, d], values [num_pages, n_kv, d, page_size]) of one layer,
        or (None, None)."""
        group = self.manager.group_of_layer[layer]
        if group is None:
            return None, None
        need = self.manager.groups[group].need
        index = self.manager.groups[group].layers.index(layer)
        pages, page_size = self.pages[group], self.manager.page_size
        shape = (self.manager.num_pages, need.n_kv_heads)
        return (pages[index, 0].view(*shape, page_size, need.head_dim),
                pages[index, 1].view(*shape, need.head_dim, page_size))

    def bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in self.pages) + \
            sum(t.numel() * t.element_size() for t in self.states.values())

    def poison(self, value: float = float("nan")) -> None:
        """Fill every page with a value that shows if a kernel reads what no request wrote."""
        for tensor in self.pages:
            tensor.fill_(value)
