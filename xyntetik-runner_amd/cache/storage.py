"""The device memory behind the cache manager.

For every entry of the run order that owns a cache: keys ``[pages, Hk, page_size, D]``
and values ``[pages, Hk, D, page_size]`` (values transposed inside a page so that
attention reads several positions of one channel with one load), in the engine's
dtype.  For every entry whose mixer has state of fixed size: ``[slots + 1, *shape]``; row
``null_slot`` (the last) belongs to no request.
Page 0 is the null page.  Nothing is zeroed when a page changes hands: reads are
bounded by a request's length, so a page's old contents are never seen.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Callable, Dict, List, Optional, Union

import torch

from ..parts.base import KVSpec, StateSpec


@dataclass
class LayerCache:
    """What one entry of the run order sees of the cache."""
    group: int                 # which block table of a request applies
    page_size: int
    owns: bool                 # this entry writes keys and values (False: it reads another entry's)
    k: Optional[torch.Tensor]
    v: Optional[torch.Tensor]
    state: Optional[torch.Tensor] = None    # [slots + 1, *shape]; the last row is nobody's


class CacheStorage:
    def __init__(self, kv_specs: List[Optional[KVSpec]], state_specs: List[Optional[StateSpec]],
                 cache_of: List[Optional[int]], page_size: int,
                 pages_per_group: Union[int, Callable[[KVSpec], int]], n_slots: int,
                 dtype: torch.dtype, device: torch.device):
        """``kv_specs[i]``/``state_specs[i]``/``cache_of[i]`` describe entry ``i`` of the run order.
        ``pages_per_group``: one number for every group, or a function of a group's ``KVSpec``
        (a group that keeps a window of keys needs fewer pages than one that keeps them all)."""
        self.page_size, self.n_slots = page_size, n_slots
        sized = pages_per_group if callable(pages_per_group) else (lambda spec: pages_per_group)
        self.null_slot = n_slots
        self.group_specs: List[KVSpec] = []
        self.group_pages: List[int] = []        # usable pages of each group (the null page comes on top)
        self.layers: List[LayerCache] = []
        for i, (kv, st) in enumerate(zip(kv_specs, state_specs)):
            owner = cache_of[i]
            if owner is not None:
                src = self.layers[owner]
                if kv is not None and src.k is not None:
                    okv = kv_specs[owner]
                    if (okv.num_kv_heads, okv.head_dim) != (kv.num_kv_heads, kv.head_dim):
                        raise ValueError(f"run order entry {i} reads the cache of entry {owner}, "
                                         f"whose heads or head size differ")
                    # the owner's window decides which pages exist: a reader that looks further
                    # back would look up pages that were given back
                    if okv.window is not None and (kv.window is None or kv.window > okv.window):
                        raise ValueError(f"run order entry {i} (window {kv.window}) reads the cache of entry {owner}, "
                                         f"which keeps only the last {okv.window} keys")
                self.layers.append(LayerCache(src.group, page_size, False, src.k, src.v, None))
                continue
            group, k, v = -1, None, None
            if kv is not None:
                if kv not in self.group_specs:
                    self.group_specs.append(kv)
                    self.group_pages.append(max(1, int(sized(kv))))
                group = self.group_specs.index(kv)
                n_pages = self.group_pages[group] + 1
                k = torch.zeros((n_pages, kv.num_kv_heads, page_size, kv.head_dim), dtype=dtype, device=device)
                v = torch.zeros((n_pages, kv.num_kv_heads, kv.head_dim, page_size), dtype=dtype, device=device)
            state = None
            if st is not None:
                # one row more than requests: the last is nobody's (rows that pad a recorded step use it)
                state = torch.zeros((n_slots + 1,) + tuple(st.shape), dtype=st.dtype, device=device)
            self.layers.append(LayerCache(group, page_size, True, k, v, state))

    def bytes_per_token(self) -> int:
        total = 0
        for lc in self.layers:
            if lc.owns and lc.k is not None:
                total += 2 * lc.k.shape[1] * lc.k.shape[3] * lc.k.element_size()
        return total
