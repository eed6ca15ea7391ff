"""How many pages each group's pool gets: from a number of tokens, or from the memory that is left.

The reference sizes its cache from a context length, by default the smaller of the model's
training context and 4,096 (src/model.h:516-592, ``-c`` in src/main.c:1523-1529), and allocates it
whole for every sequence slot.  Here the pools are shared by all requests, so the default is what
the card still holds once the weights are bound.  This file is host arithmetic only.
"""
from __future__ import annotations

from typing import List, Optional, Sequence, Tuple

from ..parts.base import KVSpec
from .manager import pages_for_spec


class CacheTooSmall(RuntimeError):
    """The memory that is left for the cache does not hold one request of the model's context."""


def cache_groups(kv_specs: Sequence[Optional[KVSpec]], cache_of: Sequence[Optional[int]]) -> Tuple[List[KVSpec], List[int]]:
    """The groups of a run order and how many of its entries keep a cache of their own in each
    (entries that read another entry's cache add nothing)."""
    specs: List[KVSpec] = []
    owners: List[int] = []
    for kv, of in zip(kv_specs, cache_of):
        if kv is None or of is not None:
            continue
        if kv not in specs:
            specs.append(kv)
            owners.append(0)
        owners[specs.index(kv)] += 1
    return specs, owners


def page_bytes(spec: KVSpec, n_layers: int, page_size: int, element_size: int) -> int:
    """Bytes of one page number of a group: keys and values of all its layers."""
    return 2 * n_layers * spec.num_kv_heads * spec.head_dim * page_size * element_size


def size_pools(specs: Sequence[KVSpec], owners: Sequence[int], page_size: int, element_size: int,
               max_requests: int, max_step_tokens: Optional[int] = None, *, max_tokens: Optional[int] = None,
               budget_bytes: Optional[int] = None, max_model_len: Optional[int] = None) -> List[int]:
    """Pages per group (the null page not counted).

    With ``max_tokens``: what that many tokens need (``pages_for_spec``).  Otherwise from
    ``budget_bytes``: the groups that keep a window take what ``max_requests`` requests and a step of
    ``max_step_tokens`` need, the groups that keep every key share the rest equally in pages, and no
    more than ``max_requests`` requests of ``max_model_len`` tokens could fill.  ``CacheTooSmall`` if
    that is less than one request of ``max_model_len`` tokens.
    """
    if max_tokens is not None:
        return [pages_for_spec(s, page_size, max_tokens, max_requests, max_step_tokens) for s in specs]
    if budget_bytes is None or max_model_len is None:
        raise ValueError("a cache is sized from max_tokens, or from budget_bytes and max_model_len")
    bpp = [page_bytes(s, n, page_size, element_size) for s, n in zip(specs, owners)]
    want = max(1, -(-int(max_model_len) // page_size))          # pages of one request
    step = max_step_tokens if max_step_tokens is not None else max_model_len
    sizes: List[Optional[int]] = []
    left = int(budget_bytes)
    for s, b in zip(specs, bpp):
        if s.window is None:
            sizes.append(None)
            left -= b                                           # the null page
        else:
            n = pages_for_spec(s, page_size, max_requests * int(max_model_len), max_requests, step)
            sizes.append(n)
            left -= (n + 1) * b
    per_page = sum(b for s, b in zip(specs, bpp) if s.window is None)
    pages = want * max_requests
    if per_page:
        pages = min(pages, left // per_page if left > 0 else 0)
    if left < 0 or (per_page and pages < want):
        need = sum(((want if s.window is None else n) + 1) * b for s, b, n in zip(specs, bpp, sizes))
        raise CacheTooSmall(
            f"the cache does not hold one request of {max_model_len} tokens: that takes {need / 2**30:.2f} GiB, "
            f"{max(0, int(budget_bytes)) / 2**30:.2f} GiB are left after the weights; "
            f"lower max_model_len, raise gpu_memory_fraction or give max_tokens")
    return [pages if n is None else n for n in sizes]


def memory_budget(total_bytes: int, free_bytes: int, fraction: float, working_bytes: int) -> int:
    """Bytes the cache may take: ``fraction`` of the card, less what is in use already (weights,
    other processes) and what a step's activations need."""
    if not (0.0 < fraction <= 1.0):
        raise ValueError(f"gpu_memory_fraction {fraction} must be in (0, 1]")
    used = total_bytes - free_bytes
    return int(fraction * total_bytes) - used - int(working_bytes)
