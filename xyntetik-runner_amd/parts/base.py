"""Interfaces of the parts a model is put together from.

A part is built from a ``PartSpec`` (its sizes and constants), names the tensors
it needs, is given them by ``bind`` and is then called by the step function.  No
part knows which architecture it is in; an architecture's builder chooses parts
layer by layer.

Families and what each must offer:

* ``Norm``: ``forward(ctx, x, rows=None) -> h``.  ``x`` is the 32-bit residual
  stream ``[T, E]``; ``h`` is in the compute dtype.  ``rows`` (device int32)
  selects rows of ``x``.  ``fold()`` may return ``(weight, eps)`` if the norm is an
  RMSNorm that the product before it may compute (see below).
* ``PositionEncoding``: ``rotary()`` returns the parameters of a rotation that
  the attention kernels apply themselves, or ``None``; then ``apply(ctx, q, k)``
  is called on the 32-bit queries and keys before they are cached.
* ``QKTransform``: ``apply(ctx, q, k)`` on an attention mixer's 32-bit queries and keys, between
  their projection and the position encoding, in place.
* ``Mixer``: ``kv_spec()`` and ``state_spec()`` say what the cache manager must
  keep for it; ``forward(ctx, cache, h) -> y`` returns ``[T, E]`` in the compute
  dtype; ``forward_add(ctx, cache, h, residual)`` adds it into the 32-bit
  residual stream (the default calls ``forward``; a part with a fused epilogue
  overrides it).
* ``FeedForward``: ``forward(ctx, h) -> y`` and ``forward_add(ctx, h, residual)``.
* ``Block``: the arrangement; it names its norms (``norm_names``), may do without a mixer or a
  feed-forward, and ``forward(ctx, cache, x)`` updates ``x`` in place.

Optional, for fewer kernels when a few tokens are decoded: a mixer or feed-forward
may override ``forward_add_norm(..., residual, norm, defer)``, which adds into the
residual stream and returns ``norm`` of the result, so that its last product can do
both (``Ops.linear_add_rmsnorm``).  With ``defer`` the result may be an
``UnscaledRows`` (the rows still lack the division by their root mean square, which
the next product applies to its own result); a caller sets ``defer`` only if the part
that reads the result has ``takes_unscaled_rows`` set, which says that it hands ``h``
to ``Ops.linear`` or ``Ops.linear_gated`` and reads nothing else of it than its
``shape``, ``dtype`` and ``device``.  A block with ``chained`` set takes the result of
its first norm from the block before it and makes the next block's
(``entry_norm()``); every default does the plain thing.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Callable, Dict, Optional, Tuple

import torch


@dataclass(frozen=True)
class ParamSpec:
    """One tensor a part reads from the checkpoint.

    ``role``: "matrix" tensors are kept in the engine's compute dtype; "vector"
    tensors keep 32 bits if the file stores them so (bfloat16 otherwise, in a
    bfloat16 engine); "int" tensors become int32.
    ``init`` tells the random-weights mode what to write: "normal", "ones",
    "ones_jitter" (1 + N(0, jitter)) or "zeros".
    """
    shape: Tuple[int, ...]
    role: str = "matrix"
    init: str = "normal"
    optional: bool = False


@dataclass(frozen=True)
class KVSpec:
    """What a mixer with keys and values asks of the cache manager.

    Layers whose specs are equal share a group: one pool of pages and one block
    table per request.  ``window`` = None keeps every key; a number keeps only
    the pages that the last ``window`` positions touch.
    """
    num_kv_heads: int
    head_dim: int
    window: Optional[int] = None


@dataclass(frozen=True)
class StateSpec:
    """Fixed-size state per request (one slot per live request)."""
    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32


class Part:
    """Common base: parameters by relative name."""

    #: False if ``forward`` reads device data on the host (which kernels it launches then
    #: depends on the data): steps of a model with such a part are never recorded as HIP graphs.
    capturable = True

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {}

    def bind(self, tensors: Dict[str, torch.Tensor], rt: "Runtime") -> None:
        """Take the loaded tensors (already on the device, in the dtype their role asks for)."""
        self.rt = rt
        for k, v in tensors.items():
            setattr(self, "w_" + k.replace(".", "_"), v)


class Norm(Part):
    def forward(self, ctx, x: torch.Tensor, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        raise NotImplementedError

    def fold(self) -> Optional[Tuple[torch.Tensor, float]]:
        """``(weight, eps)`` if this is ``x / sqrt(mean(x^2) + eps) * weight``, which the product
        that writes ``x`` may compute in its own kernel; None for any other norm."""
        return None


@dataclass(frozen=True)
class RotaryParams:
    """A rotation the attention kernels apply to queries and keys themselves."""
    inv_freq: torch.Tensor      # [rotary_dim / 2] float32, on the device
    rotary_dim: int
    interleaved: bool           # False: pairs (j, j + rotary_dim/2); True: pairs (2j, 2j+1)
    mscale: float = 1.0
    table_key: Any = None       # equal keys promise equal tables (layers then share a step's cosines and sines)


class PositionEncoding(Part):
    def rotary(self) -> Optional[RotaryParams]:
        return None

    def apply(self, ctx, q: torch.Tensor, k: Optional[torch.Tensor]) -> None:
        """Transform 32-bit ``q [T, H, D]`` and ``k [T, Hk, D]`` in place (default: nothing)."""
        return None


class QKTransform(Part):
    """Something an attention mixer does to its 32-bit queries and keys between their projection and
    the position encoding (a norm over every head's channels, say: the reference's optional
    ``attn_q_norm`` / ``attn_k_norm``, src/model.c:2838-2852, src/model.h:229-235).  Its tensors are named
    relative to the mixer's prefix."""

    def apply(self, ctx, q: torch.Tensor, k: Optional[torch.Tensor]) -> None:
        """Transform ``q [T, H, D]`` and ``k [T, Hk, D]`` (None in a layer that computes no keys) in
        place; channels are in the checkpoint's order."""
        raise NotImplementedError


class Mixer(Part):
    def kv_spec(self) -> Optional[KVSpec]:
        return None

    def state_spec(self) -> Optional[StateSpec]:
        """Fixed-size state per request: ``cache.state [slots + 1, *shape]``, request ``b`` of a step
        owning row ``ctx.slots[b]`` (on the device; zero when the request first uses it).  A mixer
        that finds its rows through ``ctx.slots`` can be recorded into a HIP graph, where the rows
        that pad a batch use the last state row, which is nobody's; one that reads the slots on
        the host (``ctx.slots_host``, absent in a recorded step) sets ``capturable = False``."""
        return None

    def forward(self, ctx, cache, h: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError

    #: True if ``h`` may be an ``UnscaledRows`` (it only goes into ``Ops.linear``)
    takes_unscaled_rows = False

    def forward_add(self, ctx, cache, h: torch.Tensor, residual: torch.Tensor) -> None:
        ctx.ops.add_(residual, self.forward(ctx, cache, h))

    def forward_add_norm(self, ctx, cache, h, residual: torch.Tensor, norm: Norm, defer: bool = False):
        """``forward_add``, then ``norm`` of the updated residual stream."""
        self.forward_add(ctx, cache, h, residual)
        return norm.forward(ctx, residual)


class FeedForward(Part):
    def forward(self, ctx, h: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError

    #: True if ``h`` may be an ``UnscaledRows`` (it only goes into ``Ops.linear`` or ``Ops.linear_gated``)
    takes_unscaled_rows = False

    def forward_add(self, ctx, h: torch.Tensor, residual: torch.Tensor) -> None:
        ctx.ops.add_(residual, self.forward(ctx, h))

    def forward_add_norm(self, ctx, h, residual: torch.Tensor, norm: Norm, defer: bool = False):
        """``forward_add``, then ``norm`` of the updated residual stream."""
        self.forward_add(ctx, h, residual)
        return norm.forward(ctx, residual)


class Block:
    """An arrangement of a layer's parts around the residual stream: a mixer, a feed-forward
    (an arrangement may do without either) and the norms it names in ``norm_names``."""

    #: the norms this arrangement has, by the names a ``LayerSpec`` gives them
    norm_names: Tuple[str, ...] = ()
    needs_mixer = True
    needs_feed_forward = True

    def __init__(self, mixer: Optional[Mixer], feed_forward: Optional[FeedForward], norms: Dict[str, Norm]):
        kind = type(self).__name__
        if (mixer is None) == self.needs_mixer or (feed_forward is None) == self.needs_feed_forward:
            raise ValueError(f"{kind}: this arrangement has {'a' if self.needs_mixer else 'no'} mixer and "
                             f"{'a' if self.needs_feed_forward else 'no'} feed-forward")
        if set(norms) != set(self.norm_names):
            raise ValueError(f"{kind}: this arrangement has the norms {sorted(self.norm_names)}, "
                             f"the layer names {sorted(norms)}")
        self.mixer, self.feed_forward, self.norms = mixer, feed_forward, dict(norms)

    def parts(self):
        """Every part of the layer by name."""
        out = dict(self.norms)
        if self.mixer is not None:
            out["mixer"] = self.mixer
        if self.feed_forward is not None:
            out["feed_forward"] = self.feed_forward
        return out

    #: True if ``forward`` also takes ``h`` (the result of this block's first norm, made by the
    #: block before) and ``after`` (the next block's ``entry_norm()``), and returns the next
    #: block's ``h`` or None
    chained = False

    def entry_norm(self) -> Optional[Tuple[Norm, bool]]:
        """(the norm this block applies to the residual stream first, whether what reads its
        result takes ``UnscaledRows``), if the block before may compute it; else None."""
        return None

    def forward(self, ctx, cache, x: torch.Tensor) -> None:
        raise NotImplementedError


@dataclass
class Runtime:
    """What every part needs at run time: the device, the dtypes, and the kernels."""
    device: torch.device
    dtype: torch.dtype              # compute dtype: torch.float32 or torch.bfloat16
    ops: Any                        # xyntetik_runner_amd.csrc.ops.Ops

    @property
    def is_fp32(self) -> bool:
        return self.dtype == torch.float32


# --------------------------------------------------------------------------- registries

_REGISTRIES: Dict[str, Dict[str, Callable[..., Any]]] = {
    "norm": {}, "position": {}, "qk_transform": {}, "mixer": {}, "feed_forward": {}, "block": {}, "embedding": {},
    "head": {},
}


def _register(family: str, kind: str, factory: Callable[..., Any], replace: bool = False) -> None:
    reg = _REGISTRIES[family]
    if kind in reg and not replace:
        raise ValueError(f"{family} part {kind!r} is already registered")
    reg[kind] = factory


def register_norm(kind, factory, replace=False):
    _register("norm", kind, factory, replace)


def register_position(kind, factory, replace=False):
    _register("position", kind, factory, replace)


def register_qk_transform(kind, factory, replace=False):
    _register("qk_transform", kind, factory, replace)


def register_mixer(kind, factory, replace=False):
    _register("mixer", kind, factory, replace)


def register_feed_forward(kind, factory, replace=False):
    _register("feed_forward", kind, factory, replace)


def register_block(kind, factory, replace=False):
    _register("block", kind, factory, replace)


def register_embedding(kind, factory, replace=False):
    _register("embedding", kind, factory, replace)


def register_head(kind, factory, replace=False):
    _register("head", kind, factory, replace)


def unregister(family: str, kind: str) -> None:
    _REGISTRIES[family].pop(kind, None)


def make_part(family: str, spec) -> Any:
    """Build the part a ``PartSpec`` describes."""
    reg = _REGISTRIES[family]
    if spec.kind not in reg:
        raise ValueError(f"no {family} part of kind {spec.kind!r}; registered: {sorted(reg)}")
    return reg[spec.kind](**spec.params)


def make_block(kind: str, mixer, feed_forward, norms) -> Block:
    """The arrangement ``kind`` around the given parts (``norms``: name -> norm)."""
    reg = _REGISTRIES["block"]
    if kind not in reg:
        raise ValueError(f"no block arrangement {kind!r}; registered: {sorted(reg)}")
    return reg[kind](mixer, feed_forward, norms)
