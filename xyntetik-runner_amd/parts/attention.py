"""Grouped-query attention over the paged cache.

Per token: ``q = Wq h``, ``k = Wk h``, ``v = Wv h`` (optional biases); the position
encoding rotates q and k; k and v go to the cache (k rotated, v as it is); query head
``h`` reads key/value head ``h // (H / Hk)``; scores are ``(q . k) * scale`` with
``scale = 1/sqrt(head_dim)`` unless given, causal by construction, limited to the last
``window`` keys if the layer has a window; softmax in 32-bit; ``a = Wo o``
(src/model.c:6243-6338, ``attn_heads`` :3548-3589, window bound :6326).

The three input projections are kept as one ``[Q + 2K, E]`` matrix.  A layer that
reads another layer's cache (``kv_shared``) has no key or value projection and writes
nothing (src/model.h:492-494).
"""
from __future__ import annotations

import math
from typing import Dict, Optional

import torch

from .base import KVSpec, Mixer, ParamSpec, make_part, register_mixer

MAX_HEAD_DIM = 256      # the attention and rotation kernels keep a head's channels in registers up to this size


class PagedAttention(Mixer):
    takes_unscaled_rows = True

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 position=None, window: Optional[int] = None, scale: Optional[float] = None,
                 bias: bool = False, out_bias: Optional[bool] = None, kv_shared: bool = False, qk_transform=None,
                 q_name: str = "q_proj", k_name: str = "k_proj", v_name: str = "v_proj",
                 o_name: str = "o_proj"):
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} query heads are not a multiple of {num_kv_heads} key/value heads")
        if window is not None and window < 1:
            raise ValueError(f"attention window {window} must be at least 1")
        if not (1 <= int(head_dim) <= MAX_HEAD_DIM):
            # refused when the model is built, not at its first step
            raise ValueError(f"attention head size {head_dim} is outside what the attention kernels take (1 to {MAX_HEAD_DIM})")
        self.hidden_size, self.num_heads = int(hidden_size), int(num_heads)
        self.num_kv_heads, self.head_dim = int(num_kv_heads), int(head_dim)
        self.window = int(window) if window is not None else None
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(self.head_dim)
        self.bias = bool(bias)
        self.out_bias = self.bias if out_bias is None else bool(out_bias)
        self.kv_shared = bool(kv_shared)
        self.names = (q_name, k_name, v_name, o_name)
        self.position = make_part("position", position) if position is not None else None
        # applied to the 32-bit projections before the position encoding; with one, the projections
        # are written out and the kernels that rotate and cache their own result are not used
        self.qk_transform = make_part("qk_transform", qk_transform) if qk_transform is not None else None
        self.q_size = self.num_heads * self.head_dim
        self.kv_size = self.num_kv_heads * self.head_dim
        self.w_in = self.b_in = self.w_out = self.b_out = None

    # what the cache manager must keep
    def kv_spec(self) -> Optional[KVSpec]:
        return KVSpec(self.num_kv_heads, self.head_dim, self.window)

    def param_specs(self) -> Dict[str, ParamSpec]:
        E, Q, K = self.hidden_size, self.q_size, self.kv_size
        q, k, v, o = self.names
        specs = {f"{q}.weight": ParamSpec((Q, E)), f"{o}.weight": ParamSpec((E, Q))}
        if not self.kv_shared:
            specs[f"{k}.weight"] = ParamSpec((K, E))
            specs[f"{v}.weight"] = ParamSpec((K, E))
        if self.bias:
            specs[f"{q}.bias"] = ParamSpec((Q,), role="vector", init="normal")
            if not self.kv_shared:
                specs[f"{k}.bias"] = ParamSpec((K,), role="vector", init="normal")
                specs[f"{v}.bias"] = ParamSpec((K,), role="vector", init="normal")
        if self.out_bias:
            specs[f"{o}.bias"] = ParamSpec((E,), role="vector", init="normal")
        if self.qk_transform is not None:
            for name, ps in self.qk_transform.param_specs().items():
                if name in specs:
                    raise ValueError(f"the query/key transform names a tensor {name!r} that the attention has itself")
                specs[name] = ps
        return specs

    @property
    def capturable(self) -> bool:
        return ((self.position is None or self.position.capturable)
                and (self.qk_transform is None or self.qk_transform.capturable))

    def bind(self, tensors, rt) -> None:
        self.rt = rt
        if self.position is not None:
            self.position.bind({}, rt)
        if self.qk_transform is not None:
            self.qk_transform.bind({n: tensors[n] for n in self.qk_transform.param_specs()}, rt)
        q, k, v, o = self.names
        H, Hk, D = self.num_heads, self.num_kv_heads, self.head_dim
        mats = [tensors[f"{q}.weight"]]
        if not self.kv_shared:
            mats += [tensors[f"{k}.weight"], tensors[f"{v}.weight"]]
        w_in = torch.cat(mats, dim=0).contiguous() if len(mats) > 1 else mats[0]
        b_in = None
        if self.bias:
            bs = [tensors[f"{q}.bias"]]
            if not self.kv_shared:
                bs += [tensors[f"{k}.bias"], tensors[f"{v}.bias"]]
            b_in = torch.cat([b.float() for b in bs]).contiguous()
        # A rotation that pairs channel j with j + rot/2: the rows of every query and key head go
        # in paired order, so that the product's kernel has both halves of a pair at hand when
        # it rotates its own result (a few decoded tokens); the rotation kernel reads that order too.
        rot = self.position.rotary() if self.position is not None else None
        self.paired = (rot is not None and not rot.interleaved and rot.rotary_dim % 16 == 0 and D % 16 == 0
                       and self.qk_transform is None)      # (a transform sees channels in the checkpoint's order)
        if self.paired:
            from ..csrc.ops import paired_order
            order = paired_order(D, rot.rotary_dim)
            heads = H + (0 if self.kv_shared else Hk)
            rows = [h * D + c for h in range(heads) for c in order] + list(range(heads * D, w_in.shape[0]))
            index = torch.tensor(rows, dtype=torch.int64, device=w_in.device)
            w_in = w_in.index_select(0, index)
            if b_in is not None:
                b_in = b_in.index_select(0, index)
        self.w_in, self.b_in = rt.ops.pack_weight(w_in), b_in
        self.w_out = rt.ops.pack_weight(tensors[f"{o}.weight"])
        if self.out_bias:
            self.b_out = tensors[f"{o}.bias"].float().contiguous()

    def _attend(self, ctx, cache, h):
        ops, rt = self.rt.ops, self.rt
        Q, K, H, Hk, D = self.q_size, self.kv_size, self.num_heads, self.num_kv_heads, self.head_dim
        T = h.shape[0]
        writes = not self.kv_shared and cache.owns
        rot = self.position.rotary() if self.position is not None else None
        table = ctx.block_table(cache.group)
        if (self.position is None or rot is not None) and writes == (not self.kv_shared) and self.qk_transform is None:
            q = ops.project_rope_kv_write(
                h, self.w_in, self.b_in, cache.k if writes else None, cache.v if writes else None, ctx.positions,
                ctx.req_of_token, table, rot.inv_freq if rot else None, H, Hk if writes else 0, D,
                rot.rotary_dim if rot else 0, rot.interleaved if rot else False, rot.mscale if rot else 1.0,
                cache.page_size, paired=self.paired, cs_table=(lambda: self._step_table(ctx, rot)) if rot else None)
        else:
            # a transform or a position encoding of its own works on the 32-bit queries and keys before
            # they are cached; or the keys and values this layer computes are another layer's to store
            proj = ops.linear(h, self.w_in, bias=self.b_in, out_dtype=torch.float32)
            q_in = proj[:, :Q]
            k_in = proj[:, Q:Q + K] if writes else None
            v_in = proj[:, Q + K:Q + 2 * K] if writes else None
            if self.qk_transform is not None:
                self.qk_transform.apply(ctx, q_in.unflatten(1, (H, D)), k_in.unflatten(1, (Hk, D)) if writes else None)
            if self.position is not None and rot is None:
                self.position.apply(ctx, q_in.unflatten(1, (H, D)), k_in.unflatten(1, (Hk, D)) if writes else None)
            q = torch.empty((T, Q), dtype=rt.dtype, device=h.device)
            ops.rope_kv_write(q_in, k_in, v_in, q, cache.k if writes else None, cache.v if writes else None,
                              ctx.positions, ctx.req_of_token, table,
                              rot.inv_freq if rot else None, H, Hk if writes else 0, D,
                              rot.rotary_dim if rot else 0, rot.interleaved if rot else False,
                              rot.mscale if rot else 1.0, cache.page_size, paired=self.paired)
        return ops.attention(q, cache.k, cache.v, ctx, cache.group, H, Hk, D, cache.page_size, self.scale,
                             self.window)

    def _step_table(self, ctx, rot):
        """The step's cosines and sines for this rotation, made once and shared by every layer
        that rotates by the same table (a step context keeps what its parts leave in ``shared``)."""
        shared = getattr(ctx, "shared", None)
        if shared is None:
            return self.rt.ops.rope_table(ctx.positions, rot.inv_freq, rot.mscale)
        key = ("rope_table", rot.table_key if rot.table_key is not None else rot.inv_freq.data_ptr(), rot.mscale)
        table = shared.get(key)
        if table is None:
            table = shared[key] = self.rt.ops.rope_table(ctx.positions, rot.inv_freq, rot.mscale)
        return table

    def forward(self, ctx, cache, h):
        return self.rt.ops.linear(self._attend(ctx, cache, h), self.w_out, bias=self.b_out)

    def forward_add(self, ctx, cache, h, residual) -> None:
        self.rt.ops.linear(self._attend(ctx, cache, h), self.w_out, bias=self.b_out, out=residual, accumulate=True)

    def forward_add_norm(self, ctx, cache, h, residual, norm, defer=False):
        fold = norm.fold()
        if fold is None:
            return super().forward_add_norm(ctx, cache, h, residual, norm, defer)
        return self.rt.ops.linear_add_rmsnorm(self._attend(ctx, cache, h), self.w_out, residual, fold[0], fold[1],
                                              self.rt.dtype, bias=self.b_out, defer=defer)


register_mixer("paged_attention", PagedAttention)
