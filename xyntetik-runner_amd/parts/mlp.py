"""Gated feed-forward: ``down(act(gate(h)) * up(h))``; act = SiLU is the one activation built
(src/model.c:6399-6407, ``gated_act`` :4451-4452).

``gate`` and ``up`` are kept as one ``[2F, E]`` matrix so that one product makes both;
the reference does the reverse for a checkpoint that stores them fused
(``slice_rows``, src/model.c:238-248).
"""
from __future__ import annotations

from typing import Dict

import torch

from .base import FeedForward, ParamSpec, register_feed_forward


class GatedMLP(FeedForward):
    takes_unscaled_rows = True

    def __init__(self, hidden_size: int, intermediate_size: int, activation: str = "silu", bias: bool = False,
                 gate_name: str = "gate_proj", up_name: str = "up_proj", down_name: str = "down_proj"):
        from ..csrc.ops import GATE_ACTIVATIONS
        if activation not in GATE_ACTIVATIONS:
            raise ValueError(f"gated feed-forward: activation {activation!r} is not built into the kernels "
                             f"(known: {sorted(GATE_ACTIVATIONS)})")
        self.activation = activation
        self.hidden_size, self.intermediate_size = int(hidden_size), int(intermediate_size)
        self.bias = bool(bias)
        self.names = (gate_name, up_name, down_name)
        self.w_gate_up = self.w_down = self.b_gate_up = self.b_down = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        E, F = self.hidden_size, self.intermediate_size
        g, u, d = self.names
        specs = {f"{g}.weight": ParamSpec((F, E)), f"{u}.weight": ParamSpec((F, E)),
                 f"{d}.weight": ParamSpec((E, F))}
        if self.bias:
            specs.update({f"{g}.bias": ParamSpec((F,), role="vector", init="normal"),
                          f"{u}.bias": ParamSpec((F,), role="vector", init="normal"),
                          f"{d}.bias": ParamSpec((E,), role="vector", init="normal")})
        return specs

    def bind(self, tensors, rt) -> None:
        self.rt = rt
        g, u, d = self.names
        # gate rows then up rows, so that one product makes both; in the kernels' own order
        self.w_gate_up = rt.ops.pack_weight(
            torch.cat([tensors[f"{g}.weight"], tensors[f"{u}.weight"]], dim=0).contiguous(), gated=True)
        self.w_down = rt.ops.pack_weight(tensors[f"{d}.weight"])
        if self.bias:
            self.b_gate_up = torch.cat([tensors[f"{g}.bias"], tensors[f"{u}.bias"]]).float().contiguous()
            self.b_down = tensors[f"{d}.bias"].float().contiguous()

    def _hidden(self, ctx, h):
        return self.rt.ops.linear_gated(h, self.w_gate_up, bias=self.b_gate_up, activation=self.activation)

    def forward(self, ctx, h):
        return self.rt.ops.linear(self._hidden(ctx, h), self.w_down, bias=self.b_down)

    def forward_add(self, ctx, h, residual) -> None:
        self.rt.ops.linear(self._hidden(ctx, h), self.w_down, bias=self.b_down, out=residual, accumulate=True)

    def forward_add_norm(self, ctx, h, residual, norm, defer=False):
        fold = norm.fold()
        if fold is None:
            return super().forward_add_norm(ctx, h, residual, norm, defer)
        return self.rt.ops.linear_add_rmsnorm(self._hidden(ctx, h), self.w_down, residual, fold[0], fold[1],
                                              self.rt.dtype, bias=self.b_down, defer=defer)


register_feed_forward("gated_mlp", GatedMLP)
