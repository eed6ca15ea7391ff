"""Picking the next token of every row of a step on the device.

One kernel call takes all rows: greedy rows and sampled rows together.  The host
supplies each sampled row's draw from its request's generator, so a request's tokens
depend on its own seed only, not on what else is in the batch.
"""
from __future__ import annotations

from typing import List, Optional, Sequence

import numpy as np
import torch

from .params import RECENT_WINDOW, SamplerState


class Sampler:
    def __init__(self, ops, device, exempt_ids: Sequence[int] = ()):
        self.ops, self.device = ops, device
        ex = [int(t) for t in exempt_ids]          # (the kernel walks the list, however long)
        self.exempt = torch.tensor(ex, dtype=torch.int32, device=device) if ex else None

    @staticmethod
    def uses_history(states: List[SamplerState]) -> bool:
        """Whether a row's pick depends on the tokens its request got before (a repeat penalty)."""
        return any((not s.params.greedy) and s.params.repeat_penalty != 1.0 for s in states)

    def sample(self, logits: torch.Tensor, states: List[SamplerState]) -> List[int]:
        """``logits [W, V]`` float32 on the device, one state per row -> token ids."""
        if logits.shape[0] == 0:
            return []
        return [int(t) for t in self.launch(logits, states).cpu().tolist()]

    def launch(self, logits: torch.Tensor, states: List[SamplerState]) -> torch.Tensor:
        """The same without waiting for the result: token ids ``[W]`` int32 on the device."""
        W = logits.shape[0]
        assert W == len(states) and W > 0
        all_greedy = all(s.params.greedy for s in states)
        # floats: temp, top_p, min_p, rp, draw ; ints: top_k, n_recent ; window
        need_window = self.uses_history(states)
        nf = 5 * W
        ni = 2 * W + (W * RECENT_WINDOW if need_window else 0)
        host = torch.empty((nf + ni,), dtype=torch.int32, pin_memory=True)
        hf = host[:nf].view(torch.float32).numpy().reshape(5, W)
        hi = host[nf:].numpy()
        for r, s in enumerate(states):
            p = s.params
            hf[0, r] = p.temperature if not p.greedy else 0.0
            hf[1, r] = p.top_p
            hf[2, r] = p.min_p
            hf[3, r] = p.repeat_penalty
            hf[4, r] = 0.0 if p.greedy else s.draw()
            hi[r] = p.top_k
            hi[W + r] = s.n_recent
        if need_window:
            win = hi[2 * W:].reshape(W, RECENT_WINDOW)
            for r, s in enumerate(states):
                win[r, :] = s.recent
        dev = host.to(self.device, non_blocking=True)
        f = dev[:nf].view(torch.float32).view(5, W)
        i = dev[nf:]
        if all_greedy:
            out = self.ops.sample(logits, f[0], f[4])
        else:
            out = self.ops.sample(
                logits, f[0], f[4], top_k=i[:W], top_p=f[1], min_p=f[2], repeat_penalty=f[3],
                recent=i[2 * W:].view(W, RECENT_WINDOW) if need_window else None,
                n_recent=i[W:2 * W] if need_window else None, exempt=self.exempt)
        return out
