"""More generality with toy parts defined here only: a feed-forward that routes every token to
one of several experts, a position encoding that is no rotation, an arrangement with a third
norm (after the mixer) and one without a feed-forward.  All are registered from this file,
named by a toy architecture's spec beside the framework's own parts, and replayed through the
framework's step function, cache and trace program in every way of cutting the work.  They
stand for no model of anyone's.
"""
import io
import math

import numpy as np
import pytest
import torch

import plain_llama as P
import traces
from tiny import logit_error, prompt_ids

pytestmark = pytest.mark.gpu

TOY2_CONFIG = {
    "architectures": ["Toy2ForCausalLM"], "hidden_size": 40, "num_attention_heads": 5, "num_key_value_heads": 5,
    "head_dim": 16, "intermediate_size": 56, "expert_size": 24, "num_experts": 3, "vocab_size": 89,
    "wave_amplitude": 0.5, "wave_base": 50.0, "rms_norm_eps": 1e-6, "rope_theta": 500.0,
    "max_position_embeddings": 256,
}


def wave_table(positions, head_dim, base):
    """[T, D]: channel d swings with the position at its own rate."""
    d = np.arange(head_dim, dtype=np.float64)
    return np.sin(np.asarray(positions, dtype=np.float64)[:, None] * base ** (-d / head_dim)[None, :] + 0.3 * d[None, :])


def register_toy2():
    from xyntetik_runner_amd.config import ExecStep, Fields, LayerSpec, ModelSpec, PartSpec, register_architecture
    from xyntetik_runner_amd.parts import (Block, FeedForward, ParamSpec, PositionEncoding, register_block,
                                           register_feed_forward, register_position)

    class SandwichBlock(Block):
        """x += post(mixer(pre(x))); x += feed_forward(norm(x)): three norms, named by the layer's spec."""
        norm_names = ("mixer_norm", "mixer_post_norm", "feed_forward_norm")

        def forward(self, ctx, cache, x):
            n = self.norms
            y = self.mixer.forward(ctx, cache, n["mixer_norm"].forward(ctx, x))
            if y.dtype != torch.float32:
                y = ctx.ops.convert(y, torch.float32)
            ctx.ops.add_(x, n["mixer_post_norm"].forward(ctx, y))
            self.feed_forward.forward_add(ctx, n["feed_forward_norm"].forward(ctx, x), x)

    class MixerOnlyBlock(Block):
        """x += mixer(norm(x)) and nothing else: a layer without a feed-forward."""
        norm_names = ("mixer_norm",)
        needs_feed_forward = False

        def forward(self, ctx, cache, x):
            self.mixer.forward_add(ctx, cache, self.norms["mixer_norm"].forward(ctx, x), x)

    class WavePosition(PositionEncoding):
        """q and k get a position-dependent vector added (the same for every head)."""

        def __init__(self, head_dim, amplitude, base):
            self.D, self.amp, self.base = head_dim, amplitude, base

        def bind(self, tensors, rt):
            self.rt = rt

        def apply(self, ctx, q, k):
            d = torch.arange(self.D, device=q.device, dtype=torch.float64)
            ang = ctx.positions.double()[:, None] * self.base ** (-d / self.D)[None, :] + 0.3 * d[None, :]
            add = (self.amp * torch.sin(ang)).float()[:, None, :]
            q += add
            if k is not None:
                k += add

    class RoutedMLP(FeedForward):
        """Every token goes to the expert its router scores highest, weighted by that
        expert's softmax probability; an expert is a gated MLP of its own."""

        capturable = False      # which experts run is read from the router's result on the host

        def __init__(self, hidden_size, expert_size, num_experts):
            self.E, self.F, self.n = hidden_size, expert_size, num_experts

        def param_specs(self):
            specs = {"router.weight": ParamSpec((self.n, self.E))}
            for e in range(self.n):
                specs[f"experts.{e}.gate_up.weight"] = ParamSpec((2 * self.F, self.E))
                specs[f"experts.{e}.down.weight"] = ParamSpec((self.E, self.F))
            return specs

        def bind(self, tensors, rt):
            self.rt, self.w = rt, tensors

        def forward(self, ctx, h):
            ops = ctx.ops
            logits = ops.linear(h, self.w["router.weight"], out_dtype=torch.float32)     # 32-bit router logits
            prob = torch.softmax(logits, dim=-1)
            top_p, top_e = prob.max(dim=-1)
            out = torch.zeros((h.shape[0], self.E), dtype=torch.float32, device=h.device)
            for e in range(self.n):
                rows = torch.nonzero(top_e == e).flatten()
                if rows.numel() == 0:
                    continue
                he = h.index_select(0, rows).contiguous()
                if h.dtype == torch.bfloat16:
                    mid = ops.linear_swiglu(he, self.w[f"experts.{e}.gate_up.weight"])
                else:
                    mid = ops.silu_mul(ops.linear(he, self.w[f"experts.{e}.gate_up.weight"]))
                y = ops.linear(mid, self.w[f"experts.{e}.down.weight"], out_dtype=torch.float32)
                out.index_copy_(0, rows, y * top_p[rows, None])
            return out.to(h.dtype)

    def parse(raw):
        f = Fields(raw)
        return {k: (f.number(k) if isinstance(TOY2_CONFIG[k], float) else f.integer(k, lo=1, hi=1 << 20))
                for k in TOY2_CONFIG if k != "architectures"}

    def build(c):
        E, D = c["hidden_size"], c["head_dim"]
        norm = lambda p: PartSpec("rmsnorm", {"size": E, "eps": c["rms_norm_eps"]}, prefix=p)
        attn = lambda p, pos: PartSpec("paged_attention", dict(
            hidden_size=E, num_heads=c["num_attention_heads"], num_kv_heads=c["num_key_value_heads"], head_dim=D,
            position=pos), prefix=p)
        wave = PartSpec("toy_wave", {"head_dim": D, "amplitude": c["wave_amplitude"], "base": c["wave_base"]})
        rot = PartSpec("rotary", {"head_dim": D, "theta": c["rope_theta"]})
        layers = [
            LayerSpec(mixer=attn("layers.0.attn.", wave),
                      feed_forward=PartSpec("toy_routed", {"hidden_size": E, "expert_size": c["expert_size"],
                                                           "num_experts": c["num_experts"]}, prefix="layers.0.moe."),
                      norms={"mixer_norm": norm("layers.0.norm1."), "feed_forward_norm": norm("layers.0.norm2.")}),
            LayerSpec(mixer=attn("layers.1.attn.", rot),
                      feed_forward=PartSpec("gated_mlp", {"hidden_size": E, "intermediate_size": c["intermediate_size"]},
                                            prefix="layers.1.mlp."),
                      norms={"mixer_norm": norm("layers.1.norm1."), "mixer_post_norm": norm("layers.1.norm_post."),
                             "feed_forward_norm": norm("layers.1.norm2.")}, block="toy_sandwich"),
            LayerSpec(mixer=attn("layers.2.attn.", rot), norms={"mixer_norm": norm("layers.2.norm1.")},
                      block="toy_mixer_only"),
        ]
        return ModelSpec(
            architecture="Toy2ForCausalLM", hidden_size=E, vocab_size=c["vocab_size"], max_position=c["max_position_embeddings"],
            embedding=PartSpec("token_embedding", {"vocab_size": c["vocab_size"], "hidden_size": E}, prefix="embed."),
            layers=layers, order=[ExecStep(0), ExecStep(1), ExecStep(2)], final_norm=norm("norm."),
            head=PartSpec("linear", {"vocab_size": c["vocab_size"], "hidden_size": E, "tied": False}, prefix="head."))

    register_block("toy_sandwich", SandwichBlock, replace=True)
    register_block("toy_mixer_only", MixerOnlyBlock, replace=True)
    register_position("toy_wave", WavePosition, replace=True)
    register_feed_forward("toy_routed", RoutedMLP, replace=True)
    register_architecture("Toy2ForCausalLM", parse, build, replace=True)


def plain_toy2(cfg, w, tokens):
    E, H, D = cfg["hidden_size"], cfg["num_attention_heads"], cfg["head_dim"]
    T, F = len(tokens), cfg["expert_size"]
    pos = np.arange(T)
    x = w["embed.weight"][tokens].copy()
    for i in range(3):
        p = f"layers.{i}."
        h = P.rmsnorm(x, w[p + "norm1.weight"], cfg["rms_norm_eps"])
        q = (h @ w[p + "attn.q_proj.weight"].T).reshape(T, H, D)
        k = (h @ w[p + "attn.k_proj.weight"].T).reshape(T, H, D)
        v = (h @ w[p + "attn.v_proj.weight"].T).reshape(T, H, D)
        if i == 0:
            add = cfg["wave_amplitude"] * wave_table(pos, D, cfg["wave_base"])[:, None, :]
            q, k = q + add, k + add
        else:
            inv = P.rope_inv_freq(D, cfg["rope_theta"])
            q, k = P.rope(q, pos, inv), P.rope(k, pos, inv)
        a = P.attention(q, k, v, 1 / math.sqrt(D)).reshape(T, H * D) @ w[p + "attn.o_proj.weight"].T
        if i == 1:                       # the arrangement with a norm after the mixer
            a = P.rmsnorm(a, w[p + "norm_post.weight"], cfg["rms_norm_eps"])
        x = x + a
        if i == 2:                       # the arrangement without a feed-forward
            continue
        h = P.rmsnorm(x, w[p + "norm2.weight"], cfg["rms_norm_eps"])
        if i == 0:
            prob = np.stack([P.softmax(row) for row in h @ w[p + "moe.router.weight"].T])
            y = np.zeros_like(x)
            for t in range(T):
                e = int(np.argmax(prob[t]))
                gu = w[p + f"moe.experts.{e}.gate_up.weight"]
                y[t] = prob[t, e] * P.mlp(h[t:t + 1], gu[:F], gu[F:], w[p + f"moe.experts.{e}.down.weight"])[0]
            x = x + y
        else:
            x = x + P.mlp(h, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
    return P.rmsnorm(x, w["norm.weight"], cfg["rms_norm_eps"]) @ w["head.weight"].T


@pytest.fixture(scope="module")
def toy2(tmp_path_factory):
    from xyntetik_runner_amd.weights import write_random_model
    register_toy2()
    d = write_random_model(TOY2_CONFIG, str(tmp_path_factory.mktemp("toy2")), seed=11, std=0.1, norm_jitter=0.1)
    cfg, w = P.load_folder(d)
    reqs = {f"t{i}": prompt_ids(n, cfg["vocab_size"], 70 + i) for i, n in enumerate([45, 12, 70, 33, 21])}
    want = {rid: plain_toy2(cfg, w, toks) for rid, toks in reqs.items()}
    yield d, cfg, w, reqs, want
    from xyntetik_runner_amd.config import unregister_architecture
    from xyntetik_runner_amd.parts import unregister
    unregister_architecture("Toy2ForCausalLM")
    unregister("position", "toy_wave")
    unregister("feed_forward", "toy_routed")
    unregister("block", "toy_sandwich")
    unregister("block", "toy_mixer_only")


def test_the_router_uses_every_expert(toy2):
    """Otherwise the comparison below would say nothing about routing."""
    d, cfg, w, reqs, want = toy2
    counts = np.zeros(cfg["num_experts"], dtype=int)
    for toks in reqs.values():
        x = w["embed.weight"][toks]
        # the router sees layer 0's second norm; its input differs from the embedding, so only the spread is judged here
        scores = P.rmsnorm(x, w["layers.0.norm2.weight"], cfg["rms_norm_eps"]) @ w["layers.0.moe.router.weight"].T
        counts += np.bincount(scores.argmax(-1), minlength=cfg["num_experts"])
    assert (counts > 0).all(), counts


SCHEDULES = {
    "whole": lambda reqs: traces.whole(reqs),
    "tail": lambda reqs: traces.tail_one_by_one(reqs, tail=16),
    "portions": lambda reqs: traces.portions(reqs),
    "mixed": lambda reqs: traces.mixed(reqs, {rid: len(t) - 8 for rid, t in reqs.items()}, max_live=3, seed=5),
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("schedule", list(SCHEDULES))
def test_toy_parts_replay_like_their_plain_counterpart(toy2, tmp_path, dtype, schedule):
    from xyntetik_runner_amd.engine.runner import ModelRunner
    from xyntetik_runner_amd.trace import replay
    d, cfg, w, reqs, want = toy2
    steps = SCHEDULES[schedule](reqs)
    runner = ModelRunner.from_folder(d, dtype=dtype, max_tokens=traces.max_live_tokens(steps, 64), page_size=16,
                                     max_requests=4)
    out = str(tmp_path / "out")
    replay(runner, traces.to_lines(steps), out, report=io.StringIO())
    runner.manager.check()
    assert not runner.manager.requests and runner.manager.free_pages() == runner.manager.pages_per_group
    got = traces.collect(steps, out, cfg["vocab_size"])
    tol = (2e-5, 2e-6) if dtype == "float32" else (2e-2, 3e-3)
    for rid in reqs:
        mx, mean = logit_error(got[rid], want[rid])
        assert mx <= tol[0] and mean <= tol[1], (schedule, rid, mx, mean)
