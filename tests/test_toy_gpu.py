"""The framework's generality, shown with toy parts that live in this file only: a mixer
with fixed-size state of its own, registered as a part and put into a toy architecture
beside the framework's attention (windowed, and a layer that reads another layer's cache),
in a run order that names a layer twice.  Nothing in the framework's files knows of them.
"""
import math

import numpy as np
import pytest
import torch

import plain_llama as P
from tiny import logit_error, prompt_ids

pytestmark = pytest.mark.gpu

TOY_CONFIG = {
    "architectures": ["ToyForCausalLM"], "hidden_size": 48, "num_attention_heads": 3, "num_key_value_heads": 1,
    "head_dim": 16, "intermediate_size": 80, "vocab_size": 101, "window": 6, "ema_size": 20, "ema_decay": 0.75,
    "rms_norm_eps": 1e-5, "rope_theta": 10000.0, "max_position_embeddings": 256,
}


# ----------------------------------------------------------------------------- the toy mixer
def register_toy():
    from xyntetik_runner_amd.config import (ExecStep, Fields, LayerSpec, ModelSpec, PartSpec,
                                            register_architecture)
    from xyntetik_runner_amd.parts import Mixer, ParamSpec, StateSpec, register_mixer

    class EmaMixer(Mixer):
        """s_t = decay * s_{t-1} + (1 - decay) * (W_in h_t);  y_t = W_out s_t.  One state row per request."""

        def __init__(self, hidden_size, state_size, decay):
            self.E, self.S, self.decay = hidden_size, state_size, decay

        def param_specs(self):
            return {"in_proj.weight": ParamSpec((self.S, self.E)), "out_proj.weight": ParamSpec((self.E, self.S))}

        def state_spec(self):
            return StateSpec((self.S,), torch.float32)

        def bind(self, tensors, rt):
            self.rt = rt
            self.w_in, self.w_out = tensors["in_proj.weight"], tensors["out_proj.weight"]

        def forward(self, ctx, cache, h):
            u = ctx.ops.linear(h, self.w_in, out_dtype=torch.float32)            # the framework's kernels
            slots = ctx.slots.long()            # on the device: nothing here looks at data on the host,
            ys, r = [], 0                       # so decode steps of this mixer can be recorded as graphs
            for b, n in enumerate(ctx.q_lens):                                    # the scan itself: plain torch
                row = slots[b:b + 1]
                s = cache.state.index_select(0, row)[0]
                for i in range(n):
                    s = self.decay * s + (1 - self.decay) * u[r + i]
                    ys.append(s)
                cache.state.index_copy_(0, row, s[None])
                r += n
            y = torch.stack(ys).to(h.dtype)
            return ctx.ops.linear(y, self.w_out)

    def parse(raw):
        f = Fields(raw)
        return {k: (f.number(k) if isinstance(TOY_CONFIG[k], float) else f.integer(k, lo=1, hi=1 << 20))
                for k in TOY_CONFIG if k != "architectures"}

    def build(c):
        E = c["hidden_size"]
        norm = lambda p: PartSpec("rmsnorm", {"size": E, "eps": c["rms_norm_eps"]}, prefix=p)
        mlp = lambda p: PartSpec("gated_mlp", {"hidden_size": E, "intermediate_size": c["intermediate_size"]}, prefix=p)
        rot = PartSpec("rotary", {"head_dim": c["head_dim"], "theta": c["rope_theta"]})
        attn = lambda p, **kw: PartSpec("paged_attention", dict(
            hidden_size=E, num_heads=c["num_attention_heads"], num_kv_heads=c["num_key_value_heads"],
            head_dim=c["head_dim"], position=rot, **kw), prefix=p)
        mixers = [attn("layers.0.attn.", window=c["window"]),
                  PartSpec("toy_ema", {"hidden_size": E, "state_size": c["ema_size"], "decay": c["ema_decay"]}, prefix="layers.1.ema."),
                  attn("layers.2.attn.", window=c["window"], kv_shared=True)]
        layers = [LayerSpec(mixer=m, feed_forward=mlp(f"layers.{i}.mlp."),
                            norms={"mixer_norm": norm(f"layers.{i}.norm1."), "feed_forward_norm": norm(f"layers.{i}.norm2.")})
                  for i, m in enumerate(mixers)]
        return ModelSpec(
            architecture="ToyForCausalLM", hidden_size=E, vocab_size=c["vocab_size"], max_position=c["max_position_embeddings"],
            embedding=PartSpec("token_embedding", {"vocab_size": c["vocab_size"], "hidden_size": E}, prefix="embed."),
            layers=layers,
            # layer 0 runs twice (each run has its own cache); layer 2 reads the cache of the first run
            order=[ExecStep(0), ExecStep(1), ExecStep(0), ExecStep(2, cache_of=0)],
            final_norm=norm("norm."), head=PartSpec("linear", {"vocab_size": c["vocab_size"], "hidden_size": E, "tied": True}))

    register_mixer("toy_ema", EmaMixer, replace=True)
    register_architecture("ToyForCausalLM", parse, build, replace=True)


# ----------------------------------------------------------------------------- its plain counterpart
def plain_toy(cfg, w, tokens):
    E, H, Hk, D = cfg["hidden_size"], cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    T = len(tokens)
    inv = P.rope_inv_freq(D, cfg["rope_theta"])
    pos = np.arange(T)
    x = w["embed.weight"][tokens].copy()
    caches = {}

    def attn_layer(x, i, run, shared_from=None):
        p = f"layers.{i}."
        h = P.rmsnorm(x, w[p + "norm1.weight"], cfg["rms_norm_eps"])
        q = P.rope((h @ w[p + "attn.q_proj.weight"].T).reshape(T, H, D), pos, inv)
        if shared_from is None:
            k = P.rope((h @ w[p + "attn.k_proj.weight"].T).reshape(T, Hk, D), pos, inv)
            v = (h @ w[p + "attn.v_proj.weight"].T).reshape(T, Hk, D)
            caches[run] = (k, v)
        else:
            k, v = caches[shared_from]
        o = P.attention(q, k, v, 1 / math.sqrt(D), cfg["window"]).reshape(T, H * D)
        x = x + o @ w[p + "attn.o_proj.weight"].T
        h = P.rmsnorm(x, w[p + "norm2.weight"], cfg["rms_norm_eps"])
        return x + P.mlp(h, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])

    def ema_layer(x, i):
        p = f"layers.{i}."
        h = P.rmsnorm(x, w[p + "norm1.weight"], cfg["rms_norm_eps"])
        u = h @ w[p + "ema.in_proj.weight"].T
        s = np.zeros(cfg["ema_size"])
        ys = []
        for t in range(T):
            s = cfg["ema_decay"] * s + (1 - cfg["ema_decay"]) * u[t]
            ys.append(s)
        x = x + np.stack(ys) @ w[p + "ema.out_proj.weight"].T
        h = P.rmsnorm(x, w[p + "norm2.weight"], cfg["rms_norm_eps"])
        return x + P.mlp(h, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])

    x = attn_layer(x, 0, run=0)
    x = ema_layer(x, 1)
    x = attn_layer(x, 0, run=2)
    x = attn_layer(x, 2, run=3, shared_from=0)
    return P.rmsnorm(x, w["norm.weight"], cfg["rms_norm_eps"]) @ w["embed.weight"].T


@pytest.fixture(scope="module")
def toy(tmp_path_factory):
    from xyntetik_runner_amd.weights import write_random_model
    register_toy()
    d = write_random_model(TOY_CONFIG, str(tmp_path_factory.mktemp("toy")), seed=4, std=0.08, norm_jitter=0.1,
                           vector_dtype="float32")
    cfg, w = P.load_folder(d)
    yield d, cfg, w
    from xyntetik_runner_amd.config import unregister_architecture
    from xyntetik_runner_amd.parts import unregister
    unregister_architecture("ToyForCausalLM")
    unregister("mixer", "toy_ema")


def test_toy_is_built_from_its_config(toy):
    from xyntetik_runner_amd.config import load_config
    from xyntetik_runner_amd.engine.model import Model
    d, cfg, w = toy
    arch, c = load_config(d)
    assert arch.name == "ToyForCausalLM"
    spec = arch.build_spec(c)
    exp = Model.expected_tensors(spec)
    assert "layers.1.ema.in_proj.weight" in exp and "layers.2.attn.k_proj.weight" not in exp     # a reader has no k/v
    assert sorted(exp) == sorted(w)
    m = Model(spec)
    kv, st, of = m.cache_needs()
    assert [k is not None for k in kv] == [True, False, True, True] and [s is not None for s in st] == [False, True, False, False]
    assert of == [None, None, None, 0]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_steps_like_its_plain_counterpart(toy, dtype):
    from xyntetik_runner_amd.engine import ModelRunner, StepEntry
    d, cfg, w = toy
    runner = ModelRunner.from_folder(d, dtype=dtype, max_tokens=192, page_size=4, max_requests=3)
    assert runner.graphs is not None and runner.graphs.usable
    assert len(runner.manager.groups) == 1 and runner.manager.groups[0].spec.window == 6
    assert runner.storage.layers[3].k is runner.storage.layers[0].k and not runner.storage.layers[3].owns
    assert runner.storage.layers[2].k is not runner.storage.layers[0].k
    assert runner.storage.layers[1].state.shape == (3 + 1, 20) and runner.storage.layers[1].k is None   # the last row is nobody's
    reqs = {f"r{i}": prompt_ids(n, 101, 30 + i) for i, n in enumerate([37, 9, 22, 50])}
    want = {k: plain_toy(cfg, w, v) for k, v in reqs.items()}
    got = {k: [] for k in reqs}
    prog = {k: 0 for k in reqs}
    live, pending = [], list(reqs)
    sizes = [5, 1, 9, 2, 1, 1, 13, 1, 3]
    k = 0
    for lc in runner.storage.layers:                      # old state and old keys must never show
        if lc.state is not None:
            lc.state.fill_(float("nan"))
        if lc.k is not None and lc.owns:
            lc.k.fill_(float("nan")); lc.v.fill_(float("nan"))
    while pending or live:
        while pending and len(live) < 3:
            live.append(pending.pop(0))
        entries = []
        for rid in live:
            n = min(sizes[k % len(sizes)], len(reqs[rid]) - prog[rid]); k += 1
            entries.append(StepEntry(rid, reqs[rid][prog[rid]:prog[rid] + n], list(range(n))))
        out = runner.step(entries).cpu().numpy()
        r = 0
        for e in entries:
            n = len(e.tokens)
            got[e.req_id].append(out[r:r + n]); r += n
            prog[e.req_id] += n
            if prog[e.req_id] == len(reqs[e.req_id]):
                runner.finish(e.req_id)
                live.remove(e.req_id)
        runner.manager.check()
        # the window gives pages back: no request ever holds more than window/page_size + 2 pages + its current portion
        for rc in runner.manager.requests.values():
            assert sum(p >= 0 for p in rc.tables[0]) <= 6 // 4 + 2 + 13 // 4 + 1
    assert runner.manager.free_pages() == runner.manager.pages_per_group and runner.manager.slots.n_free == 3
    tol = (2e-5, 2e-6) if dtype == "float32" else (2e-2, 3e-3)
    for rid in reqs:
        mx, mean = logit_error(np.concatenate(got[rid]), want[rid])
        assert mx <= tol[0] and mean <= tol[1], (rid, mx, mean)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_state_through_recorded_decode_steps(toy, dtype):
    """Three requests decode one token a step: the steps are recorded as graphs (a bucket of four
    rows, so one row pads the batch and writes the state row that is nobody's), the mixer's state
    rows are found by the slots on the device, and a request that begins in such a step (its
    prompt is one token) starts from zeroed state although every row held NaN before."""
    from xyntetik_runner_amd.engine import ModelRunner, StepEntry
    d, cfg, w = toy
    runner = ModelRunner.from_folder(d, dtype=dtype, max_tokens=256, page_size=4, max_requests=3)
    for lc in runner.storage.layers:
        if lc.state is not None:
            lc.state.fill_(float("nan"))
        if lc.k is not None and lc.owns:
            lc.k.fill_(float("nan")); lc.v.fill_(float("nan"))
    reqs = {f"r{i}": prompt_ids(n, 101, 60 + i) for i, n in enumerate([45, 38, 41])}
    want = {k: plain_toy(cfg, w, v) for k, v in reqs.items()}
    n0 = {"r0": 5, "r1": 1, "r2": 3}                       # r1 begins inside a recorded step
    got = {k: [] for k in reqs}
    first = [k for k in reqs if n0[k] > 1]
    out = runner.step([StepEntry(k, reqs[k][:n0[k]], list(range(n0[k]))) for k in first]).cpu().numpy()
    r = 0
    for k in first:
        got[k].append(out[r:r + n0[k]]); r += n0[k]
    prog = {k: (n0[k] if k in first else 0) for k in reqs}
    for step in range(36):
        entries = [StepEntry(k, [reqs[k][prog[k]]], [0]) for k in reqs]
        out = runner.step(entries).cpu().numpy()
        for i, k in enumerate(reqs):
            got[k].append(out[i:i + 1]); prog[k] += 1
        runner.manager.check()
    assert runner.graphs.replays >= 30
    null_row = runner.storage.layers[1].state[runner.storage.null_slot]
    assert not torch.isnan(runner.storage.layers[1].state[:3]).any() and null_row.shape == (20,)
    tol = (2e-5, 2e-6) if dtype == "float32" else (2e-2, 3e-3)
    for k in reqs:
        rows = np.concatenate(got[k])
        assert np.isfinite(rows).all()
        mx, mean = logit_error(rows, want[k][:len(rows)])
        assert mx <= tol[0] and mean <= tol[1], (k, mx, mean)


def test_unknown_part_kind_is_a_clear_error():
    from xyntetik_runner_amd.config import PartSpec
    from xyntetik_runner_amd.parts import make_part
    with pytest.raises(ValueError) as e:
        make_part("mixer", PartSpec("no_such_mixer", {}))
    assert "no_such_mixer" in str(e.value) and "paged_attention" in str(e.value)


# ----------------------------------------------------------------------------- windows through captured decode steps
TOYW_CONFIG = {
    "architectures": ["ToyWindowForCausalLM"], "hidden_size": 64, "num_attention_heads": 4, "num_key_value_heads": 2,
    "head_dim": 32, "intermediate_size": 96, "vocab_size": 131, "window": 40, "rms_norm_eps": 1e-5,
    "rope_theta": 10000.0, "max_position_embeddings": 512,
}


def register_toy_window():
    """Two stateless attention layers, the first with a window of 40 keys, the second with all
    keys: two cache groups, and decode steps that a HIP graph can record."""
    from xyntetik_runner_amd.config import ExecStep, Fields, LayerSpec, ModelSpec, PartSpec, register_architecture

    def parse(raw):
        f = Fields(raw)
        return {k: (f.number(k) if isinstance(TOYW_CONFIG[k], float) else f.integer(k, lo=1, hi=1 << 20))
                for k in TOYW_CONFIG if k != "architectures"}

    def build(c):
        E = c["hidden_size"]
        norm = lambda p: PartSpec("rmsnorm", {"size": E, "eps": c["rms_norm_eps"]}, prefix=p)
        rot = PartSpec("rotary", {"head_dim": c["head_dim"], "theta": c["rope_theta"]})
        attn = lambda p, **kw: PartSpec("paged_attention", dict(
            hidden_size=E, num_heads=c["num_attention_heads"], num_kv_heads=c["num_key_value_heads"],
            head_dim=c["head_dim"], position=rot, **kw), prefix=p)
        mlp = lambda p: PartSpec("gated_mlp", {"hidden_size": E, "intermediate_size": c["intermediate_size"]}, prefix=p)
        layers = [LayerSpec(mixer=attn(f"layers.{i}.attn.", window=win), feed_forward=mlp(f"layers.{i}.mlp."),
                            norms={"mixer_norm": norm(f"layers.{i}.norm1."), "feed_forward_norm": norm(f"layers.{i}.norm2.")})
                  for i, win in enumerate([c["window"], None])]
        return ModelSpec(
            architecture="ToyWindowForCausalLM", hidden_size=E, vocab_size=c["vocab_size"],
            max_position=c["max_position_embeddings"],
            embedding=PartSpec("token_embedding", {"vocab_size": c["vocab_size"], "hidden_size": E}, prefix="embed."),
            layers=layers, order=[ExecStep(0), ExecStep(1)], final_norm=norm("norm."),
            head=PartSpec("linear", {"vocab_size": c["vocab_size"], "hidden_size": E, "tied": False}, prefix="head."))

    register_architecture("ToyWindowForCausalLM", parse, build, replace=True)


def plain_toy_window(cfg, w, tokens):
    E, H, Hk, D = cfg["hidden_size"], cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    T = len(tokens)
    inv = P.rope_inv_freq(D, cfg["rope_theta"])
    pos = np.arange(T)
    x = w["embed.weight"][tokens].copy()
    for i, win in enumerate([cfg["window"], None]):
        p = f"layers.{i}."
        h = P.rmsnorm(x, w[p + "norm1.weight"], cfg["rms_norm_eps"])
        q = P.rope((h @ w[p + "attn.q_proj.weight"].T).reshape(T, H, D), pos, inv)
        k = P.rope((h @ w[p + "attn.k_proj.weight"].T).reshape(T, Hk, D), pos, inv)
        v = (h @ w[p + "attn.v_proj.weight"].T).reshape(T, Hk, D)
        x = x + P.attention(q, k, v, 1 / math.sqrt(D), win).reshape(T, H * D) @ w[p + "attn.o_proj.weight"].T
        h = P.rmsnorm(x, w[p + "norm2.weight"], cfg["rms_norm_eps"])
        x = x + P.mlp(h, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
    return P.rmsnorm(x, w["norm.weight"], cfg["rms_norm_eps"]) @ w["head.weight"].T


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_windowed_decoding_through_captured_steps(tmp_path, dtype):
    """Two requests decode far past the window through recorded graphs (bfloat16: the MFMA
    attention, pages of 16): the windowed group's block tables are rewritten every step as pages
    are given back (their entries become -1), the other group's only grow.  Every page starts
    as NaN, so a read of a page that was given back, or beyond a request's length, shows."""
    from xyntetik_runner_amd.config import unregister_architecture
    from xyntetik_runner_amd.engine import ModelRunner, StepEntry
    from xyntetik_runner_amd.weights import write_random_model
    register_toy_window()
    try:
        d = write_random_model(TOYW_CONFIG, str(tmp_path / "toyw"), seed=6, std=0.08, norm_jitter=0.1)
        cfg, w = P.load_folder(d)
        runner = ModelRunner.from_folder(d, dtype=dtype, max_tokens=640, page_size=16, max_requests=2)
        assert runner.graphs.usable and [g.spec.window for g in runner.manager.groups] == [40, None]
        for lc in runner.storage.layers:
            lc.k.fill_(float("nan")); lc.v.fill_(float("nan"))
        reqs = {"a": prompt_ids(300, cfg["vocab_size"], 41), "b": prompt_ids(170, cfg["vocab_size"], 42)}
        want = {k: plain_toy_window(cfg, w, v) for k, v in reqs.items()}
        n0 = {"a": 130, "b": 7}
        got = {k: [] for k in reqs}
        out = runner.step([StepEntry(k, reqs[k][:n0[k]], list(range(n0[k]))) for k in reqs]).cpu().numpy()
        got["a"].append(out[:130]); got["b"].append(out[130:])
        fewest = 99
        for i in range(160):
            entries = [StepEntry(k, [reqs[k][n0[k] + i]], [0]) for k in reqs]
            out = runner.step(entries).cpu().numpy()
            for r, k in enumerate(reqs):
                got[k].append(out[r:r + 1])
            runner.manager.check()
            tabs = runner.manager.get("a").tables
            fewest = min(fewest, sum(p >= 0 for p in tabs[0]))
            assert sum(p >= 0 for p in tabs[0]) <= 40 // 16 + 2 and all(p >= 0 for p in tabs[1])
        assert runner.graphs.replays >= 150 and fewest <= 4
        if dtype == "bfloat16":
            # the windowed layer's work list has fewer key ranges a request than the other layer's
            per_plan = [{key[1]: n for key, n in ctx._plan_splits.items()} for ctx, _, _ in runner.graphs.graphs.values()]
            assert any(sp[40] < sp[None] for sp in per_plan), per_plan
        assert -1 in runner.manager.get("a").tables[0]           # pages were given back while it decoded
        tol = (2e-5, 2e-6) if dtype == "float32" else (2e-2, 3e-3)
        for k in reqs:
            rows = np.concatenate(got[k])
            assert np.isfinite(rows).all()
            mx, mean = logit_error(rows, want[k][:len(rows)])
            assert mx <= tol[0] and mean <= tol[1], (k, mx, mean)
    finally:
        unregister_architecture("ToyWindowForCausalLM")
