"""Two things a later architecture may need, shown with toy parts defined here only: a transform of
the queries and keys between their projection and the rotation (a norm over every head's channels
with weights of its own), given to the framework's attention as a part and not by editing it; and a
model all of whose layers keep a window of keys, whose pools are sized for the windows and not for
the requests' lengths.  They stand for no model of anyone's.
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

TOY3_CONFIG = {
    "architectures": ["Toy3ForCausalLM"], "hidden_size": 32, "num_attention_heads": 4, "num_key_value_heads": 2,
    "head_dim": 16, "intermediate_size": 48, "vocab_size": 77, "window": 6, "second_window": 9,
    "rms_norm_eps": 1e-5, "qk_norm_eps": 1e-3, "rope_theta": 1000.0, "max_position_embeddings": 8192,
}


def register_toy3():
    from xyntetik_runner_amd.config import ExecStep, Fields, LayerSpec, ModelSpec, PartSpec, register_architecture
    from xyntetik_runner_amd.parts import ParamSpec, QKTransform, register_qk_transform

    class HeadNorm(QKTransform):
        """Every head of q and of k divided by the root mean square of its channels, times a weight
        per channel (one vector for the queries, one for the keys)."""

        def __init__(self, head_dim, eps):
            self.D, self.eps = head_dim, eps

        def param_specs(self):
            return {"q_norm.weight": ParamSpec((self.D,), role="vector", init="ones_jitter"),
                    "k_norm.weight": ParamSpec((self.D,), role="vector", init="ones_jitter")}

        def bind(self, tensors, rt):
            self.rt = rt
            self.wq, self.wk = tensors["q_norm.weight"].float(), tensors["k_norm.weight"].float()

        def apply(self, ctx, q, k):
            for x, w in ((q, self.wq), (k, self.wk)):
                if x is not None:
                    x.copy_(x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + self.eps) * w)

    def parse(raw):
        f = Fields(raw)
        return {k: (f.number(k) if isinstance(TOY3_CONFIG[k], float) else f.integer(k, lo=1, hi=1 << 20))
                for k in TOY3_CONFIG if k != "architectures"}

    def build(c):
        E, D = c["hidden_size"], c["head_dim"]
        norm = lambda p: PartSpec("rmsnorm", {"size": E, "eps": c["rms_norm_eps"]}, prefix=p)
        rot = PartSpec("rotary", {"head_dim": D, "theta": c["rope_theta"]})
        layers = [LayerSpec(
            mixer=PartSpec("paged_attention", dict(
                hidden_size=E, num_heads=c["num_attention_heads"], num_kv_heads=c["num_key_value_heads"], head_dim=D,
                position=rot, window=window, qk_transform=PartSpec("toy_head_norm", {"head_dim": D, "eps": c["qk_norm_eps"]})),
                prefix=f"layers.{i}.attn."),
            feed_forward=PartSpec("gated_mlp", {"hidden_size": E, "intermediate_size": c["intermediate_size"]},
                                  prefix=f"layers.{i}.mlp."),
            norms={"mixer_norm": norm(f"layers.{i}.norm1."), "feed_forward_norm": norm(f"layers.{i}.norm2.")})
            for i, window in enumerate([c["window"], c["second_window"]])]
        return ModelSpec(
            architecture="Toy3ForCausalLM", hidden_size=E, vocab_size=c["vocab_size"], max_position=c["max_position_embeddings"],
            embedding=PartSpec("token_embedding", {"vocab_size": c["vocab_size"], "hidden_size": E}, prefix="embed."),
            layers=layers, order=[ExecStep(0), ExecStep(1)], final_norm=norm("norm."),
            head=PartSpec("linear", {"vocab_size": c["vocab_size"], "hidden_size": E, "tied": True}))

    register_qk_transform("toy_head_norm", HeadNorm, replace=True)
    register_architecture("Toy3ForCausalLM", parse, build, replace=True)


def plain_toy3(cfg, w, tokens, rows=None):
    E, H, Hk, D = cfg["hidden_size"], cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    T = len(tokens)
    pos = np.arange(T)
    inv = P.rope_inv_freq(D, cfg["rope_theta"])
    x = w["embed.weight"][tokens].copy()
    for i, window in enumerate([cfg["window"], cfg["second_window"]]):
        p = f"layers.{i}."
        h = P.rmsnorm(x, w[p + "norm1.weight"], cfg["rms_norm_eps"])
        q = (h @ w[p + "attn.q_proj.weight"].T).reshape(T, H, D)
        k = (h @ w[p + "attn.k_proj.weight"].T).reshape(T, Hk, D)
        v = (h @ w[p + "attn.v_proj.weight"].T).reshape(T, Hk, D)
        # the norm of every head comes before the rotation
        q = P.rmsnorm(q, w[p + "attn.q_norm.weight"], cfg["qk_norm_eps"])
        k = P.rmsnorm(k, w[p + "attn.k_norm.weight"], cfg["qk_norm_eps"])
        q, k = P.rope_all_at_once(q, pos, inv), P.rope_all_at_once(k, pos, inv)
        x = x + P.attention(q, k, v, 1 / math.sqrt(D), window).reshape(T, H * D) @ w[p + "attn.o_proj.weight"].T
        h = P.rmsnorm(x, w[p + "norm2.weight"], cfg["rms_norm_eps"])
        x = x + P.mlp(h, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
    if rows is not None:
        x = x[list(rows)]
    return P.rmsnorm(x, w["norm.weight"], cfg["rms_norm_eps"]) @ w["embed.weight"].T


@pytest.fixture(scope="module")
def toy3(tmp_path_factory):
    from xyntetik_runner_amd.weights import write_random_model
    register_toy3()
    d = write_random_model(TOY3_CONFIG, str(tmp_path_factory.mktemp("toy3")), seed=21, std=0.15, norm_jitter=0.2)
    cfg, w = P.load_folder(d)
    reqs = {f"t{i}": prompt_ids(n, cfg["vocab_size"], 170 + i) for i, n in enumerate([45, 12, 70, 33, 21])}
    want = {rid: plain_toy3(cfg, w, toks) for rid, toks in reqs.items()}
    yield d, cfg, w, reqs, want
    from xyntetik_runner_amd.config import unregister_architecture
    from xyntetik_runner_amd.parts import unregister
    unregister_architecture("Toy3ForCausalLM")
    unregister("qk_transform", "toy_head_norm")


def test_the_head_norm_matters(toy3):
    """The plain counterpart without the norm of the heads gives other logits (so the comparison
    below says something about it), and so does the norm after the rotation with these weights."""
    d, cfg, w, reqs, want = toy3
    ones = dict(w)
    for k in w:
        if "q_norm" in k or "k_norm" in k:
            ones[k] = np.ones_like(w[k])
    other = plain_toy3(cfg, ones, reqs["t1"])
    assert logit_error(other, want["t1"])[1] > 1e-2


SCHEDULES = {
    "whole": lambda reqs: traces.whole(reqs),
    "tail": lambda reqs: traces.tail_one_by_one(reqs, tail=16),
    "portions": lambda reqs: traces.portions(reqs),
    "mixed": lambda reqs: traces.mixed(reqs, {rid: len(t) - 8 for rid, t in reqs.items()}, max_live=3, seed=5),
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("schedule", list(SCHEDULES))
def test_attention_with_a_transform_of_its_queries_and_keys(toy3, tmp_path, dtype, schedule):
    from xyntetik_runner_amd.engine.runner import ModelRunner
    from xyntetik_runner_amd.trace import replay
    d, cfg, w, reqs, want = toy3
    steps = SCHEDULES[schedule](reqs)
    runner = ModelRunner.from_folder(d, dtype=dtype, max_tokens=traces.max_live_tokens(steps, 64), page_size=16,
                                     max_requests=4)
    assert len(runner.manager.groups) == 2                  # two windows, two groups
    out = str(tmp_path / "out")
    replay(runner, traces.to_lines(steps), out, report=io.StringIO())
    runner.manager.check()
    assert runner.manager.all_free()
    if schedule in ("tail", "mixed"):
        assert runner.graphs.replays > 0                    # the transform does not keep decode steps from being recorded
    got = traces.collect(steps, out, cfg["vocab_size"])
    tol = (2e-5, 2e-6) if dtype == "float32" else (2e-2, 3e-3)
    for rid in reqs:
        mx, mean = logit_error(got[rid], want[rid])
        assert mx <= tol[0] and mean <= tol[1], (schedule, rid, mx, mean)


def test_a_long_request_in_pools_sized_for_windows(toy3):
    """Layers that keep the last 6 and 9 keys: their pools hold what two requests' windows and a
    step of 64 tokens need (160 and 160 positions), and a request of 4,096 tokens, which a pool
    of that size could not hold if every key were kept, is admitted, runs in portions and decodes
    the tokens the plain implementation gives."""
    from xyntetik_runner_amd.engine import Engine, ModelRunner
    from xyntetik_runner_amd.sampling import SamplingParams
    d, cfg, w, reqs, want = toy3
    runner = ModelRunner.from_folder(d, dtype="float32", max_tokens=16384, page_size=16, max_requests=2,
                                     max_step_tokens=64)
    sizes = [g.pool.size for g in runner.manager.groups]
    assert sizes == [2 * (1 + 2) + 4, 2 * (1 + 2) + 4]
    assert all(n * 16 < 4096 for n in sizes)
    eng = Engine(runner, max_batched_tokens=64, max_running=2, max_model_len=8192, stop_ids=[])
    long = prompt_ids(4096, cfg["vocab_size"], 5)
    short = prompt_ids(30, cfg["vocab_size"], 6)
    got = eng.generate([long, short], SamplingParams(max_new_tokens=5))
    assert eng.stats.preemptions == 0
    runner.manager.check()
    assert runner.manager.all_free()
    for prompt, new in zip((long, short), got):
        toks = list(prompt)
        for t in new:
            row = plain_toy3(cfg, w, toks, rows=[len(toks) - 1])[0]
            assert int(np.argmax(row)) == t
            toks.append(t)


def test_a_transform_keeps_the_kernels_that_cache_their_own_result_out(toy3):
    """With a transform the projections are written out in 32 bits and in the checkpoint's channel
    order (no paired order), whatever the number of rows."""
    from xyntetik_runner_amd.engine.runner import ModelRunner
    d, cfg, w, reqs, want = toy3
    runner = ModelRunner.from_folder(d, dtype="bfloat16", max_tokens=256, page_size=16, max_requests=2)
    mixers = [block.mixer for block in runner.model.blocks]
    assert all(m.qk_transform is not None and not m.paired for m in mixers)
