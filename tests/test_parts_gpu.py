"""Each part alone on the GPU against the plain implementation's function for it, at
sizes that are not the tiny models', in both dtypes."""
import math

import numpy as np
import pytest
import torch

import plain_llama as P
from test_kernels_gpu import FakeCtx, scatter_pages

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}
TOL = {"float32": 3e-6, "bfloat16": 1.5e-2}


@pytest.fixture(scope="module")
def rt_for():
    from xyntetik_runner_amd.csrc.ops import load_ops
    from xyntetik_runner_amd.parts import Runtime
    ops = load_ops()
    return lambda dt: Runtime(torch.device(DEV), DT[dt], ops)


def rel(got, want):
    want = np.asarray(want, dtype=np.float64)
    got = got.detach().double().cpu().numpy()
    return np.abs(got - want).max() / max(np.abs(want).max(), 1e-30)


def bf(x):
    """Round a float64 array to bfloat16 values (what the engine's tensors hold)."""
    return torch.tensor(x, dtype=torch.float32).bfloat16().double().numpy()


class Ctx:
    def __init__(self, ops):
        self.ops = ops


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
def test_rmsnorm_part(rt_for, dt):
    from xyntetik_runner_amd.parts import make_part
    from xyntetik_runner_amd.config import PartSpec
    rt = rt_for(dt)
    rng = np.random.default_rng(0)
    E = 200
    part = make_part("norm", PartSpec("rmsnorm", {"size": E, "eps": 3e-4}))
    assert part.param_specs()["weight"].shape == (E,) and part.param_specs()["weight"].role == "vector"
    w = 1 + 0.2 * rng.normal(size=E)
    x = rng.normal(size=(6, E)) * 2
    for wdt in (torch.float32, torch.bfloat16):
        wt = torch.tensor(w, dtype=torch.float32).to(wdt).to(DEV)
        part.bind({"weight": wt}, rt)
        got = part.forward(Ctx(rt.ops), torch.tensor(x, dtype=torch.float32, device=DEV))
        assert got.dtype == DT[dt]
        assert rel(got, P.rmsnorm(x.astype(np.float32).astype(np.float64), wt.double().cpu().numpy(), 3e-4)) < TOL[dt]


def test_rotary_part_tables(rt_for):
    from xyntetik_runner_amd.parts import make_part, rotary_inv_freq
    from xyntetik_runner_amd.config import PartSpec
    sc = {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
          "original_max_position_embeddings": 32}
    for D, theta, scaling, rot in [(32, 500000.0, sc, None), (64, 10000.0, None, 32),
                                   (48, 1000.0, {"rope_type": "linear", "factor": 2.0}, None)]:
        part = make_part("position", PartSpec("rotary", {"head_dim": D, "theta": theta, "scaling": scaling, "rotary_dim": rot}))
        part.bind({}, rt_for("float32"))
        r = part.rotary()
        want = P.rope_inv_freq(rot or D, theta, scaling)
        assert r.rotary_dim == (rot or D) and not r.interleaved and r.mscale == 1.0
        assert np.allclose(r.inv_freq.cpu().double().numpy(), want, rtol=1e-7)
        assert np.allclose(rotary_inv_freq(rot or D, theta, scaling).numpy(), want, rtol=1e-14)
    with pytest.raises(ValueError):
        make_part("position", PartSpec("rotary", {"head_dim": 16, "theta": 1e4, "rotary_dim": 32}))
    assert make_part("position", PartSpec("none", {})).rotary() is None


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
@pytest.mark.parametrize("bias", [False, True])
def test_gated_mlp_part(rt_for, dt, bias):
    from xyntetik_runner_amd.parts import make_part
    from xyntetik_runner_amd.config import PartSpec
    rt = rt_for(dt)
    rng = np.random.default_rng(1)
    E, F, T = 72, 104, 9
    part = make_part("feed_forward", PartSpec("gated_mlp", {"hidden_size": E, "intermediate_size": F, "bias": bias}))
    specs = part.param_specs()
    assert specs["gate_proj.weight"].shape == (F, E) and specs["down_proj.weight"].shape == (E, F)
    assert ("down_proj.bias" in specs) == bias
    w = {k: bf(rng.normal(size=s.shape) * 0.2) for k, s in specs.items()}
    part.bind({k: torch.tensor(v, dtype=torch.float32).to(DT[dt] if specs[k].role == "matrix" else torch.float32).to(DEV)
               for k, v in w.items()}, rt)
    h = bf(rng.normal(size=(T, E)))
    want = P.mlp(h, w["gate_proj.weight"], w["up_proj.weight"], w["down_proj.weight"],
                 w.get("gate_proj.bias"), w.get("up_proj.bias"), w.get("down_proj.bias"))
    ht = torch.tensor(h, dtype=torch.float32).to(DT[dt]).to(DEV)
    assert rel(part.forward(Ctx(rt.ops), ht), want) < TOL[dt]
    res = torch.tensor(rng.normal(size=(T, E)), dtype=torch.float32, device=DEV)
    base = res.clone()
    part.forward_add(Ctx(rt.ops), ht, res)
    assert rel(res, base.double().cpu().numpy() + want) < TOL[dt]


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
@pytest.mark.parametrize("H,Hk,D,window,bias", [(4, 2, 16, None, False), (6, 2, 32, 5, True), (3, 3, 48, None, True)])
def test_attention_part(rt_for, dt, H, Hk, D, window, bias):
    """The mixer over a request cut in three steps equals plain attention over the whole sequence."""
    from xyntetik_runner_amd.cache.storage import LayerCache
    from xyntetik_runner_amd.parts import make_part
    from xyntetik_runner_amd.config import PartSpec
    rt = rt_for(dt)
    rng = np.random.default_rng(2)
    E, T, ps = 40, 45, 16
    pos = PartSpec("rotary", {"head_dim": D, "theta": 10000.0})
    part = make_part("mixer", PartSpec("paged_attention", {
        "hidden_size": E, "num_heads": H, "num_kv_heads": Hk, "head_dim": D, "position": pos, "window": window, "bias": bias}))
    ks = part.kv_spec()
    assert (ks.num_kv_heads, ks.head_dim, ks.window) == (Hk, D, window) and part.state_spec() is None
    specs = part.param_specs()
    assert specs["q_proj.weight"].shape == (H * D, E) and specs["o_proj.weight"].shape == (E, H * D)
    w = {k: bf(rng.normal(size=s.shape) * 0.3) for k, s in specs.items()}
    part.bind({k: torch.tensor(v, dtype=torch.float32).to(DT[dt] if specs[k].role == "matrix" else torch.float32).to(DEV)
               for k, v in w.items()}, rt)
    h = bf(rng.normal(size=(T, E)))
    b = lambda n: w[n] if bias else 0.0
    q = (h @ w["q_proj.weight"].T + b("q_proj.bias")).reshape(T, H, D)
    k = (h @ w["k_proj.weight"].T + b("k_proj.bias")).reshape(T, Hk, D)
    v = (h @ w["v_proj.weight"].T + b("v_proj.bias")).reshape(T, Hk, D)
    inv = P.rope_inv_freq(D, 10000.0)
    o = P.attention(P.rope(q, np.arange(T), inv), P.rope(k, np.arange(T), inv), v, 1 / math.sqrt(D), window)
    want = o.reshape(T, H * D) @ w["o_proj.weight"].T + b("o_proj.bias")
    tables, n_pages = scatter_pages([T], ps, 4)
    cache = LayerCache(0, ps, True,
                       torch.full((n_pages, Hk, ps, D), float("nan"), dtype=DT[dt], device=DEV),
                       torch.full((n_pages, Hk, D, ps), float("nan"), dtype=DT[dt], device=DEV))
    outs, start = [], 0
    for n in (30, 2, 13):
        ctx = FakeCtx([start], [n], tables, ps)
        ctx.ops = rt.ops
        outs.append(part.forward(ctx, cache, torch.tensor(h[start:start + n], dtype=torch.float32).to(DT[dt]).to(DEV)))
        start += n
    assert rel(torch.cat(outs).float(), want) < (TOL[dt] if dt == "float32" else 2.5e-2)


@pytest.mark.parametrize("dt", ["float32", "bfloat16"])
def test_embedding_head_and_block(rt_for, dt):
    from xyntetik_runner_amd.parts import make_part, make_block
    from xyntetik_runner_amd.config import PartSpec
    rt = rt_for(dt)
    rng = np.random.default_rng(3)
    V, E = 77, 24
    table = bf(rng.normal(size=(V, E)))
    emb = make_part("embedding", PartSpec("token_embedding", {"vocab_size": V, "hidden_size": E}))
    emb.bind({"weight": torch.tensor(table, dtype=torch.float32).to(DT[dt]).to(DEV)}, rt)
    ids = torch.tensor([5, 0, 76, 200], dtype=torch.int32, device=DEV)
    x = emb.forward(Ctx(rt.ops), ids)
    assert x.dtype == torch.float32 and rel(x, table[[5, 0, 76, 0]]) == 0
    for tied in (True, False):
        head = make_part("head", PartSpec("linear", {"vocab_size": V, "hidden_size": E, "tied": tied}))
        assert (head.param_specs() == {}) == tied
        hw = bf(rng.normal(size=(V, E)))
        head.bind({} if tied else {"weight": torch.tensor(hw, dtype=torch.float32).to(DT[dt]).to(DEV)}, rt, tied_to=emb)
        h = bf(rng.normal(size=(3, E)))
        got = head.forward(Ctx(rt.ops), torch.tensor(h, dtype=torch.float32).to(DT[dt]).to(DEV))
        assert got.dtype == torch.float32 and rel(got, h @ (table if tied else hw).T) < 1e-5
        if tied:
            # one table for both: the head's, in the order its product reads it, from which the
            # embedding gathers the same rows as before
            assert emb.weight is head.weight
            assert rel(emb.forward(Ctx(rt.ops), ids), table[[5, 0, 76, 0]]) == 0

    # the pre-norm arrangement with stand-in parts: x += 2*norm(x) then x += 3*norm(x)
    class N:
        def __init__(self, f): self.f = f
        def forward(self, ctx, x, rows=None): return (x * self.f).to(DT[dt])
    class M:
        def forward_add(self, ctx, cache, h, res): res += h.float()
    class F:
        def forward_add(self, ctx, h, res): res += h.float()
    blk = make_block("prenorm", M(), F(), {"mixer_norm": N(2.0), "feed_forward_norm": N(3.0)})
    x = torch.ones(2, 4, device=DEV)
    blk.forward(Ctx(rt.ops), None, x)
    assert torch.equal(x, torch.full((2, 4), 12.0, device=DEV))      # 1 + 2 = 3; 3 + 9 = 12
    with pytest.raises(ValueError):
        make_block("no-such-arrangement", None, None, {})
    with pytest.raises(ValueError, match="feed_forward_norm"):     # the arrangement names its norms
        make_block("prenorm", M(), F(), {"mixer_norm": N(2.0)})
    with pytest.raises(ValueError, match="feed-forward"):
        make_block("prenorm", M(), None, {"mixer_norm": N(2.0), "feed_forward_norm": N(3.0)})
