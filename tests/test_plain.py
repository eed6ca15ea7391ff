"""What fixes the plain implementation beside the reference's text: special cases that
reduce to a library routine, invariants, and vectors the reference's own tests hold.
Each check is chosen so that a plausible mistake fails it."""
import copy
import math

import numpy as np
import pytest

import plain_llama as P
from tiny import TINY_A, TINY_B, make_model, prompt_ids

rng = np.random.default_rng(0)


# ------------------------------------------------------------------ RMSNorm
def test_rmsnorm_library_form_and_eps_placement():
    x, w = rng.normal(size=(3, 10)), rng.normal(size=10)
    want = x / np.sqrt((x ** 2).mean(-1, keepdims=True) + 1e-5) * w
    assert np.allclose(P.rmsnorm(x, w, 1e-5), want, rtol=1e-12)
    y = P.rmsnorm(x, np.ones(10), 0.0)
    assert np.allclose((y ** 2).mean(-1), 1.0)                        # w=1, eps=0: unit mean square
    assert np.allclose(P.rmsnorm(3.7 * x, w, 0.0), P.rmsnorm(x, w, 0.0))   # scale invariance without eps
    # eps inside the root, added to the mean: sqrt(ms + eps), not sqrt(ms) + eps, not sqrt(sum + eps)
    tiny = np.full((1, 4), 1e-4)
    got = P.rmsnorm(tiny, np.ones(4), 1e-6)[0, 0]
    assert math.isclose(got, 1e-4 / math.sqrt(1e-8 + 1e-6), rel_tol=1e-12)
    assert not math.isclose(got, 1e-4 / (1e-4 + 1e-6), rel_tol=1e-3)
    assert not math.isclose(got, 1e-4 / math.sqrt((4e-8 + 1e-6) / 4), rel_tol=1e-3)


# ------------------------------------------------------------------ rotary
def test_rope_identity_norm_composition_and_relative_positions():
    inv = P.rope_inv_freq(8, 10000.0)
    assert np.allclose(inv, 10000.0 ** (-np.arange(4) / 4.0))
    x = rng.normal(size=(1, 2, 8))
    assert np.allclose(P.rope(x, [0], inv), x)                         # position 0 is the identity
    y = P.rope(x, [5], inv)
    for j in range(4):                                                 # each pair (j, j+4) keeps its norm
        assert np.allclose(x[0, :, j] ** 2 + x[0, :, j + 4] ** 2, y[0, :, j] ** 2 + y[0, :, j + 4] ** 2)
    assert np.allclose(P.rope(P.rope(x, [3], inv), [4], inv), P.rope(x, [7], inv))   # angles add
    q, k = rng.normal(size=(1, 1, 8)), rng.normal(size=(1, 1, 8))
    d1 = np.dot(P.rope(q, [9], inv)[0, 0], P.rope(k, [4], inv)[0, 0])
    d2 = np.dot(P.rope(q, [105], inv)[0, 0], P.rope(k, [100], inv)[0, 0])
    # only the distance counts: as far as a float angle goes (the reference's `float a = pos * fr[j]`
    # rounds position 105 times the frequency to 24 bits, about 4e-6 rad); a wrong pairing or
    # sign changes the product by its own size
    assert math.isclose(d1, d2, rel_tol=2e-6)
    assert P.rope_angle(2048, np.float64(1) / 3) == float(np.float32(2048) * np.float32(1 / 3))
    d3 = np.dot(P.rope(q, [4], inv)[0, 0], P.rope(k, [9], inv)[0, 0])
    assert not math.isclose(d1, d3, rel_tol=1e-3)                      # and its sign matters


def test_rope_rotation_direction_and_pairing():
    # one pair, angle pi/2 at position 1: (1, 0) -> (0, 1); a wrong sign gives (0, -1)
    inv = np.array([math.pi / 2])
    x = np.array([[[1.0, 0.0]]])
    assert np.allclose(P.rope(x, [1], inv)[0, 0], [0.0, 1.0], atol=1e-7)         # (the angle is a float: pi/2 to 24 bits)
    # half-split on un-permuted rows == adjacent pairs on rows permuted as [0, D/2, 1, D/2+1, ...]
    # (the converter's relation, src/model.c:1464-1466)
    D = 8
    inv = P.rope_inv_freq(D, 10000.0)
    v = rng.normal(size=(1, 1, D))
    perm = [i // 2 + (D // 2) * (i % 2) for i in range(D)]
    a = P.rope(v, [6], inv)[0, 0][perm]
    b = P.rope(v[:, :, perm], [6], inv, interleaved=True)[0, 0]
    assert np.allclose(a, b)
    assert not np.allclose(P.rope(v, [6], inv), P.rope(v, [6], inv, interleaved=True))


def test_llama3_scaling_bands():
    sc = dict(TINY_B["rope_scaling"])
    base = P.rope_inv_freq(32, 500000.0)
    got = P.rope_inv_freq(32, 500000.0, sc)
    wl = 2 * math.pi / base
    lo, hi = 32 / 1.0, 32 / 4.0                         # thresholds: wavelengths 32 and 8
    assert (wl < hi).any() and (wl > lo).any() and ((wl >= hi) & (wl <= lo)).any()
    assert np.array_equal(got[wl < hi], base[wl < hi])                   # short wavelengths untouched
    assert np.allclose(got[wl > lo], base[wl > lo] / 8.0, rtol=1e-15)    # long ones exactly / factor
    mid = (wl >= hi) & (wl <= lo)
    assert np.all(got[mid] <= base[mid]) and np.all(got[mid] >= base[mid] / 8.0)
    inner = (wl > hi * 1.01) & (wl < lo * 0.99)
    assert np.all(got[inner] < base[inner]) and np.all(got[inner] > base[inner] / 8.0)
    assert np.allclose(P.rope_inv_freq(32, 500000.0, dict(sc, factor=1.0)), base)   # factor 1 = identity
    assert np.allclose(P.rope_inv_freq(16, 1000.0, {"rope_type": "linear", "factor": 4.0}),
                       P.rope_inv_freq(16, 1000.0) / 4.0)


def _plain_table(rot, theta, scaling=None):
    return np.asarray(P.rope_inv_freq(rot, theta, scaling), dtype=np.float64)


def _engine_table(rot, theta, scaling=None):
    from xyntetik_runner_amd.parts.rotary import rotary_inv_freq
    return rotary_inv_freq(rot, theta, scaling).numpy().astype(np.float64)


@pytest.mark.parametrize("table", [_plain_table, _engine_table], ids=["plain", "engine"])
def test_llama3_scaling_is_continuous_monotone_and_linear_in_frequency(table):
    """What fixes the interpolation between the two bands beside its text
    (hook: src/model.c:291-297, where the reference divides by the factors a file
    brings): the scaled/unscaled ratio is 1 below wavelength orig/high and 1/factor above
    orig/low, so a rule that joins them must meet both values at the band's edges, fall
    monotonically between them, and, being linear in orig/wavelength, give the mean of the two
    values where orig/wavelength is the mean of low and high.  Swapping the two weights of the
    interpolation jumps by the factor at both edges; interpolating in wavelength instead of
    frequency misses the midpoint."""
    sc = {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
          "original_max_position_embeddings": 8192}
    orig, low, high, factor = 8192.0, 1.0, 4.0, 8.0

    def ratio(wavelength):
        # a table of two entries whose second has exactly this wavelength: theta^(-1/2) = 2 pi / wavelength
        theta = (wavelength / (2.0 * math.pi)) ** 2
        return table(4, theta, sc)[1] / table(4, theta)[1]

    for edge, value in ((orig / high, 1.0), (orig / low, 1.0 / factor)):
        below, above = ratio(edge * (1 - 1e-9)), ratio(edge * (1 + 1e-9))
        assert abs(below - value) < 1e-6 and abs(above - value) < 1e-6, (edge, below, above)
    sweep = [ratio(w) for w in np.geomspace(orig / high / 2, orig / low * 2, 300)]
    assert all(a >= b - 1e-12 for a, b in zip(sweep, sweep[1:])) and sweep[0] == 1.0 and abs(sweep[-1] - 1 / factor) < 1e-15
    for share in (0.25, 0.5, 0.75):         # orig/wavelength = low + share * (high - low)
        w = orig / (low + share * (high - low))
        assert abs(ratio(w) - ((1 - share) / factor + share)) < 1e-9, share
    # the benchmark model's table (head size 128, base 5e5) has several entries inside the band
    base, got = table(128, 500000.0), table(128, 500000.0, sc)
    wl = 2 * math.pi / base
    mid = (wl > orig / high) & (wl < orig / low)
    assert mid.sum() >= 5
    r = got / base
    assert np.all(np.diff(r) <= 1e-12) and np.all((r[mid] < 1.0) & (r[mid] > 1.0 / factor))
    s = (orig / wl[mid] - low) / (high - low)
    assert np.allclose(r[mid], (1 - s) / factor + s, rtol=1e-9)


def test_plain_and_engine_tables_agree():
    for rot, theta, sc in ((32, 500000.0, TINY_B["rope_scaling"]), (128, 500000.0, dict(TINY_B["rope_scaling"], original_max_position_embeddings=8192)),
                           (16, 10000.0, None), (48, 1000.0, {"rope_type": "linear", "factor": 2.0})):
        assert np.allclose(_plain_table(rot, theta, sc), _engine_table(rot, theta, sc), rtol=1e-12)


# ------------------------------------------------------------------ attention
def test_attention_special_cases():
    T, H, Hk, D = 6, 4, 2, 8
    q, k, v = rng.normal(size=(T, H, D)), rng.normal(size=(T, Hk, D)), rng.normal(size=(T, Hk, D))
    o = P.attention(q, k, v, 1 / math.sqrt(D))
    assert np.allclose(o[0, 0], v[0, 0]) and np.allclose(o[0, 3], v[0, 1])       # one key: the value row
    z = P.attention(np.zeros_like(q), k, v, 1.0)
    for p in range(T):
        assert np.allclose(z[p, 1], v[:p + 1, 0].mean(0))                        # q = 0: mean over the causal prefix
        assert np.allclose(z[p, 2], v[:p + 1, 1].mean(0))                        # heads 2,3 -> kv head 1 (contiguous groups)
    # library form: softmax(q k^T * scale + causal mask) v, grouped == repeated heads
    kr, vr = np.repeat(k, H // Hk, axis=1), np.repeat(v, H // Hk, axis=1)
    s = np.einsum("thd,shd->hts", q, kr) / math.sqrt(D)
    s = np.where(np.tril(np.ones((T, T), bool))[None], s, -np.inf)
    e = np.exp(s - s.max(-1, keepdims=True))
    want = np.einsum("hts,shd->thd", e / e.sum(-1, keepdims=True), vr)
    assert np.allclose(o, want, rtol=1e-10)
    assert np.allclose(P.attention(q, kr, vr, 1 / math.sqrt(D)), o)
    # causality: a later token never changes an earlier output
    k2, v2 = k.copy(), v.copy()
    k2[4] += 1.0; v2[4] -= 2.0
    o2 = P.attention(q, k2, v2, 1 / math.sqrt(D))
    assert np.array_equal(o2[:4], o[:4]) and not np.allclose(o2[4], o[4])
    # window: exactly the last w keys
    w = P.attention(q, k, v, 1 / math.sqrt(D), window=2)
    assert np.allclose(w[:2], o[:2]) and not np.allclose(w[3], o[3])
    assert np.allclose(w[5], P.attention(q[4:6], k[4:6], v[4:6], 1 / math.sqrt(D))[1])


def test_softmax_properties():
    s = rng.normal(size=9) * 5
    p = P.softmax(s)
    assert math.isclose(p.sum(), 1.0) and np.allclose(P.softmax(s + 123.0), p)
    big = P.softmax(np.array([1e4, -1e4, 1e4 - 1.0]))
    assert np.all(np.isfinite(big)) and math.isclose(big[0], 1 / (1 + math.exp(-1)), rel_tol=1e-12)


def test_swiglu():
    assert P.silu(np.array([0.0]))[0] == 0.0
    g = np.array([-3.0, 0.5, 2.0])
    assert np.allclose(P.silu(g), g * (1 / (1 + np.exp(-g))))
    assert abs(P.silu(np.array([-200.0]))[0]) < 1e-80                  # large negative gate: 0, no NaN
    E, F = 6, 10
    h = rng.normal(size=(2, E))
    wg, wu, wd = rng.normal(size=(F, E)), rng.normal(size=(F, E)), rng.normal(size=(E, F))
    assert np.allclose(P.mlp(h, np.zeros_like(wg), wu, wd), 0.0)       # zero gate: zero output
    assert np.allclose(P.mlp(h, wg, wu, wd), ((h @ wg.T) / (1 + np.exp(-(h @ wg.T))) * (h @ wu.T)) @ wd.T)
    assert not np.allclose(P.mlp(h, wg, wu, wd), P.mlp(h, wu, wg, wd))  # gate and up are not interchangeable


# ------------------------------------------------------------------ the whole model
@pytest.fixture(scope="module")
def model_a(tmp_path_factory):
    return P.load_folder(make_model("A", str(tmp_path_factory.mktemp("a"))))


@pytest.fixture(scope="module")
def model_b(tmp_path_factory):
    return P.load_folder(make_model("B", str(tmp_path_factory.mktemp("b"))))


def test_residual_structure(model_a):
    cfg, w = model_a
    w0 = dict(w)
    for l in range(cfg["num_hidden_layers"]):
        w0[f"model.layers.{l}.self_attn.o_proj.weight"] = np.zeros_like(w[f"model.layers.{l}.self_attn.o_proj.weight"])
        w0[f"model.layers.{l}.mlp.down_proj.weight"] = np.zeros_like(w[f"model.layers.{l}.mlp.down_proj.weight"])
    toks = prompt_ids(5, 256, 1)
    want = P.rmsnorm(w["model.embed_tokens.weight"][toks], w["model.norm.weight"], 1e-5) @ w["lm_head.weight"].T
    assert np.allclose(P.forward(cfg, w0, toks), want)                 # logits = head(norm(embedding))
    assert not np.allclose(P.forward(cfg, w, toks), want)


def test_causality_and_prefix_invariance(model_b):
    cfg, w = model_b
    toks = prompt_ids(12, 384, 2)
    full = P.forward(cfg, w, toks)
    assert np.allclose(P.forward(cfg, w, toks[:7]), full[:7], atol=1e-12)      # row i depends on tokens [0, i]
    other = list(toks); other[9] = (other[9] + 1) % 384
    assert np.allclose(P.forward(cfg, w, other)[:9], full[:9], atol=1e-12)
    assert not np.allclose(P.forward(cfg, w, other)[9:], full[9:])


def test_tied_head_is_the_embedding(model_b):
    cfg, w = model_b
    toks = prompt_ids(4, 384, 3)
    untied = dict(cfg, tie_word_embeddings=False)
    w2 = dict(w); w2["lm_head.weight"] = w["model.embed_tokens.weight"].copy()
    assert np.array_equal(P.forward(cfg, w, toks), P.forward(untied, w2, toks))


def test_out_of_range_token_reads_row_zero(model_a):
    cfg, w = model_a
    assert np.array_equal(P.forward(cfg, w, [3, 999, 5]), P.forward(cfg, w, [3, 0, 5]))


def test_layer_norms_sit_before_the_parts(model_a):
    """Scaling a layer's input norm weight must change the attention input only (pre-norm):
    with o_proj = 0 in that layer the scaling has no effect at all."""
    cfg, w = model_a
    toks = prompt_ids(6, 256, 4)
    w1 = dict(w)
    w1["model.layers.0.self_attn.o_proj.weight"] = np.zeros_like(w["model.layers.0.self_attn.o_proj.weight"])
    w2 = dict(w1)
    w2["model.layers.0.input_layernorm.weight"] = w["model.layers.0.input_layernorm.weight"] * 3.0
    assert np.allclose(P.forward(cfg, w1, toks), P.forward(cfg, w2, toks))
    w3 = dict(w); w3["model.layers.0.input_layernorm.weight"] = w["model.layers.0.input_layernorm.weight"] * 3.0
    assert not np.allclose(P.forward(cfg, w, toks), P.forward(cfg, w3, toks))


# ------------------------------------------------------------------ the forms for long sequences
def test_whole_array_forms_equal_the_loops(tmp_path):
    """``rope_all_at_once`` and ``attention_all_at_once`` (used where the loops would take
    minutes) against the loops they stand for, with and without a window, grouped heads; and a
    model read tensor by tensor against the same model read whole."""
    T, H, Hk, D = 23, 6, 2, 16
    q, k, v = rng.normal(size=(T, H, D)), rng.normal(size=(T, Hk, D)), rng.normal(size=(T, Hk, D))
    pos = np.arange(T) + 3
    for rot in (D, 8):
        inv = P.rope_inv_freq(rot, 300.0)
        assert np.allclose(P.rope_all_at_once(q, pos, inv), P.rope(q, pos, inv), rtol=1e-13, atol=1e-15)
    for window in (None, 5):
        assert np.allclose(P.attention_all_at_once(q, k, v, 0.3, window), P.attention(q, k, v, 0.3, window), rtol=1e-12)
    d = make_model("B", str(tmp_path / "m"))
    cfg, w = P.load_folder(d)
    cfg2, lazy = P.open_folder(d)
    assert cfg2 == cfg and sorted(lazy) == sorted(w) and all(np.array_equal(lazy[n], w[n]) for n in w)
    toks = prompt_ids(40, cfg["vocab_size"], 3)
    want = P.forward(cfg, w, toks)
    got = P.forward(cfg, lazy, toks, rows=[0, 17, 39], all_at_once=True)
    assert np.allclose(got, want[[0, 17, 39]], rtol=1e-10, atol=1e-12)
