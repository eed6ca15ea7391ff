"""A plain, slow Llama dense decoder in numpy float64: whole sequences, no cache.

One function per part, written from the reference's formulas (each cites the file and
lines of the reference it follows, relative to its root).  It shares no code with the engine:
it reads config.json and model.safetensors with its own few lines and knows nothing
of pages, batches or kernels.  The tests compare everything the engine does with it.
"""
from __future__ import annotations

import json
import math
import os
import struct

import numpy as np


# ----------------------------------------------------------------------------- files
def read_safetensors(path):
    """name -> float64 array (bf16/f16/f32 widened exactly)."""
    with open(path, "rb") as f:
        (n,) = struct.unpack("<Q", f.read(8))
        header = json.loads(f.read(n).decode("utf-8"))
        blob = f.read()
    out = {}
    for name, info in header.items():
        if name == "__metadata__":
            continue
        b, e = info["data_offsets"]
        raw = blob[b:e]
        dt = info["dtype"]
        if dt == "BF16":
            u = np.frombuffer(raw, dtype="<u2").astype(np.uint32) << 16
            arr = u.view(np.float32).astype(np.float64)
        elif dt == "F32":
            arr = np.frombuffer(raw, dtype="<f4").astype(np.float64)
        elif dt == "F16":
            arr = np.frombuffer(raw, dtype="<f2").astype(np.float64)
        else:
            raise ValueError(f"{name}: dtype {dt}")
        out[name] = arr.reshape(info["shape"])
    return out


def load_folder(model_dir):
    with open(os.path.join(model_dir, "config.json")) as f:
        cfg = json.load(f)
    return cfg, read_safetensors(os.path.join(model_dir, "model.safetensors"))


class TensorsOnDemand:
    """name -> float64 array like ``read_safetensors``, but every tensor is read from the file
    and widened when it is asked for and kept nowhere: for a model whose widened weights
    should not all stand in memory at once (one product's matrix at a time)."""

    def __init__(self, path):
        self.path = path
        with open(path, "rb") as f:
            (n,) = struct.unpack("<Q", f.read(8))
            self.header = {k: v for k, v in json.loads(f.read(n).decode("utf-8")).items() if k != "__metadata__"}
        self.base = 8 + n

    def __contains__(self, name):
        return name in self.header

    def __iter__(self):
        return iter(self.header)

    def get(self, name, default=None):
        return self[name] if name in self.header else default

    def __getitem__(self, name):
        info = self.header[name]
        b, e = info["data_offsets"]
        with open(self.path, "rb") as f:
            f.seek(self.base + b)
            raw = f.read(e - b)
        dt = info["dtype"]
        if dt == "BF16":
            arr = (np.frombuffer(raw, dtype="<u2").astype(np.uint32) << 16).view(np.float32).astype(np.float64)
        elif dt == "F32":
            arr = np.frombuffer(raw, dtype="<f4").astype(np.float64)
        elif dt == "F16":
            arr = np.frombuffer(raw, dtype="<f2").astype(np.float64)
        else:
            raise ValueError(f"{name}: dtype {dt}")
        return arr.reshape(info["shape"])


def open_folder(model_dir):
    """As ``load_folder`` with the tensors read on demand."""
    with open(os.path.join(model_dir, "config.json")) as f:
        cfg = json.load(f)
    return cfg, TensorsOnDemand(os.path.join(model_dir, "model.safetensors"))


# ----------------------------------------------------------------------------- parts
def rmsnorm(x, w, eps):
    """y = x * (1/sqrt(mean(x^2) + eps)) * w: eps inside the root, added to the mean.
    src/model.c:3386-3392"""
    ss = np.sum(x * x, axis=-1, keepdims=True)
    r = 1.0 / np.sqrt(ss / x.shape[-1] + eps)
    return x * r * w


def rope_inv_freq(rot_dim, theta, scaling=None):
    """inv_freq[j] = theta^(-2j/rot_dim) (src/model.c:285-289), then divided
    by per-dimension factors (:291-297).  The reference takes the factors from the file;
    for rope_type "llama3" they follow from config.json: wavelength below orig/high is
    kept, above orig/low divided by factor, between them interpolated in orig/wavelength."""
    j = np.arange(rot_dim // 2, dtype=np.float64)
    inv = theta ** (-2.0 * j / rot_dim)
    if not scaling:
        return inv
    kind = scaling.get("rope_type", scaling.get("type"))
    if kind in (None, "default"):
        return inv
    factor = scaling["factor"]
    if kind == "linear":       # src/model.c:317-321
        return inv / factor
    assert kind == "llama3", kind
    low, high = scaling["low_freq_factor"], scaling["high_freq_factor"]
    orig = scaling["original_max_position_embeddings"]
    out = np.empty_like(inv)
    for i, f in enumerate(inv):
        wavelen = 2.0 * math.pi / f
        if wavelen < orig / high:
            out[i] = f
        elif wavelen > orig / low:
            out[i] = f / factor
        else:
            s = (orig / wavelen - low) / (high - low)
            out[i] = (1.0 - s) * f / factor + s * f
    return out


def rope_angle(position, inv_freq_j):
    """a = pos * inv_freq[j] the way the reference forms it: the table holds floats
    (src/model.c:286-289) and ``float a = pos * fr[j]`` is a float product (:3520).
    At position 2,048 that product differs from the exact one by up to 1.2e-4 rad for the fastest
    pair, which belongs to the model as it is defined; cosine and sine are then taken exactly."""
    return float(np.float32(position) * np.float32(inv_freq_j))


def rope(x, positions, inv_freq, interleaved=False):
    """Rotate pair j of every head by a = pos * inv_freq[j]:
    (x0, x1) -> (x0 cos a - x1 sin a, x0 sin a + x1 cos a).  Un-permuted checkpoints pair
    element j with j + rot/2; the other layout pairs 2j with 2j+1.
    x: [T, heads, D].  src/model.c:3514-3532"""
    T, H, D = x.shape
    half = len(inv_freq)
    y = x.copy()
    for t in range(T):
        for j in range(half):
            a = rope_angle(positions[t], inv_freq[j])
            c, s = math.cos(a), math.sin(a)
            i0, i1 = (2 * j, 2 * j + 1) if interleaved else (j, j + half)
            x0, x1 = x[t, :, i0].copy(), x[t, :, i1].copy()
            y[t, :, i0] = x0 * c - x1 * s
            y[t, :, i1] = x0 * s + x1 * c
    return y


def rope_all_at_once(x, positions, inv_freq):
    """``rope`` for pairs (j, j + rot/2) with whole arrays in place of its loops (for long sequences)."""
    half = len(inv_freq)
    a = (np.asarray(positions, dtype=np.float32)[:, None] * np.asarray(inv_freq, dtype=np.float32)[None, :]).astype(np.float64)
    c, s = np.cos(a)[:, None, :], np.sin(a)[:, None, :]
    y = x.copy()
    x0, x1 = x[:, :, :half], x[:, :, half:2 * half]
    y[:, :, :half] = x0 * c - x1 * s
    y[:, :, half:2 * half] = x0 * s + x1 * c
    return y


def softmax(s):
    """Maximum out, exponentials, divide by their sum.  src/model.c:3409-3415"""
    e = np.exp(s - np.max(s))
    return e / np.sum(e)


def attention(q, k, v, scale, window=None):
    """q [T, H, D], k/v [T, Hk, D], all of one sequence from position 0.  Head h reads
    key/value head h // (H/Hk); s_t = (q . k_t) * scale for t in [t0, p], t0 = p - window + 1
    when windowed; softmax; o = sum_t p_t v_t.
    src/model.c:3548-3589 (heads, scores, weighted values), :6326 (t0)"""
    T, H, D = q.shape
    Hk = k.shape[1]
    mul = H // Hk
    out = np.zeros((T, H, D))
    for p in range(T):
        t0 = max(0, p - window + 1) if window else 0
        for h in range(H):
            kvh = h // mul
            s = np.array([np.dot(q[p, h], k[t, kvh]) * scale for t in range(t0, p + 1)])
            pr = softmax(s)
            for i, t in enumerate(range(t0, p + 1)):
                out[p, h] += pr[i] * v[t, kvh]
    return out


def attention_all_at_once(q, k, v, scale, window=None):
    """``attention`` with one score matrix per head in place of its loops (for long sequences):
    softmax over the keys a position may see of (q k^T) * scale, times v."""
    T, H, D = q.shape
    Hk = k.shape[1]
    mul = H // Hk
    pos = np.arange(T)
    seen = pos[None, :] <= pos[:, None]
    if window:
        seen &= pos[None, :] > pos[:, None] - window
    out = np.zeros((T, H, D))
    for h in range(H):
        kvh = h // mul
        s = (q[:, h, :] @ k[:, kvh, :].T) * scale
        s = np.where(seen, s, -np.inf)
        e = np.exp(s - s.max(axis=1, keepdims=True))
        out[:, h, :] = (e / e.sum(axis=1, keepdims=True)) @ v[:, kvh, :]
    return out


def silu(g):
    """g / (1 + exp(-g)).  src/model.c:4451-4452"""
    return g / (1.0 + np.exp(-g))


def mlp(h, wg, wu, wd, bg=None, bu=None, bd=None):
    """down(silu(gate h) * (up h)).  src/model.c:6399-6407"""
    g = h @ wg.T + (0 if bg is None else bg)
    u = h @ wu.T + (0 if bu is None else bu)
    return (silu(g) * u) @ wd.T + (0 if bd is None else bd)


# ----------------------------------------------------------------------------- the model
def forward(cfg, w, tokens, return_hidden=False, rows=None, all_at_once=False):
    """Logits [T, V] of one whole sequence (of the positions ``rows`` only, if given).  Order
    per layer: norm, q/k/v, rotation of q and k, attention over positions <= own, output
    projection, add, norm, feed-forward, add; then final norm and head.
    src/model.c:6148-6483.  ``all_at_once``: rotation and attention by their
    whole-array forms (a long sequence would take the loops minutes)."""
    rope_fn = rope_all_at_once if all_at_once else rope
    attention_fn = attention_all_at_once if all_at_once else attention
    E = cfg["hidden_size"]
    H = cfg["num_attention_heads"]
    Hk = cfg.get("num_key_value_heads") or H
    D = cfg.get("head_dim") or E // H
    eps = cfg.get("rms_norm_eps", 1e-5)
    theta = cfg.get("rope_theta", 10000.0)
    inv_freq = rope_inv_freq(D, theta, cfg.get("rope_scaling"))
    V = cfg["vocab_size"]
    T = len(tokens)
    pos = np.arange(T)
    # embedding: row copy, id outside the vocabulary reads row 0 (src/model.c:6148-6162)
    ids = [t if 0 <= t < V else 0 for t in tokens]
    x = w["model.embed_tokens.weight"][ids].copy()
    scale = 1.0 / math.sqrt(D)                      # src/model.h:464-467
    for l in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{l}."
        h = rmsnorm(x, w[p + "input_layernorm.weight"], eps)
        q = h @ w[p + "self_attn.q_proj.weight"].T
        k = h @ w[p + "self_attn.k_proj.weight"].T
        v = h @ w[p + "self_attn.v_proj.weight"].T
        if cfg.get("attention_bias"):
            q = q + w[p + "self_attn.q_proj.bias"]
            k = k + w[p + "self_attn.k_proj.bias"]
            v = v + w[p + "self_attn.v_proj.bias"]
        q = rope_fn(q.reshape(T, H, D), pos, inv_freq)
        k = rope_fn(k.reshape(T, Hk, D), pos, inv_freq)
        o = attention_fn(q, k, v.reshape(T, Hk, D), scale).reshape(T, H * D)
        a = o @ w[p + "self_attn.o_proj.weight"].T
        if cfg.get("attention_bias"):
            a = a + w[p + "self_attn.o_proj.bias"]
        x = x + a                                    # src/model.c:6350-6352
        h = rmsnorm(x, w[p + "post_attention_layernorm.weight"], eps)
        mb = cfg.get("mlp_bias")
        x = x + mlp(h, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"],
                    w.get(p + "mlp.gate_proj.bias") if mb else None, w.get(p + "mlp.up_proj.bias") if mb else None,
                    w.get(p + "mlp.down_proj.bias") if mb else None)   # src/model.c:6421-6423
    if return_hidden:
        return x
    if rows is not None:
        x = x[list(rows)]
    h = rmsnorm(x, w["model.norm.weight"], eps)      # src/model.c:6479
    head = w["model.embed_tokens.weight"] if cfg.get("tie_word_embeddings") else w["lm_head.weight"]
    return h @ head.T                                # src/model.c:6481, tied :2353-2366


def greedy(cfg, w, prompt, n_new):
    """Greedy continuation: first index of the maximum (src/sample.c:169-172)."""
    toks = list(prompt)
    out = []
    for _ in range(n_new):
        nxt = int(np.argmax(forward(cfg, w, toks)[-1]))
        out.append(nxt)
        toks.append(nxt)
    return out


# ----------------------------------------------------------------------------- sampling
def xorshift64(state):
    """x ^= x<<13; x ^= x>>7; x ^= x<<17 on 64 bits.  src/sample.c:13-17"""
    x = state & 0xFFFFFFFFFFFFFFFF
    x ^= (x << 13) & 0xFFFFFFFFFFFFFFFF
    x ^= x >> 7
    x ^= (x << 17) & 0xFFFFFFFFFFFFFFFF
    return x


def rng_f32(state):
    """(new state, draw in [0,1) from the top 24 bits).  src/sample.c:18-20"""
    s = xorshift64(state)
    return s, (s >> 40) / 16777216.0


def sample_pick(logits, temp, draw, top_k=0, top_p=1.0, min_p=0.0, repeat_penalty=1.0, recent=(), exempt=()):
    """The reference's pick on a copy of ``logits`` with a given draw.
    src/sample.c:141-329 (penalty :148-166, greedy :169-172, candidates sorted by
    z descending then id ascending :32-38, softmax / top-p / min-p / roulette walk :86-127)."""
    logits = np.array(logits, dtype=np.float32)
    V = len(logits)
    if temp > 0 and repeat_penalty != 1.0:
        for tok in recent:
            if tok < 0 or tok >= V or tok in exempt:
                continue
            logits[tok] = logits[tok] / np.float32(repeat_penalty) if logits[tok] > 0 else logits[tok] * np.float32(repeat_penalty)
    if temp <= 0:
        best = 0
        for i in range(1, V):
            if logits[i] > logits[best]:
                best = i
        return best
    z = (logits / np.float32(temp)).astype(np.float64)
    order = sorted(range(V), key=lambda i: (-z[i], i))
    k = top_k if 0 < top_k < V else V
    c = order[:k]
    p = np.exp(z[c] - z[c[0]])
    p = p / p.sum()
    if top_p < 1.0:
        cum, cut = 0.0, len(c)
        for i in range(len(c)):
            cum += p[i]
            if cum >= top_p:
                cut = i + 1
                break
        c, p = c[:cut], p[:cut] / p[:cut].sum()
    if min_p > 0.0:
        floor_p = min_p * p[0]
        cut = len(c)
        for i in range(1, len(c)):
            if p[i] < floor_p:
                cut = i
                break
        c, p = c[:cut], p[:cut] / p[:cut].sum()
    cum = 0.0
    for i in range(len(c)):
        cum += p[i]
        if draw < cum:
            return c[i]
    return c[-1]
