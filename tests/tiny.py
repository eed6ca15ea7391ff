"""The tiny configurations the tests run on, and helpers to make their model folders.

TINY_A and TINY_B differ in every size and option: layers, width, heads and groups
(2:1 grouped vs one shared key/value head), head size, feed-forward width, vocabulary,
rotary base and scaling, the norms' eps, tied or separate output head, and how the norm
weights are drawn and stored.  TINY_C has heads*head_dim != hidden_size, biases, a
width and a vocabulary that are no powers of two and linear rotary scaling.
"""
import os

import numpy as np

TINY_A = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "num_hidden_layers": 2, "hidden_size": 64, "num_attention_heads": 4, "num_key_value_heads": 2,
    "head_dim": 16, "intermediate_size": 176, "vocab_size": 256, "rope_theta": 10000.0,
    "rope_scaling": None, "rms_norm_eps": 1e-5, "tie_word_embeddings": False,
    "max_position_embeddings": 128, "hidden_act": "silu",
}
TINY_B = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "num_hidden_layers": 3, "hidden_size": 96, "num_attention_heads": 3, "num_key_value_heads": 1,
    "head_dim": 32, "intermediate_size": 256, "vocab_size": 384, "rope_theta": 500000.0,
    "rope_scaling": {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                     "original_max_position_embeddings": 32},
    "rms_norm_eps": 1e-6, "tie_word_embeddings": True, "max_position_embeddings": 256, "hidden_act": "silu",
}
TINY_C = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "num_hidden_layers": 1, "hidden_size": 72, "num_attention_heads": 6, "num_key_value_heads": 3,
    "head_dim": 48, "intermediate_size": 100, "vocab_size": 333, "rope_theta": 1000.0,
    "rope_scaling": {"rope_type": "linear", "factor": 2.0},
    "rms_norm_eps": 1e-4, "tie_word_embeddings": False, "max_position_embeddings": 512,
    "attention_bias": True, "mlp_bias": True, "hidden_act": "silu",
}

# the benchmark model's head size and grouping at a small width: 128-wide heads, 4 query heads per
# key/value head, prompts long enough for the large-tile matrix kernels and 64-position pages
TINY_D = {
    "architectures": ["LlamaForCausalLM"], "model_type": "llama",
    "num_hidden_layers": 2, "hidden_size": 256, "num_attention_heads": 8, "num_key_value_heads": 2,
    "head_dim": 128, "intermediate_size": 544, "vocab_size": 1000, "rope_theta": 500000.0,
    "rope_scaling": {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                     "original_max_position_embeddings": 64},
    "rms_norm_eps": 1e-5, "tie_word_embeddings": False, "max_position_embeddings": 1024, "hidden_act": "silu",
}

MAKE = {
    "A": dict(config=TINY_A, seed=0, norm_jitter=0.0, dtype="bfloat16", vector_dtype=None),
    "B": dict(config=TINY_B, seed=1, norm_jitter=0.1, dtype="bfloat16", vector_dtype="float32"),
    "C": dict(config=TINY_C, seed=2, norm_jitter=0.1, dtype="bfloat16", vector_dtype="float32"),
    "D": dict(config=TINY_D, seed=3, norm_jitter=0.05, dtype="bfloat16", vector_dtype=None),
}


def make_model(which: str, folder: str, std: float = 0.02) -> str:
    from xyntetik_runner_amd.weights import write_random_model
    m = MAKE[which]
    return write_random_model(m["config"], folder, seed=m["seed"], std=std, norm_jitter=m["norm_jitter"],
                              dtype=m["dtype"], vector_dtype=m["vector_dtype"])


def prompt_ids(n: int, vocab: int, seed: int):
    rng = np.random.default_rng(seed)
    return [int(t) for t in rng.integers(0, vocab, size=n)]


def logit_error(got, want):
    """(max |d|, mean |d|) as fractions of the mean logit range of ``want``
    (the reference's measure, tests/test_gpu_identity.c:41-60)."""
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    rng = float(np.mean(want.max(axis=-1) - want.min(axis=-1)))
    d = np.abs(got - want)
    return float(d.max()) / rng, float(d.mean()) / rng
