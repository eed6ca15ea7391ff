"""``LlamaConfig``: the Llama dense decoder's hyper-parameters, typed.

Key by key this is the reference's hyper-parameter block
(src/model.c:1422-1470) under the names ``config.json`` uses:

===============================  ==============================  =========
reference GGUF key                config.json key                 default
===============================  ==============================  =========
``block_count``                   ``num_hidden_layers``           required
``embedding_length``              ``hidden_size``                 required
``attention.head_count``          ``num_attention_heads``         required
``attention.head_count_kv``       ``num_key_value_heads``         heads (:1438)
``attention.key_length``          ``head_dim``                    E/H (:1459)
``feed_forward_length``           ``intermediate_size``           required (:1445)
``context_length``                ``max_position_embeddings``     2048 (:1458)
``attention.layer_norm_rms_eps``  ``rms_norm_eps``                1e-5 (:1462)
``rope.freq_base``                ``rope_theta``                  10000 (:1463)
``rope.scaling.*``/``rope_freqs`` ``rope_scaling``                none (:291-321)
rows of ``token_embd``            ``vocab_size``                  required (:2338)
no ``output.weight``              ``tie_word_embeddings``         false (:2353)
===============================  ==============================  =========

The geometry checks are those of src/model.c:2295-2329.
"""
from __future__ import annotations

from dataclasses import dataclass, field, asdict
from typing import Any, Mapping, Optional, Tuple

from .base import ConfigError, Fields, MAX_AXIS


@dataclass(frozen=True)
class RopeScaling:
    """``rope_scaling`` of config.json.

    ``rope_type`` "llama3" rescales each rotary frequency by its wavelength; the
    reference does not compute this itself but divides its table by per-dimension
    factors that the file brings (src/model.c:291-297), which is
    the same thing.  "linear" divides every frequency by ``factor``
    (src/model.c:317-321).
    """
    rope_type: str
    factor: float
    low_freq_factor: float = 1.0
    high_freq_factor: float = 4.0
    original_max_position_embeddings: int = 8192

    @staticmethod
    def from_fields(f: Optional[Fields]) -> Optional["RopeScaling"]:
        if f is None:
            return None
        kind = f.string("rope_type", default=None)
        if kind is None:
            kind = f.string("type", default="default")
        if kind == "default":
            return None
        if kind not in ("llama3", "linear"):
            raise ConfigError(f"{f.where}: rope_type {kind!r} is not supported (llama3, linear, default)")
        factor = f.number("factor", lo=1.0)
        if kind == "linear":
            return RopeScaling("linear", factor)
        lo = f.number("low_freq_factor", lo=0.0, lo_open=True)
        hi = f.number("high_freq_factor", lo=0.0, lo_open=True)
        if not hi > lo:
            raise ConfigError(f"{f.where}: high_freq_factor ({hi}) must exceed low_freq_factor ({lo})")
        orig = f.integer("original_max_position_embeddings", lo=1, hi=1 << 30)
        return RopeScaling("llama3", factor, lo, hi, orig)


@dataclass(frozen=True)
class LlamaConfig:
    architecture: str
    num_hidden_layers: int
    hidden_size: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    intermediate_size: int
    vocab_size: int
    max_position_embeddings: int = 2048
    rms_norm_eps: float = 1e-5
    rope_theta: float = 10000.0
    rope_scaling: Optional[RopeScaling] = None
    tie_word_embeddings: bool = False
    attention_bias: bool = False
    mlp_bias: bool = False
    hidden_act: str = "silu"
    torch_dtype: str = "bfloat16"
    bos_token_id: Optional[int] = None
    eos_token_ids: Tuple[int, ...] = ()

    @property
    def q_size(self) -> int:
        return self.num_attention_heads * self.head_dim

    @property
    def kv_size(self) -> int:
        return self.num_key_value_heads * self.head_dim

    @staticmethod
    def from_dict(raw: Mapping[str, Any]) -> "LlamaConfig":
        f = Fields(raw)
        arch = raw.get("architectures", ["LlamaForCausalLM"])[0]
        n_layer = f.integer("num_hidden_layers", hi=100000)
        hidden = f.integer("hidden_size")
        heads = f.integer("num_attention_heads")
        kv_heads = f.integer("num_key_value_heads", default=heads)
        if "head_dim" in raw and raw["head_dim"] is not None:
            head_dim = f.integer("head_dim")
        else:
            if hidden % heads:
                raise ConfigError(
                    f"config.json: hidden_size {hidden} is not a multiple of num_attention_heads "
                    f"{heads} and no head_dim is given")
            head_dim = hidden // heads
        inter = f.integer("intermediate_size")
        vocab = f.integer("vocab_size", hi=1 << 24)
        if not (1 <= kv_heads <= heads):
            raise ConfigError(f"config.json: num_key_value_heads {kv_heads} must be in [1, {heads}]")
        if heads % kv_heads:
            raise ConfigError(
                f"config.json: num_attention_heads {heads} is not a multiple of num_key_value_heads {kv_heads}")
        if heads * head_dim > MAX_AXIS:
            raise ConfigError(f"config.json: heads*head_dim = {heads * head_dim} exceeds {MAX_AXIS}")
        if head_dim % 2:
            raise ConfigError(f"config.json: head_dim {head_dim} must be even for rotary pairs")
        act = f.string("hidden_act", default="silu", choices=("silu",))
        eos = f.int_or_list("eos_token_id", default=())
        bos = raw.get("bos_token_id")
        if bos is not None:
            bos = f.integer("bos_token_id", lo=0, hi=1 << 24)
        return LlamaConfig(
            architecture=arch,
            num_hidden_layers=n_layer,
            hidden_size=hidden,
            num_attention_heads=heads,
            num_key_value_heads=kv_heads,
            head_dim=head_dim,
            intermediate_size=inter,
            vocab_size=vocab,
            max_position_embeddings=f.integer("max_position_embeddings", default=2048, hi=1 << 30),
            rms_norm_eps=f.number("rms_norm_eps", default=1e-5, lo=0.0),
            rope_theta=f.number("rope_theta", default=10000.0, lo=0.0, lo_open=True),
            rope_scaling=RopeScaling.from_fields(f.mapping("rope_scaling")),
            tie_word_embeddings=f.boolean("tie_word_embeddings", default=False),
            attention_bias=f.boolean("attention_bias", default=False),
            mlp_bias=f.boolean("mlp_bias", default=False),
            hidden_act=act,
            torch_dtype=f.string("torch_dtype", default="bfloat16"),
            bos_token_id=bos,
            eos_token_ids=eos,
        )

    def to_dict(self) -> dict:
        """The config.json that reads back as this configuration."""
        d = {
            "architectures": [self.architecture],
            "model_type": "llama",
            "num_hidden_layers": self.num_hidden_layers,
            "hidden_size": self.hidden_size,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "intermediate_size": self.intermediate_size,
            "vocab_size": self.vocab_size,
            "max_position_embeddings": self.max_position_embeddings,
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "rope_scaling": None,
            "tie_word_embeddings": self.tie_word_embeddings,
            "attention_bias": self.attention_bias,
            "mlp_bias": self.mlp_bias,
            "hidden_act": self.hidden_act,
            "torch_dtype": self.torch_dtype,
        }
        if self.rope_scaling is not None:
            rs = asdict(self.rope_scaling)
            if self.rope_scaling.rope_type == "linear":
                rs = {"rope_type": "linear", "factor": self.rope_scaling.factor}
            d["rope_scaling"] = rs
        if self.bos_token_id is not None:
            d["bos_token_id"] = self.bos_token_id
        if self.eos_token_ids:
            d["eos_token_id"] = list(self.eos_token_ids) if len(self.eos_token_ids) > 1 else self.eos_token_ids[0]
        return d
