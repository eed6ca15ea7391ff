"""``LlamaForCausalLM``: the Llama dense decoder put together from parts.

Every layer is the same pre-norm block of grouped-query attention with rotary
position encoding and a SiLU-gated feed-forward
(src/model.c:6168-6473); the tensors carry the names of un-permuted
checkpoints, so the rotation pairs element j with j + rotary_dim/2
(src/model.c:1464-1466 explains the other pairing).
"""
from __future__ import annotations

from dataclasses import asdict

from ..config import ExecStep, LayerSpec, LlamaConfig, ModelSpec, PartSpec, register_architecture


def build_llama_spec(cfg: LlamaConfig) -> ModelSpec:
    scaling = asdict(cfg.rope_scaling) if cfg.rope_scaling is not None else None
    position = PartSpec("rotary", {"head_dim": cfg.head_dim, "theta": cfg.rope_theta, "scaling": scaling})
    layers = []
    for i in range(cfg.num_hidden_layers):
        p = f"model.layers.{i}."
        layers.append(LayerSpec(
            mixer=PartSpec("paged_attention", {
                "hidden_size": cfg.hidden_size, "num_heads": cfg.num_attention_heads,
                "num_kv_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
                "position": position, "bias": cfg.attention_bias}, prefix=p + "self_attn."),
            feed_forward=PartSpec("gated_mlp", {
                "hidden_size": cfg.hidden_size, "intermediate_size": cfg.intermediate_size,
                "activation": cfg.hidden_act, "bias": cfg.mlp_bias}, prefix=p + "mlp."),
            norms={
                "mixer_norm": PartSpec("rmsnorm", {"size": cfg.hidden_size, "eps": cfg.rms_norm_eps},
                                       prefix=p + "input_layernorm."),
                "feed_forward_norm": PartSpec("rmsnorm", {"size": cfg.hidden_size, "eps": cfg.rms_norm_eps},
                                              prefix=p + "post_attention_layernorm.")},
            block="prenorm"))
    return ModelSpec(
        architecture=cfg.architecture,
        hidden_size=cfg.hidden_size,
        vocab_size=cfg.vocab_size,
        max_position=cfg.max_position_embeddings,
        embedding=PartSpec("token_embedding", {"vocab_size": cfg.vocab_size, "hidden_size": cfg.hidden_size},
                           prefix="model.embed_tokens."),
        layers=layers,
        order=[ExecStep(i) for i in range(cfg.num_hidden_layers)],
        final_norm=PartSpec("rmsnorm", {"size": cfg.hidden_size, "eps": cfg.rms_norm_eps}, prefix="model.norm."),
        head=PartSpec("linear", {"vocab_size": cfg.vocab_size, "hidden_size": cfg.hidden_size,
                                 "tied": cfg.tie_word_embeddings}, prefix="lm_head."),
        eos_token_ids=cfg.eos_token_ids,
        bos_token_id=cfg.bos_token_id,
    )


register_architecture("LlamaForCausalLM", LlamaConfig.from_dict, build_llama_spec)
