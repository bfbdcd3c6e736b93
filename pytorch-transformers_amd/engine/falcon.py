"""The Falcon architecture as a list of parts: the builder registered for ``model_type: falcon``.

Tensor names are the checkpoint's (module tree of
src/transformers/models/falcon/modeling_falcon.py:826-850, :588-612, :221-267, :565-578, :1165-1171,
base prefix ``transformer.`` :782).  Which norms a block has follows the decoder layer's constructor
and forward (:599-612, :630-666); see ``config.falcon.FalconConfig.norm_scheme``.
"""
from __future__ import annotations

import math

from ..config.falcon import NORMS_DUAL, NORMS_SEQUENTIAL, FalconConfig
from ..config.registry import register
from ..parts import (AlibiPositions, AttentionMixer, DenseFeedForward, Embedding, LayerNorm, OutputHead,
                     ParallelBlock, RotaryPositions, SequentialBlock)
from ..parts.positions import llama3_frequencies, longrope_frequencies, yarn_frequencies
from .spec import CACHE_FULL, CacheGroupSpec, LayerCall, ModelSpec

KV_GROUP = "kv"


def rotary_positions(cfg: FalconConfig) -> RotaryPositions:
    """The rotation that ``rope_scaling`` asks for (src/transformers/models/falcon/modeling_falcon.py:112-134)."""
    rs, kind = cfg.rope_scaling or {}, cfg.rope_type
    if kind == "linear":
        return RotaryPositions(cfg.head_dim, cfg.rope_theta, scaling_factor=float(rs["factor"]))
    if kind == "yarn":
        inv, scale = yarn_frequencies(cfg.head_dim, cfg.rope_theta, float(rs["factor"]), cfg.max_position_embeddings,
                                      float(rs.get("beta_fast") or 32), float(rs.get("beta_slow") or 1),
                                      rs.get("attention_factor"))
        return RotaryPositions(cfg.head_dim, cfg.rope_theta, attention_scaling=scale, inv_freq=inv)
    if kind == "llama3":
        inv = llama3_frequencies(cfg.head_dim, cfg.rope_theta, float(rs["factor"]), float(rs["low_freq_factor"]),
                                 float(rs["high_freq_factor"]), int(rs["original_max_position_embeddings"]))
        return RotaryPositions(cfg.head_dim, cfg.rope_theta, inv_freq=inv)
    if kind == "dynamic":
        return RotaryPositions(cfg.head_dim, cfg.rope_theta, dynamic_factor=float(rs["factor"]),
                               trained_positions=cfg.max_position_embeddings)
    if kind == "longrope":
        inv, scale = longrope_frequencies(cfg.head_dim, cfg.rope_theta, rs["short_factor"], rs.get("factor"),
                                          cfg.max_position_embeddings, cfg.extra.get("original_max_position_embeddings"),
                                          rs.get("attention_factor"))
        return RotaryPositions(cfg.head_dim, cfg.rope_theta, attention_scaling=scale, inv_freq=inv)
    return RotaryPositions(cfg.head_dim, cfg.rope_theta)


def build_falcon(cfg: FalconConfig) -> ModelSpec:
    H, L, eps = cfg.hidden_size, cfg.num_hidden_layers, cfg.layer_norm_epsilon
    if cfg.alibi:
        # ``alibi_bf16_compat`` is this library's own key (default true: the reference's rounding of the bias)
        # (the bias is divided by the root of the head size when it is folded into the mask, modeling_falcon.py:1081)
        positions = AlibiPositions(cfg.num_attention_heads, bf16_compat=bool(cfg.extra.get("alibi_bf16_compat", True)),
                                   scale=1.0 / math.sqrt(cfg.head_dim))
    else:
        positions = rotary_positions(cfg)
    blocks = []
    for i in range(L):
        p = f"transformer.h.{i}"
        mixer = AttentionMixer(f"{p}.self_attention", H, cfg.num_attention_heads, cfg.kv_heads, cfg.head_dim,
                               cfg.qkv_layout, cfg.bias, positions)
        ffn = DenseFeedForward(f"{p}.mlp", H, cfg.ffn_hidden_size, cfg.bias, cfg.activation)
        if cfg.norm_scheme == NORMS_SEQUENTIAL:
            block = SequentialBlock(mixer, ffn, LayerNorm(f"{p}.input_layernorm", H, eps),
                                    LayerNorm(f"{p}.post_attention_layernorm", H, eps))
        elif cfg.norm_scheme == NORMS_DUAL:
            block = ParallelBlock(mixer, ffn, LayerNorm(f"{p}.ln_attn", H, eps), LayerNorm(f"{p}.ln_mlp", H, eps))
        else:
            block = ParallelBlock(mixer, ffn, LayerNorm(f"{p}.input_layernorm", H, eps))
        blocks.append(block)
    embed_name = "transformer.word_embeddings"
    return ModelSpec(
        config=cfg,
        embedding=Embedding(embed_name, cfg.vocab_size, H),
        blocks=blocks,
        order=[LayerCall(i, KV_GROUP, i) for i in range(L)],
        final_norm=LayerNorm("transformer.ln_f", H, eps),
        head=OutputHead("lm_head", cfg.vocab_size, H, f"{embed_name}.weight" if cfg.tie_word_embeddings else None),
        cache_groups=[CacheGroupSpec(KV_GROUP, CACHE_FULL, L, cfg.kv_heads, cfg.head_dim)],
        base_prefix="transformer.",  # src/transformers/models/falcon/modeling_falcon.py:782
    )


# "RefinedWeb" and "RefinedWebModel" are what the older custom-code checkpoints call the architecture
# (src/transformers/models/falcon/convert_custom_code_checkpoint.py:38-40)
register("falcon", FalconConfig, build_falcon, exist_ok=True, aliases=("RefinedWebModel", "RefinedWeb"))
