"""Typed configuration of the Falcon architecture.

Field names, defaults and derived values follow
src/transformers/models/falcon/configuration_falcon.py:144-208; which
combinations of the flags can be built follows what the decoder layer creates
and reads (src/transformers/models/falcon/modeling_falcon.py:599-612, :630-666)
and how the fused projection is split (:269-298).
"""
from __future__ import annotations

import dataclasses
from typing import Any, ClassVar, Dict, Optional

from .base import ConfigError, ModelConfig

# how the rows of the fused query_key_value projection are ordered
QKV_GROUPED = "grouped"  # per KV group: its query heads, then k, then v (modeling_falcon.py:281-290)
QKV_TAIL = "tail"  # all query heads, then one k, one v (modeling_falcon.py:296-298)
QKV_INTERLEAVED = "interleaved"  # per head: q, k, v (modeling_falcon.py:292-294)

# which norms a block has and where they stand
NORMS_SINGLE = "single"  # input_layernorm feeds attention and MLP
NORMS_DUAL = "dual"  # ln_attn feeds attention, ln_mlp feeds the MLP
NORMS_SEQUENTIAL = "sequential"  # input_layernorm, then post_attention_layernorm on x + attn

# src/transformers/activations.py:200-220
ACTIVATIONS_BUILT = ("gelu", "gelu_10", "gelu_fast", "gelu_new", "gelu_python", "gelu_pytorch_tanh", "gelu_accurate",
                     "laplace", "leaky_relu", "linear", "mish", "quick_gelu", "relu", "relu2", "relu6", "sigmoid", "silu",
                     "swish", "tanh")
ROPE_TYPES_KNOWN = ("default", "linear", "dynamic", "yarn", "longrope", "llama3")  # modeling_rope_utils.py:351-358
ROPE_TYPES_BUILT = ROPE_TYPES_KNOWN


@dataclasses.dataclass
class FalconConfig(ModelConfig):
    model_type: ClassVar[str] = "falcon"  # configuration_falcon.py:141
    # keys of the older custom-code checkpoints (convert_custom_code_checkpoint.py:43-51)
    key_aliases: ClassVar[Dict[str, str]] = {
        "n_embed": "hidden_size",  # configuration_falcon.py:173-174
        "n_head": "num_attention_heads",
        "n_layer": "num_hidden_layers",
    }

    vocab_size: int = 65024
    hidden_size: int = 4544
    num_hidden_layers: int = 32
    num_attention_heads: int = 71
    num_ln_in_parallel_attn: Optional[int] = None
    layer_norm_epsilon: float = 1e-5
    initializer_range: float = 0.02
    hidden_dropout: float = 0.0
    attention_dropout: float = 0.0
    num_kv_heads: Optional[int] = None
    alibi: bool = False
    new_decoder_architecture: bool = False
    multi_query: bool = True
    parallel_attn: bool = True
    bias: bool = False
    max_position_embeddings: int = 2048
    rope_theta: float = 10000.0
    rope_scaling: Optional[Dict[str, Any]] = None
    ffn_hidden_size: Optional[int] = None
    activation: str = "gelu"
    bos_token_id: Any = 11
    eos_token_id: Any = 11

    @classmethod
    def preprocess_dict(cls, d):
        d = super().preprocess_dict(d)
        # n_head_kv marks the grouped architecture in old files (convert_custom_code_checkpoint.py:47-51)
        if "n_head_kv" in d:
            d["num_kv_heads"] = d.pop("n_head_kv")
            d.setdefault("new_decoder_architecture", True)
        return d

    def normalize(self) -> None:
        if self.num_kv_heads is None:  # configuration_falcon.py:184
            self.num_kv_heads = self.num_attention_heads
        if self.ffn_hidden_size is None:  # configuration_falcon.py:195-198
            self.ffn_hidden_size = 4 * self.hidden_size
        # modeling_falcon.py:599-600
        if self.num_ln_in_parallel_attn is None and self.new_decoder_architecture:
            self.num_ln_in_parallel_attn = 2
        self.rope_theta = float(self.rope_theta)

    def validate(self) -> None:
        for name in ("vocab_size", "hidden_size", "num_hidden_layers", "num_attention_heads", "num_kv_heads",
                     "ffn_hidden_size", "max_position_embeddings"):
            v = getattr(self, name)
            if not isinstance(v, int) or isinstance(v, bool) or v <= 0:
                raise ConfigError(f"{name} must be a positive integer, got {v!r}")
        if self.hidden_size % self.num_attention_heads != 0:  # modeling_falcon.py:243-247
            raise ConfigError(
                f"hidden_size must be divisible by num_attention_heads (got hidden_size={self.hidden_size}, "
                f"num_attention_heads={self.num_attention_heads})")
        if not (self.layer_norm_epsilon > 0):
            raise ConfigError(f"layer_norm_epsilon must be positive, got {self.layer_norm_epsilon!r}")
        if self.activation not in ACTIVATIONS_BUILT:
            raise ConfigError(f"activation {self.activation!r} is not built; built: {ACTIVATIONS_BUILT}")
        if self.num_ln_in_parallel_attn not in (None, 1, 2):
            raise ConfigError(f"num_ln_in_parallel_attn must be None, 1 or 2, got {self.num_ln_in_parallel_attn!r}")
        if self.new_decoder_architecture and not self.parallel_attn:
            # the layer creates input/post norms (:602-604) but reads ln_attn or leaves the MLP input undefined (:630-666)
            raise ConfigError("new_decoder_architecture=true needs parallel_attn=true")
        if not self.new_decoder_architecture and self.parallel_attn and self.num_ln_in_parallel_attn == 2:
            # creates ln_attn/ln_mlp (:606-610) but reads input_layernorm (:634)
            raise ConfigError("num_ln_in_parallel_attn=2 needs new_decoder_architecture=true")
        nkv = self.kv_heads
        if self.num_attention_heads % nkv != 0:
            raise ConfigError(
                f"num_attention_heads ({self.num_attention_heads}) must be a multiple of the KV heads ({nkv})")
        if not self.new_decoder_architecture and not self.multi_query and nkv != self.num_attention_heads:
            # the per-head q,k,v view assumes 3*hidden rows (:292-294)
            raise ConfigError("multi_query=false without new_decoder_architecture needs num_kv_heads == num_attention_heads")
        if not self.alibi:
            if self.head_dim % 2 != 0:
                raise ConfigError(f"rotary positions need an even head size, got {self.head_dim}")
            if self.rope_scaling is not None:
                if not isinstance(self.rope_scaling, dict):
                    raise ConfigError("rope_scaling must be a dict with 'rope_type' (or 'type') and 'factor'")
                kind = self.rope_type
                if kind not in ROPE_TYPES_KNOWN:
                    raise ConfigError(f"rope_scaling type {kind!r} is unknown; known: {ROPE_TYPES_KNOWN}")
                if kind not in ROPE_TYPES_BUILT:
                    raise ConfigError(f"rope_scaling type {kind!r} is not built; built: {ROPE_TYPES_BUILT}")
                def number(key, least=None, required=True):
                    v = self.rope_scaling.get(key)
                    if v is None and not required:
                        return
                    if not isinstance(v, (int, float)) or isinstance(v, bool) or (least is not None and v < least):
                        raise ConfigError(f"rope_scaling {key} must be a number" + (f" >= {least}" if least is not None else "")
                                          + f", got {v!r}")
                if kind in ("linear", "dynamic", "yarn", "llama3"):
                    number("factor", 1.0)  # modeling_rope_utils.py:392-394, :409-411, :432-434, :512-514
                if kind == "dynamic" and self.head_dim <= 2:  # the stretched base has the exponent d / (d - 2) (:157)
                    raise ConfigError("rope_scaling type 'dynamic' needs a head size above 2")
                if kind == "longrope":  # :453-503
                    half = self.head_dim // 2
                    for key in ("short_factor", "long_factor"):
                        v = self.rope_scaling.get(key)
                        if (not isinstance(v, (list, tuple)) or len(v) != half
                                or not all(isinstance(x, (int, float)) and not isinstance(x, bool) and x > 0 for x in v)):
                            raise ConfigError(f"rope_scaling {key} must be a list of {half} positive numbers, got {v!r}")
                    number("attention_factor", 0.0, required=False)
                    original = self.extra.get("original_max_position_embeddings")
                    if original is not None:
                        if not isinstance(original, int) or isinstance(original, bool) or original <= 0:
                            raise ConfigError(f"original_max_position_embeddings must be a positive integer, got {original!r}")
                    elif self.rope_scaling.get("attention_factor") is None:
                        number("factor", 1.0)
                if kind == "yarn":  # :424-450
                    number("attention_factor", 0.0, required=False)
                    number("beta_fast", required=False)
                    number("beta_slow", required=False)
                    if (self.rope_scaling.get("beta_fast") or 32) < (self.rope_scaling.get("beta_slow") or 1):
                        raise ConfigError("rope_scaling beta_fast must not be less than beta_slow")
                if kind == "llama3":  # :505-536
                    number("low_freq_factor")
                    number("high_freq_factor")
                    number("original_max_position_embeddings", 1)
                    if self.rope_scaling["high_freq_factor"] <= self.rope_scaling["low_freq_factor"]:
                        raise ConfigError("rope_scaling high_freq_factor must be greater than low_freq_factor")
        elif self.rope_scaling is not None:  # configuration_falcon.py: alibi and rope scaling exclude each other
            raise ConfigError("rope_scaling is not supported together with alibi")

    # derived ---------------------------------------------------------------
    @property
    def head_dim(self) -> int:  # configuration_falcon.py:202-204
        return self.hidden_size // self.num_attention_heads

    @property
    def rotary(self) -> bool:  # configuration_falcon.py:206-208
        return not self.alibi

    @property
    def kv_heads(self) -> int:
        """KV heads that exist in the weights (modeling_falcon.py:263)."""
        if self.new_decoder_architecture or not self.multi_query:
            return self.num_kv_heads
        return 1

    @property
    def qkv_layout(self) -> str:
        if self.new_decoder_architecture:
            return QKV_GROUPED
        return QKV_TAIL if self.multi_query else QKV_INTERLEAVED

    @property
    def qkv_out_dim(self) -> int:  # modeling_falcon.py:252-257
        return (self.num_attention_heads + 2 * self.kv_heads) * self.head_dim

    @property
    def norm_scheme(self) -> str:
        if not self.parallel_attn:
            return NORMS_SEQUENTIAL
        if self.new_decoder_architecture and self.num_ln_in_parallel_attn == 2:
            return NORMS_DUAL
        return NORMS_SINGLE

    @property
    def rope_type(self) -> str:
        if self.rope_scaling is None:
            return "default"
        return self.rope_scaling.get("rope_type", self.rope_scaling.get("type", "default"))  # modeling_falcon.py:117-120
