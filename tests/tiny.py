"""Tiny Falcon configurations for tests.  Together they differ in every size and option:
head counts and groups, head sizes, widths and vocabularies that are no power of two, number of
layers, eps, the three fused-QKV row orders, the three norm arrangements, bias, rotary (two
thetas, linear scaling) and ALiBi (power-of-two and other head counts), tied and untied heads."""
import os

TINY = {
    # new architecture, grouped QKV, two norms, rotary
    "A": dict(model_type="falcon", num_hidden_layers=2, hidden_size=64, num_attention_heads=4, num_kv_heads=2,
              ffn_hidden_size=256, vocab_size=512, rope_theta=10000.0, max_position_embeddings=128,
              layer_norm_epsilon=1e-5, new_decoder_architecture=True, parallel_attn=True,
              num_ln_in_parallel_attn=2, bias=False, alibi=False, tie_word_embeddings=True, initializer_range=0.02),
    # RW style: per-head q,k,v rows, sequential norms, bias, ALiBi with 6 heads (not a power of two)
    "B": dict(model_type="falcon", num_hidden_layers=3, hidden_size=144, num_attention_heads=6,
              ffn_hidden_size=576, vocab_size=1000, max_position_embeddings=256, layer_norm_epsilon=1e-6,
              new_decoder_architecture=False, multi_query=False, parallel_attn=False, bias=True, alibi=True,
              tie_word_embeddings=True, initializer_range=0.02),
    # 7B style: one KV head at the tail, one norm, 7 heads
    "C": dict(model_type="falcon", num_hidden_layers=2, hidden_size=112, num_attention_heads=7,
              ffn_hidden_size=320, vocab_size=777, rope_theta=10000.0, max_position_embeddings=512,
              layer_norm_epsilon=1e-5, new_decoder_architecture=False, multi_query=True, parallel_attn=True,
              bias=False, alibi=False, tie_word_embeddings=True, initializer_range=0.02),
    # 11B style: new architecture with one norm, wide heads, large theta, untied head, linear rope scaling
    "D": dict(model_type="falcon", num_hidden_layers=2, hidden_size=256, num_attention_heads=2, num_kv_heads=1,
              ffn_hidden_size=384, vocab_size=300, rope_theta=500042.0, max_position_embeddings=8192,
              layer_norm_epsilon=1e-5, new_decoder_architecture=True, parallel_attn=True,
              num_ln_in_parallel_attn=1, bias=True, alibi=False, tie_word_embeddings=False,
              rope_scaling={"rope_type": "linear", "factor": 2.0}, initializer_range=0.02),
    # ALiBi with 20 heads: slopes that bfloat16 rounds, and (in long tests) positions past 256
    "E": dict(model_type="falcon", num_hidden_layers=1, hidden_size=320, num_attention_heads=20,
              ffn_hidden_size=160, vocab_size=211, max_position_embeddings=1024, layer_norm_epsilon=1e-5,
              new_decoder_architecture=False, multi_query=False, parallel_attn=True, bias=False, alibi=True,
              tie_word_embeddings=True, initializer_range=0.02),
}

# frequencies that follow the sequence's length: a trained context of 48 positions, so that short tests cross it
DYNAMIC = dict(model_type="falcon", num_hidden_layers=2, hidden_size=96, num_attention_heads=3, num_kv_heads=1,
               ffn_hidden_size=136, vocab_size=211, rope_theta=10000.0, max_position_embeddings=48,
               layer_norm_epsilon=1e-5, new_decoder_architecture=True, parallel_attn=True, num_ln_in_parallel_attn=1,
               bias=False, alibi=False, tie_word_embeddings=True, initializer_range=0.02,
               rope_scaling={"rope_type": "dynamic", "factor": 4.0})
# LongRoPE: a factor per frequency, and a factor on cosines and sines
LONGROPE = dict(model_type="falcon", num_hidden_layers=2, hidden_size=80, num_attention_heads=5,
                ffn_hidden_size=96, vocab_size=97, rope_theta=500042.0, max_position_embeddings=64,
                layer_norm_epsilon=1e-5, new_decoder_architecture=False, multi_query=True, parallel_attn=True,
                bias=True, alibi=False, tie_word_embeddings=False, initializer_range=0.02,
                rope_scaling={"rope_type": "longrope", "factor": 4.0, "short_factor": [1.0, 1.1, 1.3, 1.6, 2.0, 2.5, 3.1, 3.8],
                              "long_factor": [1.0, 2.0, 3.0, 4.0, 5.0, 6.0, 7.0, 8.0]})

TINY["F"] = LONGROPE
SEEDS = {"A": 0, "B": 1, "C": 2, "D": 3, "E": 4, "F": 5}


LIVELY_STD = 0.2


def write_model(name: str, folder: str, noise: float = 0.1, std=None) -> str:
    """Write tiny model ``name`` with the framework's random-weights mode; returns the folder.

    ``std`` (default: the configuration's ``initializer_range``, 0.02): with weights that small and a tied head a
    tiny model's likeliest next token is its last token over and over, whatever its layers do; tests that compare
    generated tokens pass ``LIVELY_STD``, with which greedy tokens keep changing."""
    from pytorch_transformers_amd.config import AutoConfig
    from pytorch_transformers_amd.weights import write_random_model

    cfg = AutoConfig.from_dict(TINY[name])
    sub = name if std is None else f"{name}-std{std}"
    return write_random_model(os.path.join(folder, sub), cfg, SEEDS[name], noise=noise, std=std)


def write_config(raw: dict, folder: str, name: str, seed: int, noise: float = 0.1, std=None) -> str:
    """Write a model of the configuration ``raw`` (a dict as config.json holds it); returns the folder."""
    from pytorch_transformers_amd.config import AutoConfig
    from pytorch_transformers_amd.weights import write_random_model

    return write_random_model(os.path.join(folder, name), AutoConfig.from_dict(raw), seed, noise=noise, std=std)
