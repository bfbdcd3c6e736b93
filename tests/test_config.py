"""Configuration and registry (no GPU)."""
import json

import pytest

from pytorch_transformers_amd.config import (AutoConfig, ConfigError, FalconConfig, GenerationConfig, known_model_types,
                                             lookup, register, unregister)
from pytorch_transformers_amd.config.base import ModelConfig
from tiny import TINY


def test_defaults_are_falcon_7b():
    # src/transformers/models/falcon/configuration_falcon.py:144-170
    c = FalconConfig()
    assert (c.vocab_size, c.hidden_size, c.num_hidden_layers, c.num_attention_heads) == (65024, 4544, 32, 71)
    assert c.num_kv_heads == 71 and c.kv_heads == 1  # multi_query: one KV head exists in the weights
    assert c.ffn_hidden_size == 4 * 4544 and c.head_dim == 64 and c.rotary and not c.alibi
    assert c.qkv_layout == "tail" and c.qkv_out_dim == 4544 + 2 * 64 and c.norm_scheme == "single"
    assert c.layer_norm_epsilon == 1e-5 and c.rope_theta == 10000.0 and c.bos_token_id == 11 and c.eos_token_id == 11
    assert c.tie_word_embeddings is True and c.activation == "gelu" and c.max_position_embeddings == 2048


def test_layouts_and_norm_schemes():
    a = AutoConfig.from_dict(TINY["A"])
    assert (a.qkv_layout, a.norm_scheme, a.kv_heads, a.qkv_out_dim, a.num_ln_in_parallel_attn) == ("grouped", "dual", 2, 128, 2)
    b = AutoConfig.from_dict(TINY["B"])
    assert (b.qkv_layout, b.norm_scheme, b.kv_heads, b.qkv_out_dim, b.head_dim) == ("interleaved", "sequential", 6, 432, 24)
    d = AutoConfig.from_dict(TINY["D"])
    assert (d.qkv_layout, d.norm_scheme, d.rope_type) == ("grouped", "single", "linear")
    # 40B-like: new architecture ignores multi_query
    c = FalconConfig(hidden_size=512, num_attention_heads=8, num_kv_heads=2, new_decoder_architecture=True, multi_query=True)
    assert c.kv_heads == 2 and c.norm_scheme == "dual"


def test_aliases_and_legacy_keys():
    c = AutoConfig.from_dict({"model_type": "RefinedWeb", "n_embed": 128, "n_head": 8, "n_layer": 3, "n_head_kv": 2})
    assert (c.hidden_size, c.num_attention_heads, c.num_hidden_layers, c.num_kv_heads) == (128, 8, 3, 2)
    assert c.new_decoder_architecture is True
    c = AutoConfig.from_dict({"model_type": "RefinedWebModel", "n_head": 4, "hidden_size": 64})
    assert c.new_decoder_architecture is False and c.multi_query is True


def test_unknown_keys_are_kept_and_round_trip(tmp_path):
    d = dict(TINY["A"], some_future_key=[1, 2], architectures=["FalconForCausalLM"], torch_dtype="bfloat16")
    c = AutoConfig.from_dict(d)
    assert c.extra == {"some_future_key": [1, 2]}
    c.save_pretrained(str(tmp_path))
    again = AutoConfig.from_pretrained(str(tmp_path))
    assert again == c and again.to_dict()["some_future_key"] == [1, 2]
    assert json.load(open(tmp_path / "config.json"))["model_type"] == "falcon"


@pytest.mark.parametrize("bad,match", [
    (dict(hidden_size=100, num_attention_heads=7), "divisible"),
    (dict(new_decoder_architecture=True, parallel_attn=False), "parallel_attn"),
    (dict(new_decoder_architecture=False, parallel_attn=True, num_ln_in_parallel_attn=2), "num_ln_in_parallel_attn"),
    (dict(new_decoder_architecture=False, multi_query=False, num_kv_heads=2, num_attention_heads=8, hidden_size=64), "multi_query=false"),
    (dict(new_decoder_architecture=True, num_attention_heads=8, num_kv_heads=3, hidden_size=64), "multiple"),
    (dict(activation="gelu_typo"), "activation"),
    (dict(hidden_size=66, num_attention_heads=22), "even head size"),
    (dict(rope_scaling={"rope_type": "dynamic", "factor": 0.5}), "factor"),
    (dict(rope_scaling={"rope_type": "dynamic"}), "factor"),
    (dict(hidden_size=8, num_attention_heads=4, rope_scaling={"rope_type": "dynamic", "factor": 2.0}), "head size above 2"),
    (dict(rope_scaling={"rope_type": "longrope", "factor": 2.0}), "short_factor"),
    (dict(hidden_size=64, num_attention_heads=4,
          rope_scaling={"rope_type": "longrope", "factor": 2.0, "short_factor": [1.0] * 8, "long_factor": [1.0] * 7}), "long_factor"),
    (dict(hidden_size=64, num_attention_heads=4,
          rope_scaling={"rope_type": "longrope", "short_factor": [1.0] * 8, "long_factor": [1.0] * 8}), "factor"),
    (dict(rope_scaling={"rope_type": "yarn", "factor": 0.5}), "factor"),
    (dict(rope_scaling={"rope_type": "yarn", "factor": 2.0, "beta_fast": 1.0, "beta_slow": 4.0}), "beta_fast"),
    (dict(rope_scaling={"rope_type": "llama3", "factor": 8.0}), "low_freq_factor"),
    (dict(rope_scaling={"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 4.0, "high_freq_factor": 1.0,
                        "original_max_position_embeddings": 512}), "high_freq_factor"),
    (dict(rope_scaling={"type": "bogus", "factor": 2.0}), "unknown"),
    (dict(rope_scaling={"type": "linear", "factor": 0.5}), "factor"),
    (dict(alibi=True, rope_scaling={"type": "linear", "factor": 2.0}), "alibi"),
    (dict(vocab_size=0), "positive"),
    (dict(layer_norm_epsilon=0.0), "epsilon"),
])
def test_invalid_combinations_are_rejected(bad, match):
    with pytest.raises(ConfigError, match=match):
        FalconConfig(**bad)


def test_every_rope_type_and_activation_of_the_reference_is_built():
    """modeling_rope_utils.py:351-358 and activations.py:200-220: nothing that a Falcon config.json may name is refused."""
    from pytorch_transformers_amd.config.falcon import ACTIVATIONS_BUILT, ROPE_TYPES_BUILT

    assert set(ROPE_TYPES_BUILT) == {"default", "linear", "dynamic", "yarn", "longrope", "llama3"}
    assert len(ACTIVATIONS_BUILT) == 19 and "laplace" in ACTIVATIONS_BUILT
    FalconConfig(rope_scaling={"rope_type": "dynamic", "factor": 2.0})
    FalconConfig(hidden_size=64, num_attention_heads=4,
                 rope_scaling={"rope_type": "longrope", "short_factor": [1.0] * 8, "long_factor": [2.0] * 8, "attention_factor": 1.1})
    AutoConfig.from_dict(dict(model_type="falcon", hidden_size=64, num_attention_heads=4, original_max_position_embeddings=512,
                              rope_scaling={"rope_type": "longrope", "short_factor": [1.0] * 8, "long_factor": [2.0] * 8}))


def test_odd_head_size_is_fine_with_alibi():
    assert FalconConfig(hidden_size=66, num_attention_heads=22, alibi=True).head_dim == 3


def test_registry():
    assert "falcon" in known_model_types()
    with pytest.raises(ConfigError, match="not registered.*falcon"):
        AutoConfig.from_dict({"model_type": "llama"})
    with pytest.raises(ConfigError, match="model_type"):
        AutoConfig.from_dict({"hidden_size": 8})
    with pytest.raises(ValueError, match="already registered"):
        register("falcon", FalconConfig, lambda c: None)

    import dataclasses

    @dataclasses.dataclass
    class ToyConfig(ModelConfig):
        model_type = "toy-registry-test"
        width: int = 8

    with pytest.raises(ValueError, match="must equal"):
        register("other-name", ToyConfig, lambda c: None)
    register("toy-registry-test", ToyConfig, lambda c: ("built", c.width))
    try:
        cfg = AutoConfig.from_dict({"model_type": "toy-registry-test", "width": 5, "tie_word_embeddings": False})
        assert isinstance(cfg, ToyConfig) and cfg.width == 5 and cfg.tie_word_embeddings is False
        assert lookup("toy-registry-test")[1](cfg) == ("built", 5)
    finally:
        unregister("toy-registry-test")


def test_falcon_builder_lists_the_checkpoint_tensors():
    _, builder = lookup("falcon")
    names = {s.name: s for s in builder(AutoConfig.from_dict(TINY["A"])).tensor_specs()}
    assert names["transformer.h.1.self_attention.query_key_value.weight"].shape == (128, 64)
    assert names["transformer.h.0.ln_attn.weight"].shape == (64,) and "transformer.h.0.ln_mlp.bias" in names
    assert "transformer.h.0.input_layernorm.weight" not in names
    assert names["lm_head.weight"].tied_to == "transformer.word_embeddings.weight"
    assert not any(n.endswith("query_key_value.bias") for n in names)
    names_b = {s.name: s for s in builder(AutoConfig.from_dict(TINY["B"])).tensor_specs()}
    assert names_b["transformer.h.2.self_attention.query_key_value.bias"].shape == (432,)
    assert "transformer.h.0.post_attention_layernorm.weight" in names_b and "transformer.ln_f.bias" in names_b
    assert names_b["transformer.h.0.mlp.dense_4h_to_h.weight"].shape == (144, 576)
    names_d = {s.name: s for s in builder(AutoConfig.from_dict(TINY["D"])).tensor_specs()}
    assert names_d["lm_head.weight"].tied_to is None


def test_generation_config():
    g = GenerationConfig()
    # src/transformers/generation/configuration_utils.py:391-507
    assert (g.max_length, g.max_new_tokens, g.do_sample, g.temperature, g.top_k, g.top_p, g.repetition_penalty) == \
        (20, None, False, 1.0, 50, 1.0, 1.0)
    assert GenerationConfig(eos_token_id=[3, 5]).eos_token_ids == [3, 5] and GenerationConfig(eos_token_id=7).eos_token_ids == [7]
    with pytest.raises(ValueError, match="strictly positive float"):
        GenerationConfig(do_sample=True, temperature=0.0)
    with pytest.raises(ValueError, match="top_p"):
        GenerationConfig(do_sample=True, top_p=1.5)
    with pytest.raises(ValueError, match="typical_p"):
        GenerationConfig(do_sample=True, typical_p=0.0)
    assert (g.typical_p, g.epsilon_cutoff, g.eta_cutoff) == (1.0, 0.0, 0.0)  # configuration_utils.py:423-425
    with pytest.raises(ValueError, match="num_return_sequences"):
        GenerationConfig(do_sample=False, num_return_sequences=2)
    with pytest.raises(ValueError, match="num_beams"):
        GenerationConfig(num_beams=4)
    with pytest.raises(ValueError, match="max_new_tokens"):
        GenerationConfig(max_new_tokens=0)
    with pytest.raises(ValueError, match="unknown generation option"):
        g.updated(bogus=1)
    assert g.updated(max_new_tokens=5).max_new_tokens == 5 and g.max_new_tokens is None
    fm = GenerationConfig.from_model_config(FalconConfig())
    assert (fm.bos_token_id, fm.eos_token_id, fm.pad_token_id) == (11, 11, None)


def test_generation_config_from_folder(tmp_path):
    (tmp_path / "generation_config.json").write_text(json.dumps(
        {"eos_token_id": 2, "bos_token_id": 1, "do_sample": True, "temperature": 0.7, "transformers_version": "4.33"}))
    g = GenerationConfig.from_pretrained(str(tmp_path))
    assert (g.eos_token_id, g.do_sample, g.temperature) == (2, True, 0.7)


def test_options_that_are_not_built_are_refused_by_name_and_the_rest_is_kept(tmp_path):
    """A ``generation_config.json`` that names an option which would change the tokens and is not built raises with
    the option's name and the file's; options that change nothing here are kept and written back."""
    path = tmp_path / "generation_config.json"
    harmless = {"eos_token_id": 2, "max_length": 30, "transformers_version": "4.33", "length_penalty": 2.0,
                "early_stopping": True, "num_beam_groups": 1, "penalty_alpha": None, "_from_model_config": True}
    path.write_text(json.dumps(harmless))
    g = GenerationConfig.from_pretrained(str(tmp_path))
    assert g.max_length == 30 and g.extra["length_penalty"] == 2.0 and g.extra["transformers_version"] == "4.33"
    assert g.to_dict()["early_stopping"] is True and GenerationConfig.from_dict(g.to_dict()) == g
    for bad in ({"forced_bos_token_id": 1}, {"penalty_alpha": 0.6, "top_k": 4}, {"num_beams": 4},
                {"encoder_repetition_penalty": 1.3}, {"prompt_lookup_num_tokens": 3}, {"guidance_scale": 1.5},
                {"watermarking_config": {"bias": 2.0}}, {"output_attentions": True}, {"diversity_penalty": 0.5}):
        path.write_text(json.dumps(dict(harmless, **bad)))
        name = next(k for k in bad if k != "top_k")
        with pytest.raises(ValueError, match=f"(?s)generation_config.json.*not built.*{name}"):
            GenerationConfig.from_pretrained(str(tmp_path))
    with pytest.raises(ValueError, match="arguments of generate.*guidance_scale"):
        g.updated(guidance_scale=2.0)
    path.write_text(json.dumps({"do_sample": True, "temperature": 0.0}))
    with pytest.raises(ValueError, match="generation_config.json.*temperature"):  # a bad value names its file too
        GenerationConfig.from_pretrained(str(tmp_path))


def test_bias_forced_token_and_decay_options():
    from pytorch_transformers_amd.sampling.bans import BiasRules

    g = GenerationConfig(sequence_bias={(5, 6): -2.0, (7,): 1.5}, forced_eos_token_id=3,
                         exponential_decay_length_penalty=(4, 1.1))
    assert g.sequence_bias == [[[5, 6], -2.0], [[7], 1.5]] and g.forced_eos_token_ids == [3]
    assert g.exponential_decay_length_penalty == [4, 1.1] and GenerationConfig.from_dict(json.loads(json.dumps(g.to_dict()))) == g
    for bad, match in (({"sequence_bias": []}, "non-empty"), ({"sequence_bias": [[[1, 2], 3]]}, "positive integers and float"),
                       ({"sequence_bias": [[[], 1.0]]}, "positive integers and float"), ({"sequence_bias": {"a": 1.0}}, "tuples as keys"),
                       ({"forced_eos_token_id": -1}, "positive integers"), ({"forced_eos_token_id": [2, 1.5]}, "positive integers"),
                       ({"exponential_decay_length_penalty": [1.5, 2.0]}, "start_index"),
                       ({"exponential_decay_length_penalty": [3, -1.0]}, "start_index")):
        with pytest.raises(ValueError, match=match):
            GenerationConfig(**bad)
    # tests/generation/test_logits_process.py:604-629 on the host's rule
    rules = BiasRules([[[1], 100.0], [[4], 100.0], [[1, 0], -100.0], [[0, 1, 2], -100.0], [[1, 3, 1, 3], -100.0],
                       [[1, 3, 1, 3, 1, 3], -100.0]], vocab_size=5)
    assert rules.biases([0, 1, 3, 1]) == [(0, -100.0), (1, 100.0), (3, -100.0), (4, 100.0)]
    assert rules.biases([0, 1, 0, 1]) == [(0, -100.0), (1, 100.0), (2, -100.0), (4, 100.0)]
    both = BiasRules([[[3, 1], 1.5], [[2, 3, 1], 2.0], [[1], 0.25]])
    assert both.biases([9, 2, 3]) == [(1, 3.75)] and both.biases([2, 3]) == [(1, 1.75)] and both.needs_history
    assert not BiasRules([[[1], 0.5]]).needs_history and BiasRules([[[1], 0.5]]).biases(None) == [(1, 0.5)] and not BiasRules()
    with pytest.raises(ValueError, match="vocabulary size is 5"):
        BiasRules([[[1, 7], 1.0]], vocab_size=5)


def test_command_line_refuses_what_it_cannot_do_before_anything_is_loaded(capsys):
    """``--use_cpu`` and ``--xlm_language`` of the reference's example (run_generation.py:319-330) are known and refused
    with a reason, without a model or a GPU."""
    from pytorch_transformers_amd.run_generation import main

    assert main(["--use_cpu", "--prompt_ids", "1"]) == 2
    assert "no CPU path" in capsys.readouterr().err
    assert main(["--xlm_language", "en", "--prompt_ids", "1"]) == 2
    assert "another architecture" in capsys.readouterr().err
