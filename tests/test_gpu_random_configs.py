"""Falcon configurations drawn at random (fixed seeds) against the plain implementation (GPU).

Sizes the tiny and the published configurations do not hit: head sizes from 16 to 256 that are and are not
built for the matrix cores, head counts and groups that are no power of two, widths that are no multiple
of 64, prime vocabularies, every norm arrangement and fused-row order the configuration allows.
"""
import os
import random

import pytest
import torch

import helpers
from helpers import REL_BF16, REL_F32

pytestmark = pytest.mark.gpu

HEAD_SIZES = [16, 24, 32, 40, 48, 64, 80, 96, 112, 128, 256]
VOCABS = [97, 211, 1009, 4099]


def draw(seed: int) -> dict:
    r = random.Random(seed)
    d = r.choice(HEAD_SIZES)
    new_arch = r.random() < 0.5
    alibi = r.random() < 0.3
    if new_arch:
        nkv = r.choice([1, 2, 3])
        nh = nkv * r.choice([1, 2, 3, 5])
        extra = dict(new_decoder_architecture=True, num_kv_heads=nkv, parallel_attn=True,
                     num_ln_in_parallel_attn=r.choice([1, 2]))
    else:
        nh = r.choice([1, 2, 3, 5, 7, 9])
        extra = dict(new_decoder_architecture=False, multi_query=r.random() < 0.5, parallel_attn=r.random() < 0.6)
    cfg = dict(model_type="falcon", num_hidden_layers=r.choice([1, 2, 3]), hidden_size=nh * d, num_attention_heads=nh,
               ffn_hidden_size=r.choice([nh * d * 2 + 8, nh * d * 3, 200]), vocab_size=r.choice(VOCABS),
               rope_theta=r.choice([10000.0, 500042.0]), max_position_embeddings=1024,
               layer_norm_epsilon=r.choice([1e-5, 1e-6]), bias=r.random() < 0.5, alibi=alibi,
               tie_word_embeddings=r.random() < 0.7, initializer_range=0.02, **extra)
    if not alibi and r.random() < 0.3:
        cfg["rope_scaling"] = {"rope_type": "linear", "factor": r.choice([2.0, 4.0])}
    elif not alibi and r.random() < 0.4:
        cfg["rope_scaling"] = r.choice([
            {"rope_type": "yarn", "factor": 4.0},
            {"rope_type": "yarn", "factor": 8.0, "beta_fast": 16.0, "beta_slow": 2.0, "attention_factor": 0.8},
            {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
             "original_max_position_embeddings": 256}])
    if r.random() < 0.4:
        cfg["activation"] = r.choice(["gelu_new", "silu", "relu", "quick_gelu", "gelu_pytorch_tanh", "relu2", "mish", "tanh"])
    return cfg


# Widths that are no multiple of 8 (no sixteen-byte rows in bfloat16): an odd head size, which only ALiBi allows,
# and head sizes that are no multiple of 8 with an odd number of heads.
ODD = {
    100: dict(model_type="falcon", num_hidden_layers=2, hidden_size=5 * 23, num_attention_heads=5, ffn_hidden_size=201,
              vocab_size=211, max_position_embeddings=512, layer_norm_epsilon=1e-5, new_decoder_architecture=False,
              multi_query=False, parallel_attn=False, bias=True, alibi=True, tie_word_embeddings=True,
              initializer_range=0.02),
    101: dict(model_type="falcon", num_hidden_layers=2, hidden_size=3 * 18, num_attention_heads=3, ffn_hidden_size=90,
              vocab_size=97, rope_theta=10000.0, max_position_embeddings=512, layer_norm_epsilon=1e-6,
              new_decoder_architecture=False, multi_query=True, parallel_attn=True, bias=False, alibi=False,
              tie_word_embeddings=False, initializer_range=0.02),
    102: dict(model_type="falcon", num_hidden_layers=1, hidden_size=7 * 36, num_attention_heads=7, num_kv_heads=1,
              ffn_hidden_size=7 * 36 * 2 + 4, vocab_size=1009, rope_theta=500042.0, max_position_embeddings=512,
              layer_norm_epsilon=1e-5, new_decoder_architecture=True, parallel_attn=True, num_ln_in_parallel_attn=2,
              bias=True, alibi=False, tie_word_embeddings=True, initializer_range=0.02),
}


def test_the_drawn_and_the_odd_configurations_cover_what_they_claim():
    assert all(ODD[k]["hidden_size"] % 8 for k in ODD)
    assert (ODD[100]["hidden_size"] // ODD[100]["num_attention_heads"]) % 2 == 1 and ODD[100]["alibi"]
    assert any(draw(s)["hidden_size"] % 64 for s in range(24))


@pytest.mark.parametrize("seed", list(range(24)) + sorted(ODD))
def test_random_configuration_matches_plain(tmp_path, seed):
    from pytorch_transformers_amd import AutoModelForCausalLM
    from pytorch_transformers_amd.config import AutoConfig
    from pytorch_transformers_amd.engine.replay import Replayer
    from pytorch_transformers_amd.weights import write_random_model

    raw = ODD[seed] if seed in ODD else draw(seed)
    print("configuration:", raw, flush=True)  # names the case before any kernel runs
    cfg = AutoConfig.from_dict(raw)
    folder = write_random_model(os.path.join(str(tmp_path), f"m{seed}"), cfg, seed=seed, noise=0.1)
    reqs = helpers.make_requests(cfg.vocab_size, [3, 66, 37, 130], seed=seed)
    want = helpers.plain_logits(folder, reqs)
    first_f32 = {}
    for dtype, rel in (("float32", REL_F32), ("bfloat16", REL_BF16)):
        model = AutoModelForCausalLM.from_pretrained(folder, dtype=dtype)
        rp = Replayer(model, 1024)
        for sched, records in (("whole", helpers.schedule_whole(reqs)), ("tail32", helpers.schedule_tail(reqs, 32)),
                               ("batches", helpers.schedule_batches(reqs, 3, decode=(1, 20, 5))),
                               ("staggered", helpers.schedule_staggered(reqs, 2, decode=(2, 9, 1, 30), chunks=(1, None, 16, 50)))):
            got = helpers.run_schedule(rp, records)
            for rid in reqs:
                helpers.assert_close(got[rid], want[rid], rel, f"seed {seed} {dtype} {sched} {rid}")
                if dtype == "float32":
                    first = first_f32.setdefault(rid, got[rid])
                    assert torch.equal(got[rid], first), f"seed {seed} float32: {sched} differs from whole for {rid}"
        del rp, model
    torch.cuda.empty_cache()
