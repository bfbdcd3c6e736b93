"""The engine at the layer sizes of the published Falcon models (GPU).

One layer of each geometry, so that the weights stay small enough for the float64 plain
implementation on the CPU: Falcon-7B (71 heads on one KV head at the tail, width 4544, the full
vocabulary of 65024), Falcon2-11B (32 heads in 8 groups of head size 128, one norm, large theta) and
Falcon-40B (128 heads in 8 groups, two norms, width 8192).  Every way of cutting the work is compared
with the plain logits, in 32-bit and in bfloat16.
"""
import os

import pytest
import torch

import helpers
from helpers import REL_BF16, REL_F32

pytestmark = pytest.mark.gpu

SIZES = {
    "7b": dict(model_type="falcon", num_hidden_layers=1, hidden_size=4544, num_attention_heads=71,
               ffn_hidden_size=18176, vocab_size=65024, rope_theta=10000.0, max_position_embeddings=2048,
               layer_norm_epsilon=1e-5, new_decoder_architecture=False, multi_query=True, parallel_attn=True,
               bias=False, alibi=False, tie_word_embeddings=True, initializer_range=0.02),
    "11b": dict(model_type="falcon", num_hidden_layers=1, hidden_size=4096, num_attention_heads=32, num_kv_heads=8,
                ffn_hidden_size=16384, vocab_size=4099, rope_theta=500042.0, max_position_embeddings=8192,
                layer_norm_epsilon=1e-5, new_decoder_architecture=True, parallel_attn=True,
                num_ln_in_parallel_attn=1, bias=False, alibi=False, tie_word_embeddings=False,
                initializer_range=0.02),
    "40b": dict(model_type="falcon", num_hidden_layers=1, hidden_size=8192, num_attention_heads=128, num_kv_heads=8,
                ffn_hidden_size=32768, vocab_size=4099, rope_theta=10000.0, max_position_embeddings=2048,
                layer_norm_epsilon=1e-5, new_decoder_architecture=True, parallel_attn=True,
                num_ln_in_parallel_attn=2, bias=False, alibi=False, tie_word_embeddings=False,
                initializer_range=0.02),
}
LENGTHS = [41, 9, 70]


@pytest.mark.parametrize("name", sorted(SIZES))
def test_layer_sizes_match_plain(tmp_path, name):
    from pytorch_transformers_amd import AutoModelForCausalLM
    from pytorch_transformers_amd.config import AutoConfig
    from pytorch_transformers_amd.engine.replay import Replayer
    from pytorch_transformers_amd.weights import write_random_model

    cfg = AutoConfig.from_dict(SIZES[name])
    folder = write_random_model(os.path.join(str(tmp_path), name), cfg, seed=11, noise=0.1)
    reqs = helpers.make_requests(cfg.vocab_size, LENGTHS, seed=5)
    want = helpers.plain_logits(folder, reqs)
    first_f32 = {}
    for dtype, rel in (("float32", REL_F32), ("bfloat16", REL_BF16)):
        model = AutoModelForCausalLM.from_pretrained(folder, dtype=dtype)
        rp = Replayer(model, 1024)
        for sched, records in (("whole", helpers.schedule_whole(reqs)), ("tail32", helpers.schedule_tail(reqs, 32)),
                               ("batches", helpers.schedule_batches(reqs, 2, decode=(3, 9))),
                               ("staggered", helpers.schedule_staggered(reqs, 2, decode=(6, 2, 11), chunks=(None, 5, 19)))):
            got = helpers.run_schedule(rp, records)
            for rid in reqs:
                helpers.assert_close(got[rid], want[rid], rel, f"{name} {dtype} {sched} {rid}")
                if dtype == "float32":
                    first = first_f32.setdefault(rid, got[rid])
                    assert torch.equal(got[rid], first), f"{name} float32: {sched} differs from whole for {rid}"
        del rp, model
        torch.cuda.empty_cache()


@pytest.mark.parametrize("heads", [50, 71])
def test_many_heads_on_one_kv_head_in_a_large_batch(tmp_path, heads):
    """Decode steps of 24 sequences of some 900 tokens with 50 and with 71 heads on one KV head of 64: the launch
    walks keys enough for the cut whose workgroups share their keys through LDS (four and five waves of one tile
    of heads), in captured steps as generation runs them.  Logits of three of the sequences, at their prompts'
    ends and at four decoded tokens, against the plain implementation."""
    from pytorch_transformers_amd import AutoModelForCausalLM, ops
    from pytorch_transformers_amd.config import AutoConfig
    from pytorch_transformers_amd.engine.replay import Replayer
    from pytorch_transformers_amd.weights import write_random_model

    cfg = AutoConfig.from_dict(dict(
        model_type="falcon", num_hidden_layers=2, hidden_size=heads * 64, num_attention_heads=heads, ffn_hidden_size=192,
        vocab_size=503, rope_theta=10000.0, max_position_embeddings=2048, layer_norm_epsilon=1e-5,
        new_decoder_architecture=False, multi_query=True, parallel_attn=True, bias=False, alibi=False,
        tie_word_embeddings=True, initializer_range=0.02))
    folder = write_random_model(os.path.join(str(tmp_path), f"mqa{heads}"), cfg, seed=3, noise=0.1)
    lengths = [850 + (37 * i) % 100 for i in range(24)]
    reqs = helpers.make_requests(cfg.vocab_size, lengths, seed=9)
    checked = ["r0", "r11", "r23"]
    want = helpers.plain_logits(folder, {rid: reqs[rid] for rid in checked})
    assert ops.decode_plan(24, heads, 1, 64, max(lengths), sum(lengths) // 24)[2] == ops.SHARED_KEYS
    tail = 4
    records = [{"step": 0, "end": [], "entries": [
        {"id": rid, "tokens": toks[:-tail], "want": [len(toks) - tail - 1] if rid in checked else []}
        for rid, toks in reqs.items()]}]
    for t in range(tail):
        records.append({"step": t + 1, "end": list(reqs) if t == tail - 1 else [], "entries": [
            {"id": rid, "tokens": [toks[len(toks) - tail + t]], "want": [0] if rid in checked else []}
            for rid, toks in reqs.items()]})
    model = AutoModelForCausalLM.from_pretrained(folder, dtype="bfloat16")
    got = helpers.run_schedule(Replayer(model, sum((n + 63) // 64 * 64 for n in lengths)), records)
    for rid in checked:
        helpers.assert_close(got[rid], want[rid][-tail - 1:], REL_BF16, f"{heads} heads, {rid}")
