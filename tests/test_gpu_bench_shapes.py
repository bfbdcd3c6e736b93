"""The model at the shapes and in the state that ``bench.py`` measures (GPU).

One or two layers at the widths of the published Falcon models, with the plain implementation's float64 tensors on
the GPU (plain torch, nothing of the engine): a prompt of 2,048 tokens, decode steps of 8 and 64 sequences at
contexts of about a thousand tokens, a context past 4,096 at Falcon2-11B widths and decode batches of 40 and 64
rows at Falcon-40B widths.  Each bfloat16 case runs twice over one model: with the built-in choices between
kernels, and after ``model.tune`` has timed them for these shapes (one library product for two matrices, the
ladder of row counts, stationary activations with timed ranges, the timed cut of the decode attention), which is
the state the measurements are taken in.
(The reference's counterparts: tests/models/falcon/test_modeling_falcon.py:203-263, tests/test_modeling_common.py:765-862.)
"""
import os

import pytest
import torch

import helpers
from helpers import REL_BF16, REL_F32

pytestmark = pytest.mark.gpu

WIDTHS = {
    "7b": dict(model_type="falcon", num_hidden_layers=2, hidden_size=4544, num_attention_heads=71,
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


@pytest.fixture(scope="module")
def folder_of(tmp_path_factory):
    """Model folders with random weights, written once per width for the whole file."""
    from pytorch_transformers_amd.config import AutoConfig
    from pytorch_transformers_amd.weights import write_random_model

    root = tmp_path_factory.mktemp("bench_shapes")
    made = {}

    def get(name: str) -> str:
        if name not in made:
            cfg = AutoConfig.from_dict(WIDTHS[name])
            made[name] = write_random_model(os.path.join(str(root), name), cfg, seed=21, noise=0.1)
        return made[name]

    return get


def _decode_records(reqs, checked, tail):
    """All prompts (all but the last ``tail`` tokens of each) in one step, then one token each for ``tail`` steps;
    logits are asked for at the prompt's end and at every later token of the requests in ``checked``."""
    records = [{"step": 0, "end": [], "entries": [
        {"id": rid, "tokens": toks[:-tail], "want": [len(toks) - tail - 1] if rid in checked else []}
        for rid, toks in reqs.items()]}]
    for t in range(tail):
        records.append({"step": t + 1, "end": list(reqs) if t == tail - 1 else [], "entries": [
            {"id": rid, "tokens": [toks[len(toks) - tail + t]], "want": [0] if rid in checked else []}
            for rid, toks in reqs.items()]})
    return records


def _in_both_states(model, check, **tune):
    """``check(state)`` with the built-in choices, then with the timed ones; the table is forgotten afterwards."""
    from pytorch_transformers_amd import ops

    try:
        check("untuned")
        table = model.tune(**tune)
        assert any(table.values()), "nothing was timed"
        check("tuned")
    finally:
        ops.clear_tuning()


def test_a_prompt_of_2048_tokens_at_falcon7b_widths(folder_of):
    """The logits of the last 64 places of a 2,048-token prompt, in 32-bit and in bfloat16 (the prompt attention
    with stages of keys through LDS, the vendor library's products with their epilogue passes and, once timed, the
    joined product and the pieces along the rows)."""
    from pytorch_transformers_amd import AutoModelForCausalLM
    from pytorch_transformers_amd.engine.replay import Replayer

    folder = folder_of("7b")
    reqs = helpers.make_requests(WIDTHS["7b"]["vocab_size"], [2048], seed=31)
    want = helpers.plain_logits_on_gpu(folder, reqs, last=64)["r0"]
    record = {"step": 0, "entries": [{"id": "r0", "tokens": reqs["r0"], "want": list(range(2048 - 64, 2048))}], "end": ["r0"]}
    model = AutoModelForCausalLM.from_pretrained(folder, dtype="float32")
    got = Replayer(model, 2048).run(record).float().cpu()
    helpers.assert_close(got, want, REL_F32, "7b widths, 2,048 tokens, float32")
    del model
    torch.cuda.empty_cache()
    model = AutoModelForCausalLM.from_pretrained(folder, dtype="bfloat16")

    def check(state):
        got = Replayer(model, 2048).run(record).float().cpu()
        helpers.assert_close(got, want, REL_BF16, f"7b widths, 2,048 tokens, bfloat16, {state}")

    _in_both_states(model, check, prompt_lens=(2048,), batches=())


@pytest.mark.parametrize("batch", [8, 64])
def test_decode_batches_at_falcon7b_widths(folder_of, batch):
    """8 and 64 sequences with prompts of unequal lengths around 1,024 tokens, four decoded tokens each, in captured
    steps; three sequences (the first, the longest, the last) against the plain implementation."""
    from pytorch_transformers_amd import AutoModelForCausalLM
    from pytorch_transformers_amd.engine.replay import Replayer

    folder = folder_of("7b")
    lengths = [964 + (53 * i) % 120 for i in range(batch)]
    reqs = helpers.make_requests(WIDTHS["7b"]["vocab_size"], lengths, seed=32 + batch)
    longest = max(range(batch), key=lambda i: lengths[i])
    checked = sorted({"r0", f"r{longest}", f"r{batch - 1}"})
    tail = 4
    want = helpers.plain_logits_on_gpu(folder, {rid: reqs[rid] for rid in checked}, last=tail + 1)
    records = _decode_records(reqs, checked, tail)
    model = AutoModelForCausalLM.from_pretrained(folder, dtype="bfloat16")
    room = sum((n + 63) // 64 * 64 for n in lengths)

    def check(state):
        got = helpers.run_schedule(Replayer(model, room), records)
        for rid in checked:
            helpers.assert_close(got[rid], want[rid], REL_BF16, f"7b widths, batch {batch}, {state}, {rid}")

    _in_both_states(model, check, prompt_lens=(), batches=(batch,), contexts=((max(lengths), sum(lengths) // batch),))


def test_a_context_past_4096_at_falcon2_11b_widths(folder_of):
    """Eight sequences of 2,900 to 4,400 tokens (heads of 128 in eight groups, a large theta): the prompts in one
    step, four decoded tokens, two sequences checked."""
    from pytorch_transformers_amd import AutoModelForCausalLM
    from pytorch_transformers_amd.engine.replay import Replayer

    folder = folder_of("11b")
    lengths = [4400, 2900, 3333, 4097, 3000, 4200, 3650, 4096]
    reqs = helpers.make_requests(WIDTHS["11b"]["vocab_size"], lengths, seed=41)
    checked, tail = ["r0", "r3"], 4
    want = helpers.plain_logits_on_gpu(folder, {rid: reqs[rid] for rid in checked}, last=tail + 1)
    records = _decode_records(reqs, checked, tail)
    model = AutoModelForCausalLM.from_pretrained(folder, dtype="bfloat16")
    room = sum((n + 63) // 64 * 64 for n in lengths)

    def check(state):
        got = helpers.run_schedule(Replayer(model, room), records)
        for rid in checked:
            helpers.assert_close(got[rid], want[rid], REL_BF16, f"11b widths, long contexts, {state}, {rid}")

    _in_both_states(model, check, prompt_lens=(), batches=(8,), contexts=((max(lengths), sum(lengths) // 8),))


@pytest.mark.parametrize("batch", [40, 64])
def test_decode_batches_of_33_to_64_rows_at_falcon40b_widths(folder_of, batch):
    """Decode steps of 40 and 64 sequences at Falcon-40B widths, where the feed-forward's first product leaves the
    pair launch for the vendor library and the fused query_key_value product runs as a launch of its own."""
    from pytorch_transformers_amd import AutoModelForCausalLM
    from pytorch_transformers_amd.engine.replay import Replayer

    folder = folder_of("40b")
    lengths = [150 + (37 * i) % 200 for i in range(batch)]
    reqs = helpers.make_requests(WIDTHS["40b"]["vocab_size"], lengths, seed=51 + batch)
    checked, tail = sorted({"r0", f"r{batch // 2}", f"r{batch - 1}"}), 4
    want = helpers.plain_logits_on_gpu(folder, {rid: reqs[rid] for rid in checked}, last=tail + 1)
    records = _decode_records(reqs, checked, tail)
    model = AutoModelForCausalLM.from_pretrained(folder, dtype="bfloat16")
    room = sum((n + 63) // 64 * 64 for n in lengths)

    def check(state):
        got = helpers.run_schedule(Replayer(model, room), records)
        for rid in checked:
            helpers.assert_close(got[rid], want[rid], REL_BF16, f"40b widths, batch {batch}, {state}, {rid}")

    _in_both_states(model, check, prompt_lens=(), batches=(batch,), contexts=((max(lengths), sum(lengths) // batch),))
