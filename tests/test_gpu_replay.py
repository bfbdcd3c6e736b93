"""Engine against the plain implementation, for every way of cutting the work (GPU)."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import helpers
from helpers import REL_BF16, REL_F32
from tiny import TINY, write_config, write_model

pytestmark = pytest.mark.gpu

LENGTHS = {"A": [5, 11, 17, 40, 70, 33], "B": [1, 7, 20, 33, 65, 129], "C": [64, 3, 47, 90, 128, 66],
           "D": [37, 12, 80, 5, 64, 100], "E": [9, 50, 130, 3, 64, 77], "F": [70, 2, 64, 31, 100, 65]}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    root = str(tmp_path_factory.mktemp("models"))
    return {name: write_model(name, root) for name in TINY}


@pytest.fixture(scope="module")
def plain_cache():
    return {}


def _plain(folders, plain_cache, name):
    if name not in plain_cache:
        reqs = helpers.make_requests(TINY[name]["vocab_size"], LENGTHS[name], seed=100 + ord(name))
        plain_cache[name] = (reqs, helpers.plain_logits(folders[name], reqs))
    return plain_cache[name]


def _replayer(folder, dtype, max_tokens=2048):
    from pytorch_transformers_amd import AutoModelForCausalLM
    from pytorch_transformers_amd.engine.replay import Replayer

    model = AutoModelForCausalLM.from_pretrained(folder, dtype=dtype)
    return Replayer(model, max_tokens)


@pytest.mark.parametrize("dtype,rel", [("float32", REL_F32), ("bfloat16", REL_BF16)])
@pytest.mark.parametrize("name", sorted(TINY))
def test_schedules_match_plain(folders, plain_cache, name, dtype, rel):
    """Whole / last 32 one by one / unequal batches with slot reuse / requests that join while others decode, with
    prompts in pieces: all equal the plain logits."""
    reqs, want = _plain(folders, plain_cache, name)
    rp = _replayer(folders[name], dtype)
    results = {}
    for sched_name, records in (("whole", helpers.schedule_whole(reqs)),
                                ("tail32", helpers.schedule_tail(reqs, 32)),
                                ("batches", helpers.schedule_batches(reqs, 4)),
                                ("batches-again", helpers.schedule_batches(reqs, 3, decode=(20, 2, 7))),
                                ("staggered", helpers.schedule_staggered(reqs)),
                                ("staggered-again", helpers.schedule_staggered(reqs, 1, decode=(1, 30, 3), chunks=(7, None, 64)))):
        got = helpers.run_schedule(rp, records)
        assert not rp.slots and not rp.cache.live_slots(), "slots left behind"
        assert rp.cache.free_pages() == rp.cache.num_pages, "pages left behind"
        for rid in reqs:
            helpers.assert_close(got[rid], want[rid], rel, f"{name} {dtype} {sched_name} {rid} (len {len(reqs[rid])})")
        results[sched_name] = got
    if dtype == "float32":
        # fixed summation orders: how the tokens were cut and batched changes no bit
        for sched_name in ("tail32", "batches", "batches-again", "staggered", "staggered-again"):
            for rid in reqs:
                assert torch.equal(results[sched_name][rid], results["whole"][rid]), \
                    f"{name} float32: {sched_name} differs from whole for {rid}"


@pytest.mark.parametrize("dtype,rel", [("float32", REL_F32), ("bfloat16", REL_BF16)])
def test_frequencies_that_follow_each_sequences_length(tmp_path, dtype, rel):
    """``rope_scaling: dynamic`` with a trained context of 48 positions: every piece of a sequence is rotated by the
    frequencies of the length reached with it, each sequence by its own length whatever else the step holds, and
    what is in the cache stays as it was rotated.  The plain logits are computed for the pieces of each schedule;
    sequences that stay within the trained context equal the model without scaling."""
    from pytorch_transformers_amd import AutoModelForCausalLM
    from pytorch_transformers_amd.engine.replay import Replayer
    from tiny import DYNAMIC, write_config

    folder = write_config(DYNAMIC, str(tmp_path), "dyn", seed=6)
    reqs = helpers.make_requests(DYNAMIC["vocab_size"], [30, 70, 100, 49, 48, 130], seed=21)
    model = AutoModelForCausalLM.from_pretrained(folder, dtype=dtype)
    rp = Replayer(model, 1024)
    seen = {}
    for sched_name, records in (("whole", helpers.schedule_whole(reqs)), ("tail32", helpers.schedule_tail(reqs, 32)),
                                ("batches", helpers.schedule_batches(reqs, 4, decode=(3, 25, 1, 14))),
                                ("staggered", helpers.schedule_staggered(reqs, 2, decode=(6, 2, 60, 4), chunks=(None, 40, 19, 1)))):
        want = helpers.plain_logits_as_fed(folder, reqs, records)
        got = helpers.run_schedule(rp, records)
        for rid in reqs:
            helpers.assert_close(got[rid], want[rid], rel, f"dynamic {dtype} {sched_name} {rid} (len {len(reqs[rid])})")
        seen[sched_name] = got
    if dtype == "float32":
        # the schedules do differ where a sequence crossed the trained context in pieces ...
        assert not torch.allclose(seen["tail32"]["r2"], seen["whole"]["r2"], atol=1e-4)
        # ... and do not where it never left it: bitwise the same, and the unscaled model's logits
        for rid in ("r0", "r4"):
            for sched_name in ("tail32", "batches", "staggered"):
                assert torch.equal(seen[sched_name][rid], seen["whole"][rid])
        plain_folder = write_config(dict(DYNAMIC, rope_scaling=None), str(tmp_path), "plain", seed=6)
        unscaled = helpers.plain_logits(plain_folder, {rid: reqs[rid] for rid in ("r0", "r4")})
        for rid in ("r0", "r4"):
            helpers.assert_close(seen["whole"][rid], unscaled[rid], rel, f"within the trained context, {rid}")


@pytest.mark.parametrize("dtype,rel", [("float32", REL_F32), ("bfloat16", REL_BF16)])
@pytest.mark.parametrize("name", ["C", "E"])
def test_long_decoding(folders, name, dtype, rel):
    """A short prompt, then hundreds of tokens one by one (past several pages; ALiBi past position 256)."""
    n = 330
    reqs = helpers.make_requests(TINY[name]["vocab_size"], [n], seed=7)
    want = helpers.plain_logits(folders[name], reqs)
    rp = _replayer(folders[name], dtype, max_tokens=512)
    got = helpers.run_schedule(rp, helpers.schedule_tail(reqs, n - 3))
    helpers.assert_close(got["r0"], want["r0"], rel, f"{name} {dtype} long decoding")


@pytest.mark.parametrize("dtype,rel", [("float32", REL_F32), ("bfloat16", REL_BF16)])
def test_decoding_across_the_length_bound_of_a_captured_step(folders, dtype, rel):
    """Three sequences of unequal lengths decode together across position 1,024, where the captured decode
    step is replaced by one sized for longer contexts (more key ranges, another page-table width), and the
    shortest leaves the batch on the way."""
    lens = [1075, 1010, 700]
    reqs = helpers.make_requests(TINY["D"]["vocab_size"], lens, seed=11)
    want = helpers.plain_logits(folders["D"], reqs)
    rp = _replayer(folders["D"], dtype, max_tokens=3 * 1088)
    got = helpers.run_schedule(rp, helpers.schedule_batches(reqs, 3, decode=(90, 40, 12)))
    for rid in reqs:
        helpers.assert_close(got[rid], want[rid], rel, f"D {dtype} across 1024 {rid}")


@pytest.mark.parametrize("name", ["A", "C", "E", "B without bias"])
def test_prompts_of_many_rows_in_one_step(folders, tmp_path, name):
    """Prompts of 330, 270 and 60 tokens in one step of 660 rows, then a few tokens each: beyond 512 rows the matrix
    products are the vendor library's, a wave normalises a row, and where no bias stands in the way the norm adds the
    block's terms itself (bfloat16; both parallel arrangements, ALiBi, and the sequential one)."""
    from pytorch_transformers_amd import ops

    if name in TINY:
        folder, vocab = folders[name], TINY[name]["vocab_size"]
    else:
        folder, vocab = write_config(dict(TINY["B"], bias=False), str(tmp_path), "B-no-bias", 6), TINY["B"]["vocab_size"]
    reqs = helpers.make_requests(vocab, [333, 275, 64], seed=21)
    want = helpers.plain_logits(folder, reqs)
    rp = _replayer(folder, "bfloat16", max_tokens=3 * 384)
    sums = []
    real = ops.layernorm_sum
    ops.layernorm_sum = lambda terms, H, **kw: (sums.append(len(terms)), real(terms, H, **kw))[1]
    try:
        got = helpers.run_schedule(rp, helpers.schedule_batches(reqs, 3, decode=(3, 5, 4)))
    finally:
        ops.layernorm_sum = real
    for rid in reqs:
        helpers.assert_close(got[rid], want[rid], REL_BF16, f"{name} many rows {rid}")
    assert max(sums) == (2 if name.startswith("B") else 3), "the norm was handed the block's terms to add"


@pytest.mark.parametrize("dtype,rel", [("float32", REL_F32), ("bfloat16", REL_BF16)])
@pytest.mark.parametrize("name", ["A", "C"])
def test_a_batch_of_150_sequences_that_thins_out(folders, name, dtype, rel):
    """150 short requests decode together and leave a few at a time: the steps bring 150, 133, 117, ... 17 rows,
    through every row count at which the matrix products change kernels (two chunks of rows, one, the kernels
    for few rows)."""
    lens = [6 + (7 * i) % 23 for i in range(150)]
    reqs = helpers.make_requests(TINY[name]["vocab_size"], lens, seed=150)
    want = helpers.plain_logits(folders[name], reqs)
    rp = _replayer(folders[name], dtype, max_tokens=150 * 64)
    got = helpers.run_schedule(rp, helpers.schedule_batches(reqs, 150, decode=(1, 2, 3, 4, 5, 6, 7, 8, 9)))
    for rid in reqs:
        helpers.assert_close(got[rid], want[rid], rel, f"{name} {dtype} batch of 150, {rid}")


@pytest.mark.parametrize("dtype,rel", [("float32", REL_F32), ("bfloat16", REL_BF16)])
def test_first_tokens(folders, dtype, rel):
    """The first tokens of a sequence, fed one at a time from an empty slot."""
    reqs = helpers.make_requests(TINY["A"]["vocab_size"], [6], seed=11)
    want = helpers.plain_logits(folders["A"], reqs)
    rp = _replayer(folders["A"], dtype, max_tokens=64)
    got = helpers.run_schedule(rp, helpers.schedule_tail(reqs, 100))
    helpers.assert_close(got["r0"], want["r0"], rel, f"A {dtype} first tokens")


@pytest.mark.parametrize("dtype,rel", [("float32", REL_F32), ("bfloat16", REL_BF16)])
def test_alibi_without_the_references_rounding(tmp_path, dtype, rel):
    """``alibi_bf16_compat: false`` in config.json: the bias is the exact slope times position; the default keeps the
    reference's bfloat16 rounding of both and of their product, and the two differ visibly past position 256."""
    from pytorch_transformers_amd import AutoModelForCausalLM
    from pytorch_transformers_amd.engine.replay import Replayer
    from tiny import write_config

    raw = dict(TINY["E"], alibi_bf16_compat=False)
    folder = write_config(raw, str(tmp_path), "exact", seed=4)
    reqs = helpers.make_requests(raw["vocab_size"], [330, 40], seed=8)
    want = helpers.plain_logits(folder, reqs)
    rp = Replayer(AutoModelForCausalLM.from_pretrained(folder, dtype=dtype), 1024)
    for records in (helpers.schedule_whole(reqs), helpers.schedule_batches(reqs, 2, decode=(40, 5))):
        got = helpers.run_schedule(rp, records)
        for rid in reqs:
            helpers.assert_close(got[rid], want[rid], rel, f"exact alibi {dtype} {rid}")
    if dtype == "float32":
        rounded = helpers.plain_logits(write_config(TINY["E"], str(tmp_path), "rounded", seed=4), reqs)
        assert float((rounded["r0"] - want["r0"]).abs().max()) > 1e-3 * float(want["r0"].abs().max())


def test_dtype_auto_follows_the_configuration_then_the_file(tmp_path):
    """``dtype="auto"`` (src/transformers/modeling_utils.py:3996-4058): config.json's ``torch_dtype`` if it names
    one, else the type of the first floating-point tensor of the file."""
    from pytorch_transformers_amd import AutoModelForCausalLM
    from pytorch_transformers_amd.config import AutoConfig
    from pytorch_transformers_amd.weights import write_random_model

    for i, (named, stored, want) in enumerate(((None, torch.float32, torch.float32), (None, torch.bfloat16, torch.bfloat16),
                                               ("float32", torch.bfloat16, torch.float32),
                                               ("bfloat16", torch.float32, torch.bfloat16),
                                               ("float16", torch.float32, torch.bfloat16))):
        cfg = AutoConfig.from_dict(dict(TINY["A"], torch_dtype=named))
        folder = write_random_model(str(tmp_path / f"m{i}"), cfg, seed=1, store_dtype=stored)
        model = AutoModelForCausalLM.from_pretrained(folder, dtype="auto")
        assert model.dtype == want, f"torch_dtype={named}, file {stored}: got {model.dtype}"
        assert model.spec.embedding.weight.dtype == want
    with pytest.raises(ValueError):
        AutoModelForCausalLM.from_pretrained(folder, dtype="int8")


def test_cache_full_is_an_error(folders):
    from pytorch_transformers_amd.cache import CacheFull

    rp = _replayer(folders["A"], "float32", max_tokens=128)
    rp.run({"step": 0, "entries": [{"id": "a", "tokens": list(range(100)), "want": []}], "end": []})
    with pytest.raises(CacheFull):
        rp.run({"step": 1, "entries": [{"id": "b", "tokens": list(range(100)), "want": []}], "end": []})


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(folders, tmp_path, dtype):
    """bin/trace_run as a program: stdin records, files of logits, 'done' lines; with --dump-layers also the
    residual stream after every layer, which equals the plain implementation's."""
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    reqs = helpers.make_requests(TINY["A"]["vocab_size"], [19, 40], seed=5)
    records = helpers.schedule_batches(reqs, 2, decode=(4, 9))
    out = tmp_path / "out"
    p = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", folders["A"], "--dtype", dtype,
                        "--out", str(out), "--max-tokens", "128", "--dump-layers", "--check-finite"],
                       input="".join(json.dumps(r) + "\n" for r in records), capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    assert p.stdout.split("\n")[:-1] == [f"done {r['step']}" for r in records]
    want = helpers.plain_logits(folders["A"], reqs)
    V = TINY["A"]["vocab_size"]
    fed = {rid: 0 for rid in reqs}
    for r in records:
        arr = np.fromfile(out / f"{r['step']}.f32", dtype="<f4").reshape(-1, V)
        row = 0
        for e in r["entries"]:
            for pl in e["want"]:
                helpers.assert_close(torch.from_numpy(arr[row]), want[e["id"]][fed[e["id"]] + pl],
                                     REL_F32 if dtype == "float32" else REL_BF16, f"trace_run step {r['step']}")
                row += 1
            fed[e["id"]] += len(e["tokens"])
        assert row == arr.shape[0]
    # the dumps of the first step (both prompts, laid end to end) against the plain residual streams
    cfg, w = helpers.plain.read_model(folders["A"])
    H, rel = TINY["A"]["hidden_size"], (REL_F32 if dtype == "float32" else REL_BF16)
    first = records[0]
    hidden = {}
    for e in first["entries"]:
        hidden[e["id"]] = []
        helpers.plain.forward(cfg, w, e["tokens"], hidden=hidden[e["id"]])
    for layer in range(TINY["A"]["num_hidden_layers"]):
        got = torch.from_numpy(np.fromfile(out / f"{first['step']}.layer{layer}.f32", dtype="<f4").reshape(-1, H))
        want_rows = torch.cat([hidden[e["id"]][layer] for e in first["entries"]]).float()
        helpers.assert_close(got, want_rows, rel, f"trace_run layer {layer} dump")


def test_two_processes_write_the_same_bfloat16_bits(folders, tmp_path):
    """bfloat16 logits are a function of weights, tokens and schedule: two fresh processes of the replay program
    write identical files.  The trace has a prompt long enough for the vendor library's product (300 rows), short
    ones, a batch that decodes together and requests that join while others run."""
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    reqs = helpers.make_requests(TINY["C"]["vocab_size"], [300, 40, 7, 130], seed=9)
    records = helpers.schedule_batches(reqs, 4, decode=(20, 9, 3, 14)) + \
        [dict(r, step=r["step"] + 1000) for r in helpers.schedule_staggered(reqs, 2, decode=(4, 9, 2, 30), chunks=(None, 16, 1, 50))]
    text = "".join(json.dumps(r) + "\n" for r in records)
    outs = []
    for run in range(2):
        out = tmp_path / f"out{run}"
        env = dict(os.environ, PTA_TUNE="0")
        p = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", folders["C"], "--dtype",
                            "bfloat16", "--out", str(out), "--max-tokens", "1024"], input=text, capture_output=True,
                           text=True, timeout=300, env=env)
        assert p.returncode == 0, p.stderr[-2000:]
        outs.append(out)
    names = sorted(os.listdir(outs[0]))
    assert names == sorted(os.listdir(outs[1])) and len(names) == len(records)
    for name in names:
        a, b = (np.fromfile(o / name, dtype="<u4") for o in outs)
        assert np.array_equal(a, b), f"{name}: the two processes wrote different bits"


def test_steps_time_nothing_unless_asked_and_a_table_carries_the_choices(folders):
    """An untuned step makes no timed choice and keeps no half-gigabyte buffer; ``tune`` fills the table, the table
    as plain data restores the same choices after they were forgotten, and logits follow the choices in use."""
    from pytorch_transformers_amd import AutoModelForCausalLM, ops

    model = AutoModelForCausalLM.from_pretrained(folders["C"], dtype="bfloat16")
    ops.clear_tuning()
    cache = model.new_cache(2048, max_slots=4)
    slot = cache.alloc()
    prompt = list(range(600))
    before = model.step(cache, [slot], [prompt], "last").clone()
    cache.free(slot)
    assert ops._flush is None and not any(ops.tuning_table().values()), "a plain step timed something"
    table = model.tune(prompt_lens=(600,), batches=(4, 40))
    assert ops._flush is None, "the buffer for cold timings outlives tune()"
    assert table["pair_parts"], "tune() of a parallel block times its pair launches"
    import json as _json
    table = _json.loads(_json.dumps(table))  # plain data
    ops.clear_tuning()
    assert not any(ops.tuning_table().values())
    ops.load_tuning(table)
    assert ops.tuning_table() == table
    slot = cache.alloc()
    tuned = model.step(cache, [slot], [prompt], "last").clone()
    cache.free(slot)
    ops.clear_tuning()
    slot = cache.alloc()
    again = model.step(cache, [slot], [prompt], "last").clone()
    cache.free(slot)
    assert torch.equal(before, again), "without a table the same step gives the same bits"
    helpers.assert_close(tuned, before, 2e-2, "tuned against untuned logits")


def test_a_configuration_that_no_kernel_takes_is_refused_before_a_weight_is_read(tmp_path):
    """Heads of 512 elements (1,024 wide, two heads): the folder holds a configuration and no weights at all, and the
    error is about the head size, from the part that has it; the same from a configuration alone."""
    from pytorch_transformers_amd import AutoModelForCausalLM
    from pytorch_transformers_amd.config import AutoConfig

    raw = dict(TINY["C"], hidden_size=1024, num_attention_heads=2, ffn_hidden_size=64)
    (tmp_path / "config.json").write_text(json.dumps(raw))
    for dtype in ("bfloat16", "float32"):
        with pytest.raises(ValueError, match=r"transformer\.h\.0\.self_attention: attention: head size 512 is outside 1\.\.256"):
            AutoModelForCausalLM.from_pretrained(str(tmp_path), dtype=dtype)
    with pytest.raises(ValueError, match="head size 512"):
        AutoModelForCausalLM.from_config(AutoConfig.from_dict(raw))


def test_two_models_in_one_process_keep_their_own_timed_choices(folders):
    """A model's table is its own: timing the choices of one model, or loading a table into it, changes neither
    another model's table nor its bits, however their steps interleave; a table file given to ``from_pretrained``
    makes the choices of the model that wrote it."""
    import json as _json

    from pytorch_transformers_amd import AutoModelForCausalLM, tuning

    first = AutoModelForCausalLM.from_pretrained(folders["C"], dtype="bfloat16")
    second = AutoModelForCausalLM.from_pretrained(folders["C"], dtype="bfloat16")
    prompt = list(range(600))

    def logits(model):
        cache = model.new_cache(1024, max_slots=1)
        slot = cache.alloc()
        out = model.step(cache, [slot], [prompt], "last").clone()
        more = model.step(cache, [slot], [[5]], "last").clone()
        return torch.cat([out, more])

    plain_bits = logits(second)
    assert torch.equal(logits(first), plain_bits)
    table = first.tune(prompt_lens=(600,), batches=(4, 40))
    assert table["pair_parts"] and first.tuning.pair_parts and not any(second.tuning.to_dict().values())
    tuned_bits = logits(first)
    assert tuning.active() is first.tuning
    assert torch.equal(logits(second), plain_bits), "another model's timed choices changed this model's bits"
    assert tuning.active() is second.tuning
    assert torch.equal(logits(first), tuned_bits) and torch.equal(logits(second), plain_bits)
    path = os.path.join(os.path.dirname(folders["C"]), "tuning_table.json")
    with open(path, "w") as f:
        _json.dump(table, f)
    third = AutoModelForCausalLM.from_pretrained(folders["C"], dtype="bfloat16", tuning_table=path)
    assert third.tuning.to_dict() == table
    assert torch.equal(logits(third), tuned_bits) and torch.equal(logits(second), plain_bits)
    with pytest.raises(ValueError, match="sections"):
        second.tune(table={"pair_ranges": {}})


def test_tune_times_whole_steps_with_each_cut_of_the_decode_attention(folders):
    """``tune(contexts=...)`` replays captured decode steps at those contexts once per candidate cut of the attention
    and leaves every bucket either at the rule's cut or at a candidate.  Decoding with every candidate fixed by hand
    still matches the plain implementation, and forgetting the table restores the untuned bits."""
    from pytorch_transformers_amd import AutoModelForCausalLM, ops
    from pytorch_transformers_amd.engine.replay import Replayer

    name = "C"
    ops.clear_tuning()
    model = AutoModelForCausalLM.from_pretrained(folders[name], dtype="bfloat16")
    reqs = helpers.make_requests(TINY[name]["vocab_size"], [700], seed=11)
    records = helpers.schedule_tail(reqs, 40)
    want = helpers.plain_logits(folders[name], reqs)
    run = lambda: helpers.run_schedule(Replayer(model, 1024), records)["r0"]
    before = run()
    helpers.assert_close(before, want["r0"], REL_BF16, "untuned")
    try:
        table = model.tune(prompt_lens=(), batches=(1, 3), contexts=(690, (700, 300)))
        for k, cut in table["decode_plans"].items():
            assert tuple(cut) in ops.decode_plan_candidates(tuple(int(v) for v in k.split(",")))[1:]
        assert ops.take_decode_keys() == [] and ops._flush is None
        cfg = model.config
        key = ops.decode_key(1, cfg.num_attention_heads, cfg.kv_heads, cfg.head_dim, 700, 700)
        cuts = ops.decode_plan_candidates(key)
        assert any(c[2] > 1 for c in cuts)
        for cut in cuts:
            ops.set_decode_plan(key, cut)
            helpers.assert_close(run(), want["r0"], REL_BF16, f"cut {cut}")
    finally:
        ops.clear_tuning()
    assert torch.equal(run(), before)


def test_logits_of_a_step_outlive_the_next_step(folders):
    """What ``step`` returns is the caller's: the next step, replayed from the same captured graph, writes a
    buffer of its own."""
    from pytorch_transformers_amd import AutoModelForCausalLM

    got = {}
    for graphs in (False, True):
        model = AutoModelForCausalLM.from_pretrained(folders["A"], dtype="bfloat16")
        model.use_graphs = graphs
        cache = model.new_cache(512, max_slots=2)
        slots = [cache.alloc(), cache.alloc()]
        model.step(cache, slots, [[1, 2, 3], [4, 5]], "last")
        held = [model.step(cache, slots, [[6 + k], [9 + k]], "last") for k in range(4)]  # no clone by the caller
        torch.cuda.synchronize()
        got[graphs] = [h.clone() for h in held]
    for k, (a, b) in enumerate(zip(got[False], got[True])):
        assert torch.equal(a, b), f"the logits of step {k} were overwritten by a later replay"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_graph_replays_equal_eager_steps(folders, name, dtype):
    """Decode steps replayed from a captured graph give the bits of the same steps launched one by one,
    on every replay, with eager work (prompts of other batches, frees) and synchronisation in between."""
    from pytorch_transformers_amd import AutoModelForCausalLM
    from pytorch_transformers_amd.engine.replay import Replayer

    reqs = helpers.make_requests(TINY[name]["vocab_size"], [40, 9, 70, 33, 17, 64, 5, 21, 90, 12], seed=3)
    records = helpers.schedule_batches(reqs, 4, decode=(12, 5, 30, 9)) + \
        [dict(r, step=r["step"] + 1000) for r in helpers.schedule_batches(reqs, 10, decode=(7, 3))]
    outs = {}
    for graphs in (False, True):
        model = AutoModelForCausalLM.from_pretrained(folders[name], dtype=dtype)
        model.use_graphs = graphs
        rp = Replayer(model, 4096)
        outs[graphs] = []
        for rec in records:
            logits = rp.run(rec)
            outs[graphs].append(None if logits is None else logits.clone())
            torch.cuda.synchronize()
        if graphs:
            assert getattr(rp.cache, "_decode_graphs", None), "no graph was captured"
    for rec, a, b in zip(records, outs[False], outs[True]):
        assert (a is None) == (b is None)
        if a is not None:
            assert torch.equal(a, b), f"step {rec['step']}: graph replay differs from eager launch"


def test_a_dropped_cache_takes_its_graphs_along(folders):
    """A cache and the decode steps captured for it form no reference cycle: dropping the cache frees them at
    once, never later from the collector of cycles (which could then run while another step is captured, when
    the runtime permits no graph to be destroyed), and captures of later caches go on working."""
    import gc
    import weakref

    from pytorch_transformers_amd import AutoModelForCausalLM

    model = AutoModelForCausalLM.from_pretrained(folders["A"], dtype="bfloat16")
    assert model.use_graphs
    gc.collect()
    gc.disable()
    try:
        refs = []
        for n in (2, 3):  # the second round captures while the first round's cache is already gone
            cache = model.new_cache(1024, max_slots=4)
            slots = [cache.alloc() for _ in range(n)]
            model.step(cache, slots, [[1, 2, 3]] * n, "last")
            model.step(cache, slots, [[4]] * n, "last")
            graphs = list(cache._decode_graphs.values())
            assert graphs and graphs[0].graph is not None
            refs.append((weakref.ref(cache), weakref.ref(graphs[0])))
            del graphs
            for s in slots:
                cache.free(s)
            del cache
            assert refs[-1][0]() is None and refs[-1][1]() is None, "the cache or its graph outlives its last reference"
    finally:
        gc.enable()
