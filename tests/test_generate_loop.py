"""The generation loop's decisions, with a scripted model and sampler in place of the GPU (no GPU)."""
import pytest
import torch

from pytorch_transformers_amd.cache import PagedCache
from pytorch_transformers_amd.config import GenerationConfig
from pytorch_transformers_amd.engine.generate import GenerateOutput, generate, pad_sequences, resolve_lengths
from pytorch_transformers_amd.engine.spec import CACHE_FULL, CacheGroupSpec

V = 50


class ScriptedModel:
    """The next token of a sequence is (sum of its tokens so far) % V; records every step."""

    vocab_size = V
    device = torch.device("cpu")
    generation_config = None

    def __init__(self):
        self.steps = []
        self.seen = {}
        self.caches = []

    def new_cache(self, max_tokens, max_slots=None):
        c = PagedCache([CacheGroupSpec("kv", CACHE_FULL, 1, 1, 16)], max_tokens, torch.float32, "cpu", max_slots=max_slots)
        self.caches.append(c)
        return c

    def step(self, cache, slots, tokens, want):
        assert want == "last"
        cache.reserve(slots, [len(t) for t in tokens])
        rows = []
        for s, t in zip(slots, tokens):
            if cache.length(s) == 0:
                self.seen[s] = []
            else:
                assert len(t) == 1, "after its prompt a sequence brings one token a step"
            self.seen[s] = self.seen[s] + list(t)
            row = torch.zeros(V)
            row[sum(self.seen[s]) % V] = 5.0
            rows.append(row)
        cache.commit(slots, [len(t) for t in tokens])
        cache.check_consistent()
        self.steps.append((list(slots), [list(t) for t in tokens]))
        return torch.stack(rows)


class ArgmaxSampler:
    def __init__(self, eos=()):
        self.calls = []
        self.eos = list(eos)

    def sample(self, logits, *, rng_seq, rng_step, histories, suppress_eos, uniforms=None, new_counts=None,
               need_scores=True):
        self.calls.append(dict(rng_seq=list(rng_seq), rng_step=list(rng_step), suppress=list(suppress_eos),
                               histories=[list(h) for h in histories], new_counts=list(new_counts)))
        scores = logits.clone()
        for r, sup in enumerate(suppress_eos):
            if sup:
                scores[r, self.eos] = float("-inf")
        return scores.argmax(-1).tolist(), scores


def expected(prompt, n, eos=()):
    seq = list(prompt)
    for _ in range(n):
        seq.append(sum(seq) % V)
        if seq[-1] in eos:
            break
    return seq


def test_unequal_prompts_each_get_their_tokens():
    m = ScriptedModel()
    prompts = [[1, 2, 3], [4], [5, 6, 7, 8, 9, 10, 11]]
    out = generate(m, prompts, GenerationConfig(max_new_tokens=4), sampler=ArgmaxSampler())
    assert out == [expected(p, 4) for p in prompts]
    assert m.steps[0][1] == prompts  # prompts go through one step together, unpadded
    assert all(len(t) == 1 for _, toks in m.steps[1:] for t in toks)
    assert len(m.steps) == 4  # prompt step + 3 single-token steps (the 4th token needs no further step)
    assert not m.caches[0].live_slots() and m.caches[0].free_pages() == m.caches[0].num_pages


def test_eos_ends_a_sequence_early_keeps_the_token_and_frees_the_slot():
    m = ScriptedModel()
    prompts = [[1, 2, 3], [20, 5]]
    # sequence 0: 6, 12, 24, 48 ...; sequence 1: 25, 0, 0 ...  -> EOS 12 stops sequence 0 after two tokens
    out = generate(m, prompts, GenerationConfig(max_new_tokens=5, eos_token_id=12), sampler=ArgmaxSampler([12]))
    assert out[0] == [1, 2, 3, 6, 12] and out[1] == expected([20, 5], 5)
    assert [len(s) for s, _ in m.steps] == [2, 2, 1, 1, 1]  # the batch shrinks at once
    assert not m.caches[0].live_slots()
    # a list of stop tokens
    out = generate(ScriptedModel(), prompts, GenerationConfig(max_new_tokens=5, eos_token_id=[99, 25]),
                   sampler=ArgmaxSampler([99, 25]))
    assert out[1] == [20, 5, 25]


def test_min_new_tokens_and_min_length_suppress_eos():
    s = ArgmaxSampler([6])
    generate(ScriptedModel(), [[1, 2, 3]], GenerationConfig(max_new_tokens=4, eos_token_id=6, min_new_tokens=2), sampler=s)
    # 6 is masked twice (the argmax falls to token 0), then allowed, chosen, and ends the sequence
    assert [c["suppress"][0] for c in s.calls] == [True, True, False]
    s = ArgmaxSampler([6])
    # min_length counts the (longest) prompt: 3 + new < 5 for the first two choices
    generate(ScriptedModel(), [[1, 2, 3]], GenerationConfig(max_new_tokens=4, eos_token_id=6, min_length=5), sampler=s)
    assert [c["suppress"][0] for c in s.calls] == [True, True, False]


def test_max_length_counts_from_the_longest_prompt():
    assert resolve_lengths(GenerationConfig(max_length=10), [3, 7]) == (3, 7)
    assert resolve_lengths(GenerationConfig(max_length=10, max_new_tokens=2), [3, 7]) == (2, 7)
    with pytest.raises(ValueError, match="max_length"):
        resolve_lengths(GenerationConfig(max_length=7), [3, 7])
    out = generate(ScriptedModel(), [[1, 2, 3], [4] * 7], GenerationConfig(max_length=10), sampler=ArgmaxSampler())
    assert [len(o) for o in out] == [6, 10]


def test_batches_run_one_after_another_on_one_cache():
    m = ScriptedModel()
    prompts = [[i + 1, i + 2] for i in range(7)]
    out = generate(m, prompts, GenerationConfig(max_new_tokens=3), batch_size=3, sampler=ArgmaxSampler())
    assert out == [expected(p, 3) for p in prompts]
    assert len(m.caches) == 1 and m.caches[0].max_slots == 3
    starts = [toks for _, toks in m.steps if len(toks[0]) == 2]
    assert [len(t) for t in starts] == [3, 3, 1]  # three batches
    used = {s for slots, _ in m.steps for s in slots}
    assert used == {0, 1, 2}  # slots are used again


def test_rng_streams_follow_the_prompt_not_the_batch():
    s = ArgmaxSampler()
    generate(ScriptedModel(), [[1], [2], [3]], GenerationConfig(max_new_tokens=2, do_sample=True), batch_size=2, sampler=s)
    assert [c["rng_seq"] for c in s.calls] == [[0, 1], [0, 1], [2], [2]]
    assert [c["rng_step"] for c in s.calls] == [[0, 0], [1, 1], [0], [1]]
    s = ArgmaxSampler()
    generate(ScriptedModel(), [[3]], GenerationConfig(max_new_tokens=1, do_sample=True), rng_ids=[2], sampler=s)
    assert s.calls[0]["rng_seq"] == [2]
    s = ArgmaxSampler()
    out = generate(ScriptedModel(), [[1], [2]], GenerationConfig(max_new_tokens=1, do_sample=True, num_return_sequences=2), sampler=s)
    assert len(out) == 4 and s.calls[0]["rng_seq"] == [0, 1, 2, 3] and out[0][:1] == out[1][:1] == [1]


def test_histories_streamer_and_outputs():
    s = ArgmaxSampler()
    seen = []

    class Streamer:
        ended = False

        def __call__(self, i, tok):
            seen.append((i, tok))

        def end(self):
            self.ended = True

    st = Streamer()
    out = generate(ScriptedModel(), [[1, 2], [7]], GenerationConfig(max_new_tokens=2, return_dict_in_generate=True,
                                                                    output_scores=True, output_logits=True),
                   sampler=s, streamer=st)
    assert isinstance(out, GenerateOutput) and out.sequences == [[1, 2, 3, 6], [7, 7, 14]]
    assert s.calls[1]["histories"] == [[1, 2, 3], [7, 7]]  # prompt and new tokens, for the repetition penalty
    assert seen == [(0, 3), (1, 7), (0, 6), (1, 14)] and st.ended
    assert len(out.scores[0]) == 2 and out.logits[1][0].shape == (V,)


def test_empty_prompt_starts_from_bos_and_slots_return_on_error():
    out = generate(ScriptedModel(), [[]], GenerationConfig(max_new_tokens=1, bos_token_id=9), sampler=ArgmaxSampler())
    assert out == [[9, 9]]
    with pytest.raises(ValueError, match="empty"):
        generate(ScriptedModel(), [[]], GenerationConfig(max_new_tokens=1), sampler=ArgmaxSampler())

    class Boom(ScriptedModel):
        def step(self, *a, **k):
            if len(self.steps) == 1:
                raise RuntimeError("boom")
            return super().step(*a, **k)

    m = Boom()
    with pytest.raises(RuntimeError, match="boom"):
        generate(m, [[1], [2]], GenerationConfig(max_new_tokens=3), sampler=ArgmaxSampler())
    assert not m.caches[0].live_slots() and m.caches[0].free_pages() == m.caches[0].num_pages


def test_stop_strings_need_a_tokenizer_and_end_a_sequence_with_the_completing_token():
    """src/transformers/generation/utils.py:1118-1125: no tokenizer is an error; with one, a sequence ends with
    the token that completes a stop string in the text of its new tokens (the token stays), the others go on."""
    class Letters:
        def decode(self, ids):
            return "".join(chr(ord("a") + t % 26) for t in ids)

    prompts = [[1, 2, 3], [4]]
    free = [expected(p, 8) for p in prompts]
    with pytest.raises(ValueError, match="tokenizer"):
        generate(ScriptedModel(), prompts, GenerationConfig(max_new_tokens=8, stop_strings="ab"), sampler=ArgmaxSampler())
    text = Letters().decode(free[0][3:])
    stop = text[2:4]  # completed by the fourth new token of the first prompt
    assert stop not in Letters().decode(free[1][1:]) and stop not in text[:3]
    out = generate(ScriptedModel(), prompts, GenerationConfig(max_new_tokens=8, stop_strings=[stop, "zzzz"]),
                   sampler=ArgmaxSampler(), tokenizer=Letters())
    assert out[0] == free[0][:3 + 4] and out[1] == free[1]
    # a stop string that the prompt holds does not count: only new tokens are read
    out = generate(ScriptedModel(), [[0, 1]], GenerationConfig(max_new_tokens=3, stop_strings="ab"), sampler=ArgmaxSampler(),
                   tokenizer=Letters())
    assert len(out[0]) == 2 + 3 or "ab" in Letters().decode(out[0][2:])


def test_pad_sequences_matches_the_reference_layout():
    t = pad_sequences([[1, 2, 3, 9, 9], [4, 8]], [3, 1], pad_token_id=0)
    assert t.tolist() == [[1, 2, 3, 9, 9], [0, 0, 4, 8, 0]]


def test_kept_slots_go_on_in_a_later_call():
    """Four new tokens at once equal three and then one from the kept slots (the reference's test of continuing
    from a returned cache, tests/generation/test_utils.py:1775-1855); the later call runs only the tokens that
    the slots do not hold, and whoever does not keep the slots gives them back."""
    m = ScriptedModel()
    prompts = [[1, 2, 3], [4], [5, 6, 7, 8]]
    at_once = generate(m, prompts, GenerationConfig(max_new_tokens=4), sampler=ArgmaxSampler())
    m2 = ScriptedModel()
    first = generate(m2, prompts, GenerationConfig(max_new_tokens=3), sampler=ArgmaxSampler(), keep_slots=True,
                     cache=m2.new_cache(64 * 8, max_slots=4))
    assert isinstance(first, GenerateOutput) and sorted(first.slots) == [0, 1, 2]
    cache = first.cache
    assert sorted(cache.live_slots()) == [0, 1, 2]
    assert [cache.length(s) for s in first.slots] == [len(seq) - 1 for seq in first.sequences]  # the last token is not run yet
    steps_before = len(m2.steps)
    more = generate(m2, first.sequences, GenerationConfig(max_new_tokens=1), sampler=ArgmaxSampler(), cache=cache,
                    slots=first.slots)
    assert more == at_once
    assert m2.steps[steps_before:] == [(first.slots, [[seq[-1]] for seq in first.sequences])]  # one token each, no prompt again
    assert cache.live_slots() == [] and cache.free_pages() == cache.num_pages
    # one sequence ends early by its stop token and still keeps its slot; batches one after another keep all
    m3 = ScriptedModel()
    eos = expected(prompts[1], 2)[-1]
    out = generate(m3, prompts, GenerationConfig(max_new_tokens=3, eos_token_id=eos), sampler=ArgmaxSampler(), keep_slots=True,
                   batch_size=2)
    assert len(out.sequences[1]) == len(prompts[1]) + 2 and all(s is not None for s in out.slots)
    assert sorted(out.cache.live_slots()) == sorted(out.slots)
    for s in out.slots:
        out.cache.free(s)
    # misuse is refused before anything runs
    with pytest.raises(ValueError, match="cache"):
        generate(m3, prompts, GenerationConfig(max_new_tokens=1), sampler=ArgmaxSampler(), slots=[0, 1, 2])
    c = m3.new_cache(256, max_slots=2)
    a = c.alloc()
    c.reserve([a], [3]); c.commit([a], [3])
    with pytest.raises(ValueError, match="already holds"):
        generate(m3, [[1, 2, 3]], GenerationConfig(max_new_tokens=1), sampler=ArgmaxSampler(), cache=c, slots=[a])
    with pytest.raises(ValueError, match="one slot"):
        generate(m3, [[1, 2, 3, 4], [1, 2, 3, 4]], GenerationConfig(max_new_tokens=1), sampler=ArgmaxSampler(), cache=c, slots=[a, a])


# ---- steps ahead of the host -------------------------------------------------------------------------------
class FakeAhead:
    """Stands in for tokens that are still on the device: the model may use the values, the host's reading is logged."""

    def __init__(self, values, log):
        self.values, self.log, self.rows = list(values), log, None
        self.name = len([e for e in log if e[0] == "chosen"])
        log.append(("chosen", self.name))

    def __len__(self):
        return len(self.values)

    def take(self, rows):
        self.rows = None if rows is None or list(rows) == list(range(len(self.values))) else list(rows)
        return self

    def tolist(self):
        self.log.append(("read", self.name))
        return list(self.values)


class AheadModel(ScriptedModel):
    steps_ahead = True

    def __init__(self, log):
        super().__init__()
        self.log = log

    def step(self, cache, slots, tokens, want, own_logits=True):
        if isinstance(tokens, FakeAhead):
            self.log.append(("step from", tokens.name))
            picked = tokens.rows if tokens.rows is not None else range(len(tokens.values))
            tokens = [[tokens.values[r]] for r in picked]
        else:
            self.log.append(("step", None))
        return super().step(cache, slots, tokens, want)


class AheadSampler(ArgmaxSampler):
    needs_histories = False

    def __init__(self, log, eos=()):
        super().__init__(eos)
        self.log = log

    def sample(self, logits, *, rng_seq, rng_step, suppress_eos, need_scores=True, ahead=False, **_):
        tokens, scores = super().sample(logits, rng_seq=rng_seq, rng_step=rng_step, histories=[[]] * len(rng_seq),
                                        suppress_eos=suppress_eos, new_counts=[0] * len(rng_seq))
        return (FakeAhead(tokens, self.log) if ahead else tokens), scores


def test_steps_ahead_choose_the_same_tokens_and_wait_for_none_before_the_next_step_is_launched():
    prompts = [[1, 2, 3], [20, 5], [7, 7, 7, 7], [9]]
    for cfg, eos in ((GenerationConfig(max_new_tokens=5, eos_token_id=12), [12]),
                     (GenerationConfig(max_new_tokens=6, eos_token_id=[25, 12], min_new_tokens=2), [25, 12]),
                     (GenerationConfig(max_new_tokens=1), [])):
        want = generate(ScriptedModel(), prompts, cfg, batch_size=3, sampler=ArgmaxSampler(eos))
        log = []
        m, s = AheadModel(log), AheadSampler(log, eos)
        assert generate(m, prompts, cfg, batch_size=3, sampler=s) == want
        assert not m.caches[0].live_slots() and m.caches[0].free_pages() == m.caches[0].num_pages
        # the choices were asked for as in the loop that waits: same streams, steps and masks of EOS per sequence
        waits = ArgmaxSampler(eos)
        generate(ScriptedModel(), prompts, cfg, batch_size=3, sampler=waits)
        per_seq = lambda calls: sorted((q, st, sup) for c in calls for q, st, sup in zip(c["rng_seq"], c["rng_step"], c["suppress"]))
        assert set(per_seq(waits.calls)) <= set(per_seq(s.calls))  # (plus the rows that nobody read)
        # every step after a batch's first was launched from tokens that the host had not read yet
        for at, (what, name) in enumerate(log):
            if what == "step from":
                assert ("read", name) not in log[:at]
        if cfg.max_new_tokens > 1:
            assert any(what == "step from" for what, _ in log)


def test_a_sequence_that_ends_on_a_stop_token_takes_part_in_one_step_too_many_and_one_that_ends_by_length_in_none():
    log = []
    m = AheadModel(log)
    prompts = [[1, 2, 3], [20, 5]]
    out = generate(m, prompts, GenerationConfig(max_new_tokens=5, eos_token_id=12), sampler=AheadSampler(log, [12]))
    assert out[0] == [1, 2, 3, 6, 12] and out[1] == expected([20, 5], 5)
    assert [len(s) for s, _ in m.steps] == [2, 2, 2, 1, 1]  # (the loop that waits: 2, 2, 1, 1, 1)
    assert not m.caches[0].live_slots() and m.caches[0].free_pages() == m.caches[0].num_pages


def test_a_step_ahead_that_finds_no_room_waits_for_the_tokens_and_goes_on_with_who_is_left():
    a, b = [1] * 60, [2] * 62
    eos = expected(a, 3)[-1]  # the third new token of the first sequence ends it
    assert eos not in expected(b, 6)[len(b):]
    cfg = GenerationConfig(max_new_tokens=6, eos_token_id=eos)
    want = [expected(a, 3), expected(b, 6)]
    for model, sampler in ((ScriptedModel(), ArgmaxSampler([eos])), (AheadModel([]), AheadSampler([], [eos]))):
        # two pages of 64: the second sequence's 65th token finds a page only once the first sequence has given its own back
        cache = model.new_cache(128, max_slots=2)
        assert cache.page_size == 64 and cache.num_pages == 2
        assert generate(model, [a, b], cfg, sampler=sampler, cache=cache) == want
        assert not cache.live_slots() and cache.free_pages() == 2
    log = []
    model = AheadModel(log)
    generate(model, [a, b], cfg, sampler=AheadSampler(log, [eos]), cache=model.new_cache(128, max_slots=2))
    assert ("step", None) in log[1:]  # the step that waited


def test_what_needs_the_tokens_on_the_host_keeps_the_loop_that_waits():
    class Reads(AheadSampler):
        needs_histories = True

    for kw, sampler_cls in ((dict(output_scores=True, return_dict_in_generate=True), AheadSampler), (dict(max_time=100.0), AheadSampler),
                            (dict(), Reads)):
        log = []
        generate(AheadModel(log), [[1, 2], [3]], GenerationConfig(max_new_tokens=3, **kw), sampler=sampler_cls(log))
        assert not any(what == "step from" for what, _ in log)
    log = []
    generate(AheadModel(log), [[1, 2], [3]], GenerationConfig(max_new_tokens=3), sampler=AheadSampler(log), streamer=lambda i, t: None)
    assert not any(what == "step from" for what, _ in log)


# ---- the caller's own stopping criteria and streamers ------------------------------------------------------------

def test_a_callers_stopping_criterion_ends_its_rows_only():
    """A criterion is handed the rows' ids, the new token included, padded on the left, and the step's scores; the
    rows it flags end with that token and give their slots back, the others go on."""
    m = ScriptedModel()
    prompts = [[1, 2, 3], [4], [5, 6]]
    seen = []

    def has_an_even_sum(input_ids, scores):
        seen.append((input_ids.clone(), None if scores is None else tuple(scores.shape)))
        return (input_ids.sum(-1) % 4 == 0)

    out = generate(m, prompts, GenerationConfig(max_new_tokens=6, pad_token_id=0), sampler=ArgmaxSampler(),
                   stopping_criteria=[has_an_even_sum])
    for p, o in zip(prompts, out):
        want = list(p)
        for _ in range(6):
            want.append(sum(want) % V)
            if sum(want) % 4 == 0:
                break
        assert o == want
    assert len({len(o) - len(p) for p, o in zip(prompts, out)}) > 1, "the case must end its rows at different steps"
    first_ids, first_shape = seen[0]
    assert first_ids.dtype == torch.long and first_ids.shape == (3, 4) and first_shape == (3, V)
    assert first_ids[1].tolist() == [0, 0, 4, 4] and first_ids[0].tolist() == [1, 2, 3, 6]  # left-padded with pad_token_id
    assert all(not c.live_slots() and c.free_pages() == c.num_pages for c in m.caches)
    # one flag for all rows ends all of them
    out = generate(ScriptedModel(), prompts, GenerationConfig(max_new_tokens=6), sampler=ArgmaxSampler(),
                   stopping_criteria=[lambda ids, scores: ids.shape[1] >= 4])
    assert [len(o) for o in out] == [4, 2, 3]
    with pytest.raises(ValueError, match="gave 2 flags for 3 rows"):
        generate(ScriptedModel(), prompts, GenerationConfig(max_new_tokens=2), sampler=ArgmaxSampler(),
                 stopping_criteria=[lambda ids, scores: torch.tensor([True, False])])


def test_the_callers_processors_reach_the_sampler_with_the_pad_id():
    class Recording(ArgmaxSampler):
        def sample(self, logits, *, extra_processors=None, pad_token_id=None, **kw):
            self.extra = (extra_processors, pad_token_id)
            return super().sample(logits, **kw)

    s = Recording()
    fn = lambda ids, scores: scores
    generate(ScriptedModel(), [[1, 2]], GenerationConfig(max_new_tokens=1, pad_token_id=7), sampler=s, logits_processor=[fn])
    assert s.extra == ([fn], 7)
    s = ArgmaxSampler()  # without processors a sampler that knows nothing of them is called as before
    generate(ScriptedModel(), [[1, 2]], GenerationConfig(max_new_tokens=1), sampler=s)


class WordTokenizer:
    """id -> a word; decoding joins with spaces, except that id 0 is a line break and ids from 40 on are CJK."""

    def decode(self, ids, **kw):
        self.kw = kw
        out = ""
        for t in ids:
            if t == 0:
                out += "\n"
            elif t >= 40:
                out += chr(0x4E00 + t)
            else:
                out += ("" if out == "" or out.endswith("\n") else " ") + f"w{t}"
        return out


def test_text_streamer_shows_whole_words_and_flushes_at_line_breaks(capsys):
    from pytorch_transformers_amd import TextStreamer

    st = TextStreamer(WordTokenizer(), skip_special_tokens=True)
    st.put(torch.tensor([[1, 2]]))  # the prompt: "w1 w2" -> up to the last space
    assert capsys.readouterr().out == "w1 "
    st.put(torch.tensor([3]))
    assert capsys.readouterr().out == "w2 "
    st.put(torch.tensor([0]))  # a line break flushes, and decoding starts anew behind it
    assert capsys.readouterr().out == "w3\n"
    st.put(torch.tensor([4]))
    assert capsys.readouterr().out == ""
    st.put(torch.tensor([41]))  # a character of a script without spaces is shown at once, with what was held back
    assert capsys.readouterr().out == "w4" + chr(0x4E00 + 41)
    st.put(torch.tensor([5]))
    st.end()
    assert capsys.readouterr().out == " w5\n"
    assert st.tokenizer.kw == {"skip_special_tokens": True}
    with pytest.raises(ValueError, match="batch size 1"):
        st.put(torch.tensor([[1], [2]]))
    quiet = TextStreamer(WordTokenizer(), skip_prompt=True)
    quiet.put(torch.tensor([1, 2]))
    quiet.put(torch.tensor([3]))
    quiet.put(torch.tensor([4]))
    quiet.end()
    assert capsys.readouterr().out == "w3 w4\n"
    quiet.put(torch.tensor([9]))  # the next call's prompt is skipped again
    quiet.put(torch.tensor([5]))
    quiet.end()
    assert capsys.readouterr().out == "w5\n"


def test_generate_feeds_a_streamer_the_prompt_then_every_token_and_iterates_in_a_thread():
    import threading

    from pytorch_transformers_amd import TextIteratorStreamer

    class Tape:
        def __init__(self):
            self.got, self.ended = [], 0

        def put(self, value):
            assert value.dtype == torch.long and value.dim() == 1
            self.got.append(value.tolist())

        def end(self):
            self.ended += 1

    tape = Tape()
    out = generate(ScriptedModel(), [[1, 2, 3]], GenerationConfig(max_new_tokens=3), sampler=ArgmaxSampler(), streamer=tape)
    assert tape.got == [[1, 2, 3]] + [[t] for t in out[0][3:]] and tape.ended == 1
    with pytest.raises(ValueError, match="batch size 1"):
        generate(ScriptedModel(), [[1], [2]], GenerationConfig(max_new_tokens=1), sampler=ArgmaxSampler(), streamer=Tape())
    it = TextIteratorStreamer(WordTokenizer(), skip_prompt=True, timeout=30)
    th = threading.Thread(target=generate, args=(ScriptedModel(), [[1, 2, 3]], GenerationConfig(max_new_tokens=4)),
                          kwargs=dict(sampler=ArgmaxSampler(), streamer=it))
    th.start()
    text = "".join(piece for piece in it)
    th.join()
    assert text == WordTokenizer().decode(expected([1, 2, 3], 4)[3:])


def test_processor_and_criteria_lists_are_callable():
    from pytorch_transformers_amd import LogitsProcessorList, StoppingCriteriaList

    ids, scores = torch.tensor([[1, 2], [3, 4]]), torch.zeros(2, 5)
    procs = LogitsProcessorList([lambda i, s: s + 1.0, lambda i, s: s * i.sum(-1, keepdim=True)])
    assert procs(ids, scores).tolist() == [[3.0] * 5, [7.0] * 5]
    crit = StoppingCriteriaList([lambda i, s: i[:, -1] == 2, lambda i, s: False])
    assert crit(ids, scores).tolist() == [True, False]


def test_rectangular_input_ids_with_a_mask_come_back_as_the_references_tensor():
    """``input_ids`` padded on the left with an ``attention_mask``: each row generates from its own ids, and the result
    is one tensor, prompts padded on the left, rows that ended early padded on the right with the pad token (the EOS
    token if no pad token is set)."""
    pad = 49
    prompts = [[1, 2, 3], [4], [5, 6]]
    ids = torch.tensor([[1, 2, 3], [pad, pad, 4], [pad, 5, 6]])
    mask = torch.tensor([[1, 1, 1], [0, 0, 1], [0, 1, 1]])
    want = [expected(p, 5, eos=(12,)) for p in prompts]
    assert len({len(w) for w in want}) > 1, "the case must end a row early"
    m = ScriptedModel()
    out = generate(m, ids, GenerationConfig(max_new_tokens=5, eos_token_id=12, pad_token_id=pad), sampler=ArgmaxSampler(),
                   attention_mask=mask)
    assert isinstance(out, torch.Tensor) and out.dtype == torch.long
    assert m.steps[0][1] == prompts  # no padding reaches the model
    width = 3 + max(len(w) - len(p) for w, p in zip(want, prompts))
    assert out.shape == (3, width)
    for row, p, w in zip(out.tolist(), prompts, want):
        assert row == [pad] * (3 - len(p)) + w + [pad] * (width - 3 - (len(w) - len(p)))
    # no pad token set: the EOS token pads; return_dict keeps the tensor under `sequences`
    res = generate(ScriptedModel(), ids, GenerationConfig(max_new_tokens=5, eos_token_id=12, return_dict_in_generate=True),
                   sampler=ArgmaxSampler(), attention_mask=mask)
    assert isinstance(res, GenerateOutput) and res.sequences.shape == (3, width)
    assert res.sequences[1].tolist()[:3] == [12, 12, 4]
    # without a mask every id of a row counts
    out = generate(ScriptedModel(), torch.tensor([[1, 2, 3], [7, 8, 9]]), GenerationConfig(max_new_tokens=2), sampler=ArgmaxSampler())
    assert out.tolist() == [expected([1, 2, 3], 2), expected([7, 8, 9], 2)]
    with pytest.raises(ValueError, match="shape of input_ids"):
        generate(ScriptedModel(), ids, GenerationConfig(max_new_tokens=1), sampler=ArgmaxSampler(), attention_mask=mask[:, :2])
    with pytest.raises(ValueError, match="lists have no padding"):
        generate(ScriptedModel(), prompts, GenerationConfig(max_new_tokens=1), sampler=ArgmaxSampler(), attention_mask=mask)


def test_transition_scores_are_the_chosen_tokens_scores():
    from pytorch_transformers_amd.engine.generate import compute_transition_scores

    prompts = [[1, 2, 3], [4]]
    out = generate(ScriptedModel(), prompts, GenerationConfig(max_new_tokens=3, output_scores=True, return_dict_in_generate=True),
                   sampler=ArgmaxSampler())
    raw = compute_transition_scores(out, [len(p) for p in prompts])
    assert [r.tolist() for r in raw] == [[5.0] * 3, [5.0] * 3]  # the scripted model scores its next token 5, the rest 0
    norm = compute_transition_scores(out, [len(p) for p in prompts], normalize_logits=True)
    want = float(torch.log_softmax(torch.tensor([5.0] + [0.0] * (V - 1)), -1)[0])
    assert all(abs(v - want) < 1e-6 for r in norm for v in r.tolist())
    with pytest.raises(ValueError, match="output_scores"):
        compute_transition_scores(GenerateOutput([[1, 2]]), [1])
