"""The sampling kernel against the plain processors, and generation through the entry point (GPU)."""
import math
import os

import pytest
import torch

import plain_falcon as P
from tiny import LIVELY_STD, TINY, write_model

pytestmark = pytest.mark.gpu


def _ops():
    from pytorch_transformers_amd import ops
    return ops


def _dev(x, dtype=torch.float32):
    return torch.as_tensor(x, dtype=dtype).cuda()


def _finite_mask(t):
    return (t != float("-inf")).cpu()


def test_argmax_lowest_index_on_ties():
    ops = _ops()
    x = torch.zeros(3, 1000)
    x[0, 517] = 2.0; x[0, 900] = 2.0
    x[1, 0] = -1.0
    x[2, 999] = 0.5
    tok, scores = ops.sample(_dev(x), do_sample=False)
    assert tok.tolist() == [517, 1, 999]
    assert torch.equal(scores.cpu(), x)


@pytest.mark.parametrize("V", [10, 211, 65024])
def test_processors_match_plain(V):
    """Penalty, EOS suppression, temperature, top-k, top-p, min-p: same tokens survive as in the plain code."""
    ops = _ops()
    g = torch.Generator().manual_seed(V)
    R = 5
    logits = torch.randn(R, V, generator=g) * 3
    hist = [[int(t) for t in torch.randint(0, V, (n,), generator=g)] for n in (3, 0, 7, 1, 12)]
    off = [0]
    for h in hist:
        off.append(off[-1] + len(h))
    flat = [t for h in hist for t in h]
    eos = [1, V - 1]
    suppress = [1, 0, 1, 0, 0]
    for kw in (dict(temperature=0.7, top_k=min(50, V - 1)), dict(top_p=0.9), dict(min_p=0.02),
               dict(temperature=1.3, top_k=min(40, V - 1), top_p=0.8, min_p=0.01, penalty=1.7),
               dict(top_k=1), dict(top_p=0.05), dict(top_k=V + 5, penalty=0.5)):
        tok, scores = ops.sample(
            _dev(logits), do_sample=True, temperature=kw.get("temperature", 1.0), top_k=kw.get("top_k", 0),
            top_p=kw.get("top_p", 1.0), min_p=kw.get("min_p", 0.0), penalty=kw.get("penalty", 1.0),
            hist=_dev(flat, torch.int32) if flat else None, hist_off=_dev(off, torch.int32), eos=_dev(eos, torch.int32),
            suppress=_dev(suppress, torch.int32), uniforms=_dev([0.5] * R))
        for r in range(R):
            want = P.process(logits[r], hist[r], do_sample=True, temperature_=kw.get("temperature", 1.0),
                             top_k_=kw.get("top_k", 0), top_p_=kw.get("top_p", 1.0), min_p_=kw.get("min_p"),
                             repetition_penalty_=kw.get("penalty", 1.0), suppress_ids=eos if suppress[r] else ())
            got = scores[r].cpu()
            keep_want, keep_got = want != float("-inf"), _finite_mask(got)
            # a token whose cumulative mass sits within rounding of the top-p cut may fall on either side
            diff = (keep_want != keep_got).nonzero().flatten().tolist()
            if diff and "top_p" in kw:
                probs = torch.softmax(torch.where(keep_want | keep_got, want if kw.get("min_p") is None else got, want).double(), -1)
                assert len(diff) <= 1, f"V={V} {kw} row {r}: kept sets differ at {diff}"
            else:
                assert not diff, f"V={V} {kw} row {r}: kept sets differ at {diff}"
            both = keep_want & keep_got
            torch.testing.assert_close(got[both], want[both], rtol=1e-6, atol=1e-6)
            assert keep_got[int(tok[r])], "the chosen token was filtered out"


def test_reference_vectors_on_the_kernel():
    """The reference's own small cases (tests/generation/test_logits_process.py:235-355) through the kernel."""
    ops = _ops()
    ramp = torch.arange(10.0)[None]
    _, s = ops.sample(_dev(ramp), do_sample=True, top_k=3, uniforms=_dev([0.1]))
    assert torch.isinf(s[0]).tolist() == 7 * [True] + 3 * [False]
    dist = torch.log(torch.tensor([[0.15, 0.3, 0.3, 0.25], [0.3, 0.1, 0.1, 0.5], [0.3, 0.1, 0.1, 0.5]]))
    for top_p, row, want in ((0.8, 0, [0.0, 0.3, 0.3, 0.25]), (0.79, 1, [0.3, 0.0, 0.0, 0.5]), (0.85, 2, [0.3, 0.0, 0.1, 0.5])):
        _, s = ops.sample(_dev(dist[row:row + 1]), do_sample=True, top_p=top_p, uniforms=_dev([0.1]))
        torch.testing.assert_close(torch.exp(s[0]).cpu(), torch.tensor(want), atol=1e-3, rtol=0)
    dist = torch.log(torch.tensor([[0.9, 0.0274, 0.047, 0.0274], [0.15, 0.3, 0.3, 0.25], [0.97, 0.01, 0.01, 0.01]]))
    _, s = ops.sample(_dev(dist), do_sample=True, min_p=0.05, uniforms=_dev([0.1] * 3))
    want = torch.tensor([[0.9, 0.0, 0.047, 0.0], [0.15, 0.3, 0.3, 0.25], [0.97, 0.0, 0.0, 0.0]])
    torch.testing.assert_close(torch.exp(s).cpu(), want, atol=1e-3, rtol=0)
    # typical-p, epsilon and eta cut-offs (:357-378, :405-428, :445-468)
    dist = torch.log(torch.tensor([[0.97, 0.01, 0.01, 0.01], [0.4, 0.2, 0.2, 0.2]]))
    _, s = ops.sample(_dev(dist), do_sample=True, typical_p=0.5, uniforms=_dev([0.1] * 2))
    torch.testing.assert_close(torch.exp(s).cpu(), torch.tensor([[0.97, 0.0, 0.0, 0.0], [0.0, 0.2, 0.2, 0.2]]), atol=1e-3, rtol=0)
    dist = torch.log(torch.tensor([[0.87, 0.099, 0.001, 0.03], [0.4, 0.299, 0.101, 0.2]]))
    _, s = ops.sample(_dev(dist), do_sample=True, epsilon_cutoff=0.1, uniforms=_dev([0.1] * 2))
    torch.testing.assert_close(torch.exp(s).cpu(), torch.tensor([[0.87, 0.0, 0.0, 0.0], [0.4, 0.299, 0.101, 0.2]]), atol=1e-3, rtol=0)
    dist = torch.log(torch.tensor([[0.0, 0.1, 0.8, 0.1], [0.01, 0.04, 0.9, 0.05]]))
    _, s = ops.sample(_dev(dist), do_sample=True, eta_cutoff=0.0625, uniforms=_dev([0.1] * 2))
    torch.testing.assert_close(torch.exp(s).cpu(), torch.tensor([[0.0, 0.1, 0.8, 0.1], [0.0, 0.0, 0.9, 0.0]]), atol=1e-3, rtol=0)
    # top_p so small that everything could go: the best token stays
    _, s = ops.sample(_dev(torch.arange(6.0)[None]), do_sample=True, top_p=0.0, uniforms=_dev([0.9]))
    assert _finite_mask(s[0]).tolist() == [False] * 5 + [True]
    # remove_invalid_values and renormalize_logits
    bad = torch.tensor([[float("nan"), float("inf"), -float("inf"), 1.0]])
    _, s = ops.sample(_dev(bad), do_sample=False, remove_invalid=True)
    assert s[0].tolist() == [0.0, torch.finfo(torch.float32).max, torch.finfo(torch.float32).min, 1.0]
    x = torch.randn(2, 300)
    _, s = ops.sample(_dev(x), do_sample=False, renorm=True)
    torch.testing.assert_close(s.cpu(), torch.log_softmax(x, -1), rtol=1e-5, atol=1e-5)


def test_draw_inverts_the_cumulative_distribution():
    """A given uniform number picks the token whose CDF interval holds it; frequencies follow softmax."""
    ops = _ops()
    logits = torch.tensor([[0.0, math.log(2.0), math.log(3.0), math.log(4.0)]])  # p = .1 .2 .3 .4
    for u, want in ((0.0, 0), (0.09, 0), (0.11, 1), (0.29, 1), (0.31, 2), (0.59, 2), (0.61, 3), (0.999, 3)):
        tok, _ = ops.sample(_dev(logits), do_sample=True, uniforms=_dev([u]))
        assert int(tok[0]) == want, (u, int(tok[0]))
    R = 4000
    big = logits.expand(R, 4).contiguous()
    tok, _ = ops.sample(_dev(big), do_sample=True, seed=5, rng_seq=_dev(list(range(R)), torch.int32),
                        rng_step=_dev([0] * R, torch.int32))
    freq = torch.bincount(tok.cpu().long(), minlength=4).double() / R
    assert float((freq - torch.tensor([0.1, 0.2, 0.3, 0.4], dtype=torch.float64)).abs().max()) < 4 * math.sqrt(0.25 / R)
    # random logits over a wide vocabulary, against the plain choice fed the same uniform numbers
    g = torch.Generator().manual_seed(0)
    x = torch.randn(64, 5000, generator=g) * 2
    u = torch.rand(64, generator=g)
    tok, _ = ops.sample(_dev(x), do_sample=True, uniforms=_dev(u))
    for r in range(64):
        cdf = torch.softmax(x[r].double(), -1).cumsum(-1)
        t = int(tok[r])
        lo = float(cdf[t - 1]) if t else 0.0
        assert lo - 1e-5 <= float(u[r]) <= float(cdf[t]) + 1e-5, (r, t, float(u[r]), lo, float(cdf[t]))


def test_top_k_by_the_short_way_and_the_long_way():
    """A draw with top-k runs on a short list of candidates, or over the whole row where the list would be long
    (a large k, many equal scores at the threshold): both keep what the plain processors keep, tied scores
    included, and draw the token whose interval of the survivors' cumulative distribution holds the number."""
    ops = _ops()
    g = torch.Generator().manual_seed(7)
    V, R = 65024, 6
    logits = torch.randn(R, V, generator=g) * 3
    logits[1, 100:900] = 50.0        # 800 equal scores at the top: more candidates than the short list holds
    logits[2, 5000:5040] = 40.0      # 40 equal scores that straddle the k-th place
    logits[3, :] = 0.25              # everything equal
    logits[4, :] = -30.0             # ten equal scores at the top-p cut: the first four in index order go
    logits[4, 7] = math.log(0.5)
    logits[4, 100:110] = math.log(0.05)
    u = torch.rand(R, generator=g)
    for kw in (dict(top_k=50), dict(top_k=50, top_p=0.7, temperature=0.6), dict(top_k=300, top_p=0.9), dict(top_k=7, min_p=0.1),
               dict(top_k=256, temperature=1.5), dict(top_k=1), dict(top_k=20, top_p=0.78), dict(top_k=300, top_p=0.78)):
        tok, scores = ops.sample(_dev(logits), do_sample=True, temperature=kw.get("temperature", 1.0), top_k=kw["top_k"],
                                 top_p=kw.get("top_p", 1.0), min_p=kw.get("min_p", 0.0), uniforms=_dev(u))
        tok2, none = ops.sample(_dev(logits), do_sample=True, temperature=kw.get("temperature", 1.0), top_k=kw["top_k"],
                                top_p=kw.get("top_p", 1.0), min_p=kw.get("min_p", 0.0), uniforms=_dev(u), need_scores=False)
        assert none is None and tok2.tolist() == tok.tolist(), "the choice does not depend on whether the scores are wanted"
        for r in range(R):
            want = P.process(logits[r], [], do_sample=True, temperature_=kw.get("temperature", 1.0), top_k_=kw["top_k"],
                             top_p_=kw.get("top_p", 1.0), min_p_=kw.get("min_p"), repetition_penalty_=1.0, suppress_ids=())
            got = scores[r].cpu()
            keep_want, keep_got = want != float("-inf"), _finite_mask(got)
            diff = (keep_want != keep_got).nonzero().flatten().tolist()
            assert len(diff) <= (1 if "top_p" in kw and r != 4 else 0), f"{kw} row {r}: kept sets differ at {diff[:10]}"
            if r == 4 and kw.get("top_p") == 0.78:
                assert keep_got.nonzero().flatten().tolist() == [7, 104, 105, 106, 107, 108, 109]
            assert int(keep_got.sum()) >= min(kw["top_k"], 1)
            cdf = torch.softmax(got.double(), -1).cumsum(-1)
            t = int(tok[r])
            lo = float(cdf[t - 1]) if t else 0.0
            assert keep_got[t] and lo - 1e-5 <= float(u[r]) <= float(cdf[t]) + 1e-5, (kw, r, t, float(u[r]), lo, float(cdf[t]))


@pytest.mark.parametrize("V", [1, 2, 63, 65, 1000, 4100, 65536, 70001])
def test_random_settings_match_plain(V):
    """Random processor settings over vocabularies around the kernel's edges (one score, partly filled tiles,
    the longest row of the short way, a row too long for it): the survivors are the plain code's and the
    chosen token is the one whose interval of their cumulative distribution holds the uniform number."""
    ops = _ops()
    g = torch.Generator().manual_seed(1000 + V)
    R = 4
    for trial in range(6):
        logits = torch.randn(R, V, generator=g) * float(torch.rand((), generator=g) * 4 + 0.5)
        if trial % 3 == 2 and V > 4:  # groups of equal scores
            logits = (logits * 2).round() / 2
        rnd = lambda: float(torch.rand((), generator=g))
        kw = dict(temperature=0.5 + rnd() * 1.5 if rnd() < 0.7 else 1.0,
                  top_k=int(rnd() * min(V, 300)) if rnd() < 0.7 else 0,
                  top_p=0.3 + 0.69 * rnd() if rnd() < 0.6 else 1.0,
                  min_p=0.2 * rnd() if rnd() < 0.3 else 0.0,
                  penalty=0.5 + rnd() * 1.5 if rnd() < 0.5 else 1.0)
        hist = [[int(t) for t in torch.randint(0, V, (n,), generator=g)] for n in (0, 5, 40, 300)]
        off = [0]
        for h in hist:
            off.append(off[-1] + len(h))
        flat = [t for h in hist for t in h]
        u = torch.rand(R, generator=g)
        tok, scores = ops.sample(_dev(logits), do_sample=True, temperature=kw["temperature"], top_k=kw["top_k"], top_p=kw["top_p"],
                                 min_p=kw["min_p"], penalty=kw["penalty"], hist=_dev(flat, torch.int32),
                                 hist_off=_dev(off, torch.int32), uniforms=_dev(u))
        for r in range(R):
            want = P.process(logits[r], hist[r], do_sample=True, temperature_=kw["temperature"], top_k_=kw["top_k"],
                             top_p_=kw["top_p"], min_p_=kw["min_p"] or None, repetition_penalty_=kw["penalty"])
            got = scores[r].cpu()
            keep_want, keep_got = want != float("-inf"), _finite_mask(got)
            diff = (keep_want != keep_got).nonzero().flatten().tolist()
            # a token whose mass sits within rounding of the top-p cut or of the min-p threshold may fall on either side
            loose = kw["top_p"] < 1.0 or kw["min_p"] > 0.0
            assert len(diff) <= (2 if loose else 0), f"V={V} trial {trial} {kw} row {r}: kept sets differ at {diff[:10]}"
            both = keep_want & keep_got
            torch.testing.assert_close(got[both], want[both], rtol=1e-6, atol=1e-6)
            cdf = torch.softmax(got.double(), -1).cumsum(-1)
            t = int(tok[r])
            lo = float(cdf[t - 1]) if t else 0.0
            assert keep_got[t] and lo - 1e-5 <= float(u[r]) <= float(cdf[t]) + 1e-5, (V, trial, kw, r, t)


@pytest.mark.parametrize("V", [5, 211, 4100, 65024, 70001])
def test_typical_epsilon_eta_match_plain(V):
    """The three later warpers alone, together, and behind top-k and top-p: the survivors are the plain code's
    (a token within rounding of a bound may fall on either side), and the draw comes from among them, also
    where typical-p has taken the likeliest token away."""
    ops = _ops()
    g = torch.Generator().manual_seed(77 + V)
    R = 4
    for trial, kw in enumerate((dict(typical_p=0.9), dict(typical_p=0.2), dict(epsilon_cutoff=3e-4), dict(eta_cutoff=2e-3),
                                dict(typical_p=0.95, epsilon_cutoff=1e-4, eta_cutoff=1e-3, temperature=0.8),
                                dict(top_k=40, typical_p=0.6), dict(top_k=50, top_p=0.9, eta_cutoff=0.05, epsilon_cutoff=0.02),
                                dict(typical_p=1e-6), dict(epsilon_cutoff=0.9), dict(eta_cutoff=0.9))):
        logits = torch.randn(R, V, generator=g) * (1.0 + trial % 4)
        logits[R - 1] = (logits[R - 1] * 2).round() / 2  # groups of equal scores
        u = torch.rand(R, generator=g)
        names = dict(temperature=1.0, top_k=0, top_p=1.0, typical_p=1.0, epsilon_cutoff=0.0, eta_cutoff=0.0)
        names.update(kw)
        names["top_k"] = min(names["top_k"], V)
        tok, scores = ops.sample(_dev(logits), do_sample=True, uniforms=_dev(u), **names)
        for r in range(R):
            want = P.process(logits[r], [], do_sample=True, temperature_=names["temperature"], top_k_=names["top_k"],
                             top_p_=names["top_p"], typical_p_=names["typical_p"], epsilon_cutoff_=names["epsilon_cutoff"],
                             eta_cutoff_=names["eta_cutoff"])
            got = scores[r].cpu()
            keep_want, keep_got = want != float("-inf"), _finite_mask(got)
            diff = (keep_want != keep_got).nonzero().flatten().tolist()
            assert len(diff) <= 2, f"V={V} {kw} row {r}: kept sets differ at {diff[:10]} ({int(keep_want.sum())} kept)"
            assert int(keep_got.sum()) >= 1
            both = keep_want & keep_got
            torch.testing.assert_close(got[both], want[both], rtol=1e-6, atol=1e-6)
            cdf = torch.softmax(got.double(), -1).cumsum(-1)
            t = int(tok[r])
            lo = float(cdf[t - 1]) if t else 0.0
            assert keep_got[t] and lo - 1e-5 <= float(u[r]) <= float(cdf[t]) + 1e-5, (V, kw, r, t)
    # the likeliest token goes where it is far from typical, and the draw never returns it
    x = torch.log(torch.tensor([[0.4] + [0.6 / 30] * 30]))
    tok, s = ops.sample(_dev(x), do_sample=True, typical_p=0.5, uniforms=_dev([0.0]))
    assert not _finite_mask(s[0])[0] and int(tok[0]) == 1


@pytest.mark.parametrize("V", [40, 65024, 70001])
def test_banned_tokens_per_row(V):
    """A list of tokens per row that may not be taken: gone from the scores and never chosen, greedy or drawn,
    by the short way and the long way, with the other processors around them."""
    ops = _ops()
    g = torch.Generator().manual_seed(V)
    R = 4
    logits = torch.randn(R, V, generator=g) * 2
    best = logits.argmax(-1).tolist()
    bans = [[best[0], 3], [], [best[2]] + list(range(10, 30)), [V - 1, 0, best[3]]]
    off = [0]
    for b in bans:
        off.append(off[-1] + len(b))
    flat = [t for b in bans for t in b]
    kw_ban = dict(ban=_dev(flat, torch.int32), ban_off=_dev(off, torch.int32))
    tok, scores = ops.sample(_dev(logits), do_sample=False, **kw_ban)
    for r in range(R):
        want = P.suppress(logits[r], bans[r])
        assert torch.equal(scores[r].cpu(), want) and int(tok[r]) == int(want.argmax())
    u = torch.rand(R, generator=g)
    for kw in (dict(top_k=5), dict(top_k=0, top_p=0.9), dict(top_k=20, temperature=0.7, penalty=1.3)):
        hist = [[best[r], 1, 2] for r in range(R)]
        tok, scores = ops.sample(_dev(logits), do_sample=True, uniforms=_dev(u), temperature=kw.get("temperature", 1.0),
                                 top_k=kw["top_k"], top_p=kw.get("top_p", 1.0), penalty=kw.get("penalty", 1.0),
                                 hist=_dev([t for h in hist for t in h], torch.int32),
                                 hist_off=_dev([0, 3, 6, 9, 12], torch.int32), **kw_ban)
        for r in range(R):
            want = P.process(P.suppress(logits[r], bans[r]), hist[r], do_sample=True, temperature_=kw.get("temperature", 1.0),
                             top_k_=kw["top_k"], top_p_=kw.get("top_p", 1.0), repetition_penalty_=kw.get("penalty", 1.0))
            keep_want, keep_got = want != float("-inf"), _finite_mask(scores[r])
            assert int((keep_want != keep_got).sum()) <= (1 if "top_p" in kw else 0), (V, kw, r)
            assert int(tok[r]) not in bans[r] and keep_got[int(tok[r])]


@pytest.mark.parametrize("V", [40, 65024, 70001])
def test_bias_forced_token_and_bonus_on_eos_per_row(V):
    """Additive biases on a list of tokens per row (before the repetition penalty), a token forced in this step
    (over bans that come before it, under bans that come after it), and the bonus on the EOS scores (after the
    removal of invalid values): scores and choices equal the plain processors', greedy and drawn, by the short way
    and the long way, and by the path for vocabularies beyond the bitmaps."""
    ops = _ops()
    g = torch.Generator().manual_seed(V + 1)
    R = 4
    logits = torch.randn(R, V, generator=g) * 2
    best = logits.argmax(-1).tolist()
    eos = [2, V - 3]
    logits[:, eos[0]] = logits[:, eos[0]].abs() + 0.5  # one EOS score above zero, one below: the bonus raises both
    logits[:, eos[1]] = -logits[:, eos[1]].abs() - 0.5
    biases = [[(best[0], -50.0), (5, 3.0)], [], [(V - 1, 60.0)] + [(t, -1.0) for t in range(10, 30)], [(best[3], 0.5)]]
    hist = [[best[r], 5, V - 1] + [1] * 7 for r in range(R)]  # ten ids so far
    off = [0]
    for b in biases:
        off.append(off[-1] + len(b))
    kw_bias = dict(bias_tok=_dev([t for b in biases for t, _ in b], torch.int32),
                   bias_val=_dev([v for b in biases for _, v in b]), bias_off=_dev(off, torch.int32))
    kw_hist = dict(hist=_dev([t for h in hist for t in h], torch.int32), hist_off=_dev([0, 10, 20, 30, 40], torch.int32))
    entries = [{(t,): v for t, v in b} for b in biases]
    # biases and the penalty, greedy: every score
    tok, scores = ops.sample(_dev(logits), do_sample=False, penalty=1.5, **kw_hist, **kw_bias)
    for r in range(R):
        want = P.process(logits[r], hist[r], do_sample=False, sequence_bias_=entries[r], repetition_penalty_=1.5)
        torch.testing.assert_close(scores[r].cpu(), want, rtol=1e-6, atol=1e-6)
        assert int(tok[r]) == int(want.argmax())
    assert int(tok[0]) != best[0] and int(tok[2]) == V - 1, "the biases decide these rows"
    # the bonus on EOS with invalid values removed before it, and with biases
    m = 1.1 ** 7 - 1
    tok, scores = ops.sample(_dev(logits), do_sample=False, eos=_dev(eos, torch.int32), decay=m, **kw_bias)
    for r in range(R):
        want = P.process(logits[r], hist[r], do_sample=False, sequence_bias_=entries[r], eos_ids_=eos,
                         exponential_decay_=(3, 0, 1.1))  # three ids of a prompt, start index 0: 10 - 3 = 7 ids past it
        torch.testing.assert_close(scores[r].cpu(), want, rtol=1e-6, atol=1e-6)
        assert float(want[eos[0]]) > float(logits[r, eos[0]]) and float(want[eos[1]]) > float(logits[r, eos[1]])
    with pytest.raises(ops.KernelError, match="EOS"):
        ops.sample(_dev(logits), do_sample=False, decay=m)
    # a forced token: everything else goes, whatever was banned or suppressed before; a ban that comes after it stays
    forced = [eos[0], 7]
    bans = [[7], [], [eos[0], 7], [3]]
    boff = [0, 1, 1, 3, 4]
    tok, scores = ops.sample(_dev(logits), do_sample=False, forced=_dev(forced, torch.int32), eos=_dev(eos, torch.int32),
                             suppress=_dev([1, 0, 0, 1], torch.int32), ban=_dev([t for b in bans for t in b], torch.int32),
                             ban_off=_dev(boff, torch.int32), **kw_bias)
    for r in range(R):
        want = P.suppress(P.forced_eos(logits[r], 4, 5, forced), bans[r])
        assert torch.equal(scores[r].cpu(), want)
    assert tok.tolist() == [eos[0], eos[0], 0, eos[0]]  # (row 2: both forced tokens are banned afterwards, nothing is left)
    # drawn, with the other processors around them (top-k: the short way; top-p alone: the long way)
    u = torch.rand(R, generator=g)
    for kw in (dict(top_k=5), dict(top_k=0, top_p=0.9), dict(top_k=20, temperature=0.7, penalty=1.3)):
        tok, scores = ops.sample(_dev(logits), do_sample=True, uniforms=_dev(u), temperature=kw.get("temperature", 1.0),
                                 top_k=kw["top_k"], top_p=kw.get("top_p", 1.0), penalty=kw.get("penalty", 1.0),
                                 eos=_dev(eos, torch.int32), decay=m, **kw_hist, **kw_bias)
        for r in range(R):
            want = P.process(logits[r], hist[r], do_sample=True, temperature_=kw.get("temperature", 1.0), top_k_=kw["top_k"],
                             top_p_=kw.get("top_p", 1.0), repetition_penalty_=kw.get("penalty", 1.0),
                             sequence_bias_=entries[r], eos_ids_=eos, exponential_decay_=(3, 0, 1.1))
            keep_want, keep_got = want != float("-inf"), _finite_mask(scores[r])
            assert int((keep_want != keep_got).sum()) <= (1 if "top_p" in kw else 0), (V, kw, r)
            both = keep_want & keep_got
            torch.testing.assert_close(scores[r].cpu()[both], want[both], rtol=1e-5, atol=1e-5)
            assert keep_got[int(tok[r])]


def test_generation_with_bias_forced_last_token_and_bonus_on_eos_equals_plain(folders):
    """Greedy and sampled generation with ``sequence_bias`` (entries of one and of several tokens), ``forced_eos_token_id``
    and ``exponential_decay_length_penalty`` against the plain loop, in a batch of unequal prompts of one length class
    each (the reference counts lengths on the padded batch: one prompt a call keeps both sides on the same count),
    with steps ahead of the host where nothing reads the tokens so far."""
    from pytorch_transformers_amd import AutoModelForCausalLM, GenerationConfig
    from pytorch_transformers_amd.sampling import philox_uniform

    cfg, w = P.read_model(folders["A"])
    g = torch.Generator().manual_seed(6)
    prompts = [torch.randint(0, cfg["vocab_size"], (n,), generator=g).tolist() for n in (4, 9)]
    model = AutoModelForCausalLM.from_pretrained(folders["A"], dtype="float32")
    free = [p + P.generate(cfg, w, p, 12) for p in prompts]
    for i, p in enumerate(prompts):
        new = free[i][len(p):]
        bias = [[[new[1]], -30.0], [new[3:5], -30.0], [[new[0], new[1], new[2]], 5.0]]
        as_dict = {tuple(e[0]): e[1] for e in bias}
        eos = next(t for t in range(cfg["vocab_size"]) if t not in free[i])  # a token that does not come by itself
        # the bias alone: the tokens change where it says
        want = p + P.generate(cfg, w, p, 12, sequence_bias_=as_dict)
        got = model.generate([p], GenerationConfig(max_new_tokens=12, do_sample=False, eos_token_id=None, sequence_bias=bias))
        assert got == [want] and want != free[i]
        # a forced last token, with and without a bias on single tokens (which lets steps run ahead of the host)
        for sb in (None, [[[new[1]], -30.0]]):
            want = p + P.generate(cfg, w, p, 6, eos_ids=(eos,), forced_eos_ids=[eos],
                                  sequence_bias_={tuple(e[0]): e[1] for e in sb} if sb else None)
            got = model.generate([p], GenerationConfig(max_new_tokens=6, do_sample=False, eos_token_id=eos,
                                                       forced_eos_token_id=eos, sequence_bias=sb))
            assert got == [want] and want[-1] == eos and len(want) == len(p) + 6
        # the bonus on EOS: the sequence ends earlier than without it, and where the plain loop ends
        late = p + P.generate(cfg, w, p, 40, eos_ids=(eos,), no_repeat_ngram_size_=2)
        want = p + P.generate(cfg, w, p, 40, eos_ids=(eos,), no_repeat_ngram_size_=2, exponential_decay_length_penalty=(2, 1.6))
        got = model.generate([p], GenerationConfig(max_new_tokens=40, do_sample=False, eos_token_id=eos,
                                                   no_repeat_ngram_size=2, exponential_decay_length_penalty=(2, 1.6)))
        assert got == [want] and len(want) < len(late) and want[-1] == eos
        # sampled, with all three, from the same uniform numbers
        us = [philox_uniform(3, 0, s) for s in range(10)]
        want = p + P.generate(cfg, w, p, 10, uniforms=us, temperature_=0.9, eos_ids=(eos,), forced_eos_ids=[eos],
                              sequence_bias_=as_dict, exponential_decay_length_penalty=(1, 1.2))
        got = model.generate([p], GenerationConfig(max_new_tokens=10, do_sample=True, temperature=0.9, top_k=0, seed=3,
                                                   eos_token_id=eos, forced_eos_token_id=eos, sequence_bias=bias,
                                                   exponential_decay_length_penalty=(1, 1.2)))[0]
        _same_or_a_draw_on_a_boundary(cfg, w, got, want, len(p), us, 0.9)
    with pytest.raises(ValueError, match="eos_token_id"):
        model.generate([prompts[0]], GenerationConfig(max_new_tokens=3, eos_token_id=None, exponential_decay_length_penalty=(1, 1.2)))


def test_sampled_generation_goes_on_from_kept_slots_with_its_random_stream(folders):
    """Five sampled tokens at once equal three and then two more from kept slots when the second call starts each
    sequence's random stream where the first one stopped (``rng_step_start``); started at 0 again, it would draw
    with the first call's numbers."""
    from pytorch_transformers_amd import AutoModelForCausalLM

    model = AutoModelForCausalLM.from_pretrained(folders["A"], dtype="float32")
    prompts = [[3, 1, 4, 1, 5], [9, 2], [6, 5, 3, 5, 8, 9, 7]]
    kw = dict(do_sample=True, temperature=1.5, top_k=0, seed=11, eos_token_id=None)
    at_once = model.generate(prompts, max_new_tokens=5, **kw)
    first = model.generate(prompts, max_new_tokens=3, keep_slots=True, **kw)
    assert first.rng_steps == [3, 3, 3]
    again = model.generate(first.sequences, max_new_tokens=2, cache=first.cache, slots=first.slots, **kw)  # from draw 0
    assert not first.cache.live_slots()
    first = model.generate(prompts, max_new_tokens=3, keep_slots=True, **kw)
    more = model.generate(first.sequences, max_new_tokens=2, cache=first.cache, slots=first.slots,
                          rng_step_start=first.rng_steps, **kw)
    assert more == at_once
    assert again != at_once, "the stream started anew gives other tokens: the test sees the counter"
    assert not first.cache.live_slots()


def test_generation_without_repeated_ngrams_equals_plain(folders):
    """Greedy generation with no_repeat_ngram_size and bad_words_ids against the plain loop: a tiny random model
    repeats itself soon, so the option decides tokens."""
    from pytorch_transformers_amd import AutoModelForCausalLM, GenerationConfig

    cfg, w = P.read_model(folders["A"])
    g = torch.Generator().manual_seed(5)
    prompts = [torch.randint(0, cfg["vocab_size"], (n,), generator=g).tolist() for n in (3, 9)]
    model = AutoModelForCausalLM.from_pretrained(folders["A"], dtype="float32")
    free = [p + P.generate(cfg, w, p, 24) for p in prompts]
    bad = [[free[0][len(prompts[0]) + 1]], free[1][len(prompts[1]) + 2:len(prompts[1]) + 4]]
    for opts in (dict(no_repeat_ngram_size=1), dict(no_repeat_ngram_size=2), dict(bad_words_ids=bad),
                 dict(no_repeat_ngram_size=3, bad_words_ids=bad)):
        want = [p + P.generate(cfg, w, p, 24, no_repeat_ngram_size_=opts.get("no_repeat_ngram_size", 0),
                               bad_words_ids_=opts.get("bad_words_ids")) for p in prompts]
        got = model.generate(prompts, GenerationConfig(max_new_tokens=24, do_sample=False, eos_token_id=None, **opts))
        assert got == want, opts
        assert want != free, f"{opts} changed nothing: the test would not see the option"
    new = want[0][len(prompts[0]):]
    grams = [tuple(want[0][j:j + 3]) for j in range(len(want[0]) - 2)]
    assert len(set(grams)) == len(grams) and bad[0][0] not in new
    # suppress_tokens never come, begin_suppress_tokens do not come first
    first, second = free[0][len(prompts[0])], free[0][len(prompts[0]) + 1]
    got = model.generate(prompts[:1], GenerationConfig(max_new_tokens=24, do_sample=False, eos_token_id=None,
                                                       suppress_tokens=[second], begin_suppress_tokens=[first]))
    new = got[0][len(prompts[0]):]
    assert second not in new and new[0] != first
    want_first = int(P.suppress(P.forward(cfg, w, prompts[0])[-1].float(), [first, second]).argmax())
    assert new[0] == want_first


def test_counter_based_uniforms():
    """Same (seed, sequence, step) -> same draw whatever the batch; the host function gives the number."""
    from pytorch_transformers_amd.sampling import philox_uniform

    ops = _ops()
    V = 1000
    x = torch.randn(6, V, generator=torch.Generator().manual_seed(1))
    seqs, steps = [4, 9, 2, 7, 7, 1], [0, 3, 3, 1, 2, 0]
    tok_all, _ = ops.sample(_dev(x), do_sample=True, seed=1234, rng_seq=_dev(seqs, torch.int32), rng_step=_dev(steps, torch.int32))
    for r in range(6):
        alone, _ = ops.sample(_dev(x[r:r + 1]), do_sample=True, seed=1234, rng_seq=_dev([seqs[r]], torch.int32),
                              rng_step=_dev([steps[r]], torch.int32))
        assert int(alone[0]) == int(tok_all[r])
        u = philox_uniform(1234, seqs[r], steps[r])
        assert 0.0 <= u < 1.0
        via_u, _ = ops.sample(_dev(x[r:r + 1]), do_sample=True, uniforms=_dev([u]))
        assert int(via_u[0]) == int(tok_all[r])
    us = [philox_uniform(7, s, 0) for s in range(2000)]
    assert abs(sum(us) / len(us) - 0.5) < 0.03 and len(set(us)) > 1990
    assert philox_uniform(7, 3, 0) != philox_uniform(8, 3, 0) != philox_uniform(8, 3, 1)


# --- generation through the entry point ---------------------------------------------------------------
@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    root = str(tmp_path_factory.mktemp("gen"))
    return {n: write_model(n, root, std=LIVELY_STD) for n in ("A", "B")}


def test_greedy_generation_equals_plain(folders):
    """Tiny A: batch of 3 prompts of 5/11/17 ids, 16 greedy tokens, 32-bit."""
    from pytorch_transformers_amd import AutoModelForCausalLM, GenerationConfig

    cfg, w = P.read_model(folders["A"])
    g = torch.Generator().manual_seed(0)
    prompts = [torch.randint(0, cfg["vocab_size"], (n,), generator=g).tolist() for n in (5, 11, 17)]
    want = [p + P.generate(cfg, w, p, 16) for p in prompts]
    # tokens that keep changing: equality of constant tokens would hold with the layers switched off
    assert all(len(set(w_[len(p):])) > 3 for p, w_ in zip(prompts, want)), want
    model = AutoModelForCausalLM.from_pretrained(folders["A"], dtype="float32")
    got = model.generate(prompts, GenerationConfig(max_new_tokens=16, do_sample=False, eos_token_id=None))
    assert got == want
    # one batch after another, and a stop token that ends one sequence early
    eos = want[1][len(prompts[1]) + 4]
    got = model.generate(prompts, GenerationConfig(max_new_tokens=16, eos_token_id=eos), batch_size=2)
    for p, g_, w_ in zip(prompts, got, want):
        new = w_[len(p):]
        cut = new.index(eos) + 1 if eos in new else len(new)
        assert g_ == p + new[:cut]
    bf = AutoModelForCausalLM.from_pretrained(folders["A"], dtype="bfloat16")
    got_bf = bf.generate(prompts, max_new_tokens=16, do_sample=False, eos_token_id=None)
    # bfloat16: equal up to a first difference, which must be a near tie of the plain logits (after it the
    # sequences differ by right)
    for p, got_seq, want_seq in zip(prompts, got_bf, want):
        if got_seq == want_seq:
            continue
        k = next(j for j, (a, b) in enumerate(zip(got_seq, want_seq)) if a != b)
        assert k >= len(p)
        logits = P.forward(cfg, w, want_seq[:k])[-1].float()
        gap = float(logits[want_seq[k]] - logits[got_seq[k]])
        assert 0 <= gap <= 4e-2 * float(logits.abs().max()), \
            f"bfloat16 took token {got_seq[k]} at position {k}, {gap:.3f} below the plain choice"


def test_sampled_generation_equals_plain_fed_the_same_uniforms(folders):
    """Tiny B: batch of 4 prompts of 1/7/20/33 ids, 24 tokens at temperature 0.8 (32-bit), alone and batched."""
    from pytorch_transformers_amd import AutoModelForCausalLM, GenerationConfig
    from pytorch_transformers_amd.sampling import philox_uniform

    cfg, w = P.read_model(folders["B"])
    g = torch.Generator().manual_seed(1)
    prompts = [torch.randint(0, cfg["vocab_size"], (n,), generator=g).tolist() for n in (1, 7, 20, 33)]
    gen = GenerationConfig(max_new_tokens=24, do_sample=True, temperature=0.8, top_k=0, eos_token_id=None, seed=77)
    model = AutoModelForCausalLM.from_pretrained(folders["B"], dtype="float32")
    got = model.generate(prompts, gen)
    for i, p in enumerate(prompts):
        us = [philox_uniform(77, i, s) for s in range(24)]
        want = p + P.generate(cfg, w, p, 24, uniforms=us, temperature_=0.8)
        # a draw within rounding of a CDF boundary may differ and then the tails differ: compare up to the first
        # difference and require it to be such a boundary case
        if got[i] != want:
            k = next(j for j, (a, b) in enumerate(zip(got[i], want)) if a != b)
            logits = P.forward(cfg, w, want[:k])[-1].float() / 0.8
            cdf = torch.softmax(logits.double(), -1).cumsum(-1)
            u = us[k - len(p)]
            assert min(abs(float(cdf[t]) - u) for t in (got[i][k], want[k], got[i][k] - 1, want[k] - 1) if t >= 0) < 1e-5
    alone = model.generate([prompts[2]], gen, rng_ids=[2])
    assert alone[0] == got[2]
    two = model.generate(prompts, gen, batch_size=2)
    assert two == got


def test_steps_ahead_of_the_host_choose_what_the_loop_that_waits_chooses(folders):
    """Tiny B, six prompts of 3 to 64 ids in batches of four, 40 tokens, a stop token that ends some early: with every
    step launched from the tokens on the device, and with a wait after every step (a streamer makes the loop wait)."""
    from pytorch_transformers_amd import AutoModelForCausalLM, GenerationConfig

    cfg, _ = P.read_model(folders["B"])
    g = torch.Generator().manual_seed(5)
    prompts = [torch.randint(0, cfg["vocab_size"], (n,), generator=g).tolist() for n in (3, 9, 1, 30, 17, 64)]
    for dtype in ("float32", "bfloat16"):
        model = AutoModelForCausalLM.from_pretrained(folders["B"], dtype=dtype)
        assert model.steps_ahead
        for kw in (dict(do_sample=False), dict(do_sample=True, temperature=0.9, top_k=50, top_p=0.95, seed=3)):
            free_run = model.generate(prompts, GenerationConfig(max_new_tokens=40, eos_token_id=None, **kw), batch_size=4)
            eos = free_run[1][len(prompts[1]) + 5]
            gen = GenerationConfig(max_new_tokens=40, eos_token_id=eos, min_new_tokens=2, **kw)
            cache = model.new_cache(4 * 128, max_slots=4)
            ahead = model.generate(prompts, gen, batch_size=4, cache=cache)
            assert not cache.live_slots() and cache.free_pages() == cache.num_pages
            waits = model.generate(prompts, gen, batch_size=4, cache=cache, streamer=lambda i, t: None)
            assert ahead == waits
            ended_early = [len(a) - len(p) < 40 for a, p in zip(ahead, prompts)]
            assert any(ended_early) and not all(ended_early), ended_early
            for a, p in zip(ahead, prompts):  # the stop token is kept, nothing follows it, and it is not among the first two
                new = a[len(p):]
                assert eos not in new[:-1] and (len(new) == 40 or new[-1] == eos) and eos not in new[:2]


def test_a_step_from_tokens_on_the_device_equals_the_step_from_the_same_tokens_on_the_host(folders):
    """Tiny A in bfloat16: three sequences' next step from a ``TokensAhead`` (all rows, then two of them in another
    order) against the step from the tokens as lists, with captured steps and, where there are none, after a wait."""
    from pytorch_transformers_amd import AutoModelForCausalLM, GenerationConfig
    from pytorch_transformers_amd.sampling import Sampler, TokensAhead

    model = AutoModelForCausalLM.from_pretrained(folders["A"], dtype="bfloat16")
    sampler = Sampler(GenerationConfig(do_sample=False), model.vocab_size, model.device)
    prompts = [[5, 6, 7, 8], [9, 10], [11, 12, 13, 14, 15, 16]]

    def start():
        cache = model.new_cache(3 * 64, max_slots=3)
        slots = [cache.alloc() for _ in prompts]
        return cache, slots, model.step(cache, slots, prompts, "last")

    for graphs in (True, False):
        model.use_graphs = graphs
        assert model.steps_ahead == graphs
        (c1, s1, l1), (c2, s2, l2) = start(), start()
        ahead, _ = sampler.sample(l1, rng_seq=[0, 1, 2], rng_step=[0, 0, 0], need_scores=False, ahead=True)
        assert isinstance(ahead, TokensAhead) and len(ahead) == 3
        host_tokens, _ = sampler.sample(l2, rng_seq=[0, 1, 2], rng_step=[0, 0, 0], need_scores=False)
        a = model.step(c1, s1, ahead.take(None), "last", own_logits=False).clone()
        b = model.step(c2, s2, [[t] for t in host_tokens], "last")
        assert ahead.tolist() == host_tokens and torch.equal(a, b)
        # two of the three rows, in another order
        a = model.step(c1, [s1[2], s1[0]], ahead.take([2, 0]), "last", own_logits=False).clone()
        b = model.step(c2, [s2[2], s2[0]], [[host_tokens[2]], [host_tokens[0]]], "last")
        assert torch.equal(a, b)
        if graphs:
            with pytest.raises(Exception, match="tokens ahead for 2"):  # three sequences, two rows taken
                model.step(c1, s1, ahead.take([2, 0]), "last")
    model.use_graphs = True


def test_pipeline_entry(folders):
    from pytorch_transformers_amd import pipeline

    cfg, w = P.read_model(folders["A"])
    pipe = pipeline("text-generation", model=folders["A"], dtype="float32")
    out = pipe([[3, 4, 5]], max_new_tokens=4, do_sample=False, eos_token_id=None)
    assert len(out) == 1 and out[0][0]["generated_token_ids"] == [3, 4, 5] + P.generate(cfg, w, [3, 4, 5], 4)
    new_only = pipe([3, 4, 5], max_new_tokens=4, do_sample=False, eos_token_id=None, return_full_text=False)
    assert new_only[0]["generated_token_ids"] == P.generate(cfg, w, [3, 4, 5], 4)


def _run_cli(*argv):
    """The command line as a program: ``python -m pytorch_transformers_amd.run_generation ...``; returns the
    sequences it printed, in order."""
    import os
    import subprocess
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    p = subprocess.run([sys.executable, "-m", "pytorch_transformers_amd.run_generation", *argv], cwd=root,
                       capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-3000:]
    lines = [ln for ln in p.stdout.splitlines() if ln.strip()]
    heads = [i for i, ln in enumerate(lines) if ln.startswith("=== GENERATED SEQUENCE")]
    assert [lines[i] for i in heads] == [f"=== GENERATED SEQUENCE {n + 1} ===" for n in range(len(heads))], p.stdout
    return [[int(t) for t in lines[i + 1].split(",")] for i in heads]


def _same_or_a_draw_on_a_boundary(cfg, w, got, want, prompt_len, uniforms, temperature):
    """Equal sequences, or a first difference where the uniform number lies within rounding of a boundary of the
    cumulative distribution (after which the tails differ by right)."""
    if got == want:
        return
    k = next(j for j, (a, b) in enumerate(zip(got, want)) if a != b)
    logits = P.forward(cfg, w, want[:k])[-1].float() / temperature
    cdf = torch.softmax(logits.double(), -1).cumsum(-1)
    u = uniforms[k - prompt_len]
    assert min(abs(float(cdf[t]) - u) for t in (got[k], want[k], got[k] - 1, want[k] - 1) if t >= 0) < 1e-5, \
        f"position {k}: the program drew {got[k]}, the plain implementation {want[k]}"


def test_command_line_as_a_program(folders, tmp_path):
    """run_generation as a subprocess on a tiny folder, in 32-bit: greedy and sampled with --seed, several
    sequences per prompt, a stop token, and a model made from --random_config; the printed ids are the plain
    implementation's (fed the same uniform numbers where it samples)."""
    import json

    from pytorch_transformers_amd.config import AutoConfig
    from pytorch_transformers_amd.sampling import philox_uniform
    from pytorch_transformers_amd.weights import write_random_model

    cfg, w = P.read_model(folders["A"])
    eos_default = 11  # FalconConfig's eos_token_id, which the tiny configuration does not change
    prompts = [[1, 2, 3], [4, 5]]
    # greedy, two prompts in one call
    got = _run_cli("--model_type", "falcon", "--model_name_or_path", folders["A"], "--prompt_ids", "1,2,3;4,5", "--length",
                   "7", "--greedy", "--dtype", "float32")
    want = [p + P.generate(cfg, w, p, 7, eos_ids=(eos_default,)) for p in prompts]
    assert got == want
    assert all(len(set(s[len(p):])) > 3 for s, p in zip(want, prompts)), "tokens that keep changing carry the comparison"
    # sampled with a seed, two sequences for each prompt, and a stop token that some sequence meets
    stop = want[0][len(prompts[0]) + 2]
    got = _run_cli("--model_name_or_path", folders["A"], "--prompt_ids", "1,2,3;4,5", "--length", "6", "--seed", "7",
                   "--temperature", "0.8", "--k", "0", "--p", "1.0", "--num_return_sequences", "2", "--stop_token_id",
                   str(stop), "--dtype", "float32")
    assert len(got) == 4
    for n, seq in enumerate(got):  # sequence n is prompt n // 2; its random stream is number n
        p = prompts[n // 2]
        us = [philox_uniform(7, n, s) for s in range(6)]
        want_n = p + P.generate(cfg, w, p, 6, uniforms=us, temperature_=0.8, eos_ids=(stop,))
        _same_or_a_draw_on_a_boundary(cfg, w, seq, want_n, len(p), us, 0.8)
        assert stop not in seq[len(p):-1], "a sequence went on after its stop token"
    assert got[0] != got[1] or got[2] != got[3], "two sequences of one prompt come from different random streams"
    # a model folder made on the spot from a configuration file and a seed
    raw = dict(TINY["C"], initializer_range=LIVELY_STD)
    cfg_file = tmp_path / "c.json"
    cfg_file.write_text(json.dumps(raw))
    got = _run_cli("--random_config", str(cfg_file), "--random_seed", "3", "--prompt_ids", "9,8,7,6", "--length", "5",
                   "--greedy", "--dtype", "float32")
    folder = write_random_model(str(tmp_path / "same"), AutoConfig.from_dict(raw), 3)
    cfg_c, w_c = P.read_model(folder)
    assert got == [[9, 8, 7, 6] + P.generate(cfg_c, w_c, [9, 8, 7, 6], 5, eos_ids=(eos_default,))]


WORDS = ["[UNK]", "the", "cat", "sat", "on", "a", "mat", "dog", "ran", "to", "its", "house", "and", "then", "slept", "all",
         "day", "long", "while", "it", "rained", "outside", "again", "today"]


def _folder_with_a_tokenizer(tmp_path):
    """A tiny model whose vocabulary is ``WORDS``, with a word-level ``tokenizer.json`` beside its weights (written
    with the ``tokenizers`` package: words split at spaces, joined by spaces again)."""
    from tokenizers import Tokenizer
    from tokenizers.models import WordLevel
    from tokenizers.pre_tokenizers import Whitespace

    from tiny import write_config

    folder = write_config(dict(TINY["C"], vocab_size=len(WORDS)), str(tmp_path), "words", seed=8, std=LIVELY_STD)
    tok = Tokenizer(WordLevel({w: i for i, w in enumerate(WORDS)}, unk_token="[UNK]"))
    tok.pre_tokenizer = Whitespace()
    tok.save(os.path.join(folder, "tokenizer.json"))
    return folder


def test_text_through_the_command_line_and_the_pipeline(tmp_path):
    """The text path of both entry points (examples/pytorch/text-generation/run_generation.py:365-441,
    src/transformers/pipelines/text_generation.py:349-449): ``--prompt``, ``--prefix`` and ``--stop_token`` of the
    program, text in and out of the pipeline, ``stop_strings`` and ``return_full_text``.  Under the text the ids are
    the plain loop's."""
    import subprocess
    import sys

    from pytorch_transformers_amd import pipeline

    folder = _folder_with_a_tokenizer(tmp_path)
    cfg, w = P.read_model(folder)
    ids_of = lambda text: [WORDS.index(t) if t in WORDS else 0 for t in text.split()]
    text_of = lambda ids: " ".join(WORDS[t] for t in ids)
    eos = 11  # FalconConfig's default, "house" here
    prompt, prefix = "cat sat on zebra", "the "
    ids = ids_of(prefix + prompt)
    assert ids == [1, 2, 3, 4, 0]  # a word the vocabulary lacks becomes [UNK]
    new = P.generate(cfg, w, ids, 10, eos_ids=(eos,))
    assert len(set(new)) > 4, "tokens that keep changing carry the comparison"
    whole = text_of(ids + new)

    def program(*argv):
        root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
        p = subprocess.run([sys.executable, "-m", "pytorch_transformers_amd.run_generation", "--model_name_or_path", folder,
                            "--dtype", "float32", *argv], cwd=root, capture_output=True, text=True, timeout=300)
        assert p.returncode == 0, p.stderr[-3000:]
        lines = [ln for ln in p.stdout.splitlines() if ln.strip()]
        assert lines[0] == "=== GENERATED SEQUENCE 1 ===", p.stdout
        return lines[1:]

    assert program("--prompt", prompt, "--prefix", prefix, "--length", "10", "--greedy") == [whole]
    # the older name of --prefix, and the reference's --jit, which changes nothing here (run_generation.py:318, :382, :332)
    assert program("--prompt", prompt, "--padding_text", prefix, "--length", "10", "--greedy", "--jit") == [whole]
    stop = WORDS[new[3]]  # a word that is generated: the printed text is cut in front of its first occurrence
    assert whole.find(stop) > 0
    assert program("--prompt", prompt, "--prefix", prefix, "--length", "10", "--greedy", "--stop_token", stop) == \
        [whole[:whole.find(stop)]]
    # the prompt read from standard input when none is given (run_generation.py:365)
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    p = subprocess.run([sys.executable, "-m", "pytorch_transformers_amd.run_generation", "--model_name_or_path", folder,
                        "--dtype", "float32", "--length", "4", "--greedy"], cwd=root, input=prefix + prompt + "\n",
                       capture_output=True, text=True, timeout=300)
    assert p.returncode == 0 and text_of(ids + new[:4]) in p.stdout, p.stderr[-2000:]

    pipe = pipeline("text-generation", model=folder, dtype="float32")
    out = pipe(prefix + prompt, max_new_tokens=10, do_sample=False)
    assert out == [{"generated_text": whole}]
    assert pipe(prompt, prefix=prefix, max_new_tokens=10, do_sample=False, return_full_text=False) == \
        [{"generated_text": text_of(new)}]
    # a stop string of two words, completed by the fourth new token: that token is kept, nothing follows it
    stop_string = text_of(new[2:4])
    cut = next(k for k in range(1, len(new) + 1) if stop_string in text_of(new[:k]))
    assert cut < len(new)
    out = pipe([prefix + prompt, "the dog"], max_new_tokens=10, do_sample=False, stop_strings=[stop_string])
    assert out[0] == [{"generated_text": text_of(ids + new[:cut])}]
    other = P.generate(cfg, w, ids_of("the dog"), 10, eos_ids=(eos,))
    cut2 = next((k for k in range(1, len(other) + 1) if stop_string in text_of(other[:k])), len(other))
    assert out[1] == [{"generated_text": text_of(ids_of("the dog") + other[:cut2])}]
    # token ids through the same pipeline stay ids
    assert pipe([ids], max_new_tokens=3, do_sample=False)[0] == [{"generated_token_ids": ids + new[:3]}]
    # a streamer sees the same text while it is generated, prompt included or not
    from pytorch_transformers_amd import TextIteratorStreamer

    for skip in (False, True):
        it = TextIteratorStreamer(pipe.tokenizer, skip_prompt=skip, timeout=60)
        assert pipe(prefix + prompt, max_new_tokens=10, do_sample=False, streamer=it) == [{"generated_text": whole}]
        assert "".join(it) == (text_of(new) if skip else whole)
    with pytest.raises(ValueError, match="tokenizer"):
        pipeline("text-generation", model=pipe.model)("the cat", max_new_tokens=2)


def test_generation_goes_on_from_kept_slots(folders):
    """tests/generation/test_utils.py:1775-1855 in this engine's terms: four new tokens at once equal three and then
    one more from the slots the first call kept, for a batch of unequal prompts."""
    from pytorch_transformers_amd import AutoModelForCausalLM

    model = AutoModelForCausalLM.from_pretrained(folders["A"], dtype="float32")
    prompts = [[3, 1, 4, 1, 5], [9, 2], [6, 5, 3, 5, 8, 9, 7]]
    at_once = model.generate(prompts, max_new_tokens=4, do_sample=False, eos_token_id=None)
    first = model.generate(prompts, max_new_tokens=3, do_sample=False, eos_token_id=None, keep_slots=True)
    assert [len(s) for s in first.sequences] == [len(p) + 3 for p in prompts]
    more = model.generate(first.sequences, max_new_tokens=1, do_sample=False, eos_token_id=None, cache=first.cache,
                          slots=first.slots)
    assert more == at_once
    assert not first.cache.live_slots() and first.cache.free_pages() == first.cache.num_pages


def test_greedy_without_scores_is_an_argmax():
    """The plain argmax path: ties go to the lowest index, rows of odd length start off a 16-byte boundary."""
    from pytorch_transformers_amd import ops

    for V in (1, 5, 211, 4099, 65024):
        g = torch.Generator().manual_seed(V)
        logits = torch.randn(5, V, generator=g).cuda()
        if V > 4:
            logits[1, [V - 1, 2]] = 50.0  # equal maxima: the lower index wins
            logits[2, V - 1] = 60.0  # the last element, in the tail past the 16-byte groups
            logits[3, 0] = 70.0  # the first element, before the first 16-byte boundary of an odd row
        tok, scores = ops.sample(logits, do_sample=False, need_scores=False)
        assert scores is None
        want = [int(torch.nonzero(r == r.max())[0]) for r in logits]
        assert tok.tolist() == want
        full, _ = ops.sample(logits, do_sample=False)
        assert full.tolist() == want


def test_the_callers_processors_and_criteria_through_generate_equal_plain(folders):
    """Tiny B in 32-bit, prompts of 2 to 19 ids in one batch.  The caller's processor (here: odd ids are forbidden and
    the id behind the last one is raised) runs behind the options' processors (a repetition penalty) and in front of
    the warpers: with top-k 1 a draw can only take the token the processor has made the best, which a processor run
    behind the warpers could not have made it.  A criterion ends its rows with the token that fulfils it."""
    from pytorch_transformers_amd import AutoModelForCausalLM, GenerationConfig, LogitsProcessorList, StoppingCriteriaList

    cfg, w = P.read_model(folders["B"])
    V = cfg["vocab_size"]
    g = torch.Generator().manual_seed(5)
    prompts = [torch.randint(0, V, (n,), generator=g).tolist() for n in (2, 19, 7)]
    model = AutoModelForCausalLM.from_pretrained(folders["B"], dtype="float32")
    calls = []

    def even_only(input_ids, scores):
        assert input_ids.dtype == torch.long and input_ids.is_cuda and scores.dtype == torch.float32
        assert scores.shape == (input_ids.shape[0], V)
        calls.append(tuple(input_ids.shape))
        out = scores.clone()
        out[:, 1::2] = float("-inf")
        return out

    def even_only_plain(history, s):
        s = s.clone()
        s[1::2] = float("-inf")
        return s

    gen = GenerationConfig(max_new_tokens=12, do_sample=False, repetition_penalty=1.3, eos_token_id=None, pad_token_id=0)
    got = model.generate(prompts, gen, logits_processor=LogitsProcessorList([even_only]))
    for p, o in zip(prompts, got):
        assert o == p + P.generate(cfg, w, p, 12, repetition_penalty_=1.3, custom_=[even_only_plain])
        assert all(t % 2 == 0 for t in o[len(p):])
    assert calls[0] == (3, 19) and calls[1] == (3, 20)  # the rows' ids so far, as one rectangle

    def raise_the_next_id(input_ids, scores):
        out = scores.clone()
        out[torch.arange(out.shape[0]), (input_ids[:, -1] + 1) % V] += 1e4
        return out

    drawn = model.generate(prompts, GenerationConfig(max_new_tokens=6, do_sample=True, top_k=1, temperature=0.7, seed=3,
                                                     eos_token_id=None), logits_processor=[raise_the_next_id])
    for p, o in zip(prompts, drawn):
        assert o[len(p):] == [(p[-1] + k) % V for k in range(1, 7)]

    ends_on_a_multiple_of_five = lambda input_ids, scores: input_ids[:, -1] % 5 == 0
    stopped = model.generate(prompts, GenerationConfig(max_new_tokens=30, do_sample=False, eos_token_id=None),
                             stopping_criteria=StoppingCriteriaList([ends_on_a_multiple_of_five]))
    lens = set()
    for p, o in zip(prompts, stopped):
        want = P.generate(cfg, w, p, 30, stop_when=[lambda seq: seq[-1] % 5 == 0])
        assert o == p + want
        lens.add(len(want))
    assert len(lens) > 1 and min(lens) < 30, f"rows must end at different steps, some by the criterion: {lens}"


def test_tensor_prompts_in_the_references_spelling(folders):
    """``model.generate(input_ids=..., attention_mask=...)`` with rows padded on the left gives, row by row, what the
    same prompts give as lists, as one tensor padded as the reference pads it."""
    from pytorch_transformers_amd import AutoModelForCausalLM, GenerationConfig

    model = AutoModelForCausalLM.from_pretrained(folders["A"], dtype="float32")
    g = torch.Generator().manual_seed(2)
    prompts = [torch.randint(1, model.vocab_size, (n,), generator=g).tolist() for n in (9, 2, 5)]
    ids = torch.zeros((3, 9), dtype=torch.long)
    mask = torch.zeros((3, 9), dtype=torch.long)
    for r, p in enumerate(prompts):
        ids[r, 9 - len(p):] = torch.tensor(p)
        mask[r, 9 - len(p):] = 1
    gen = GenerationConfig(max_new_tokens=7, do_sample=False, eos_token_id=None, pad_token_id=0)
    lists = model.generate(prompts, gen)
    out = model.generate(input_ids=ids.cuda(), attention_mask=mask.cuda(), generation_config=gen)
    assert out.is_cuda and out.shape == (3, 16)
    for r, (p, want) in enumerate(zip(prompts, lists)):
        assert out[r].tolist() == [0] * (9 - len(p)) + want
