"""The cache's bookkeeping: slots and pages are never lost, held twice or freed twice (no GPU)."""
import random

import pytest
import torch

from pytorch_transformers_amd.cache import CacheError, CacheFull, PagedCache
from pytorch_transformers_amd.engine.spec import CACHE_FULL, CACHE_STATE, CACHE_WINDOW, CacheGroupSpec
from pytorch_transformers_amd.engine.step import StepError, plan_step

KV = CacheGroupSpec("kv", CACHE_FULL, num_layers=2, kv_heads=2, head_dim=16)


def _cache(max_tokens=512, groups=(KV,), **kw):
    return PagedCache(list(groups), max_tokens, torch.float32, "cpu", **kw)


def test_shapes_and_capacity():
    c = _cache(1000)
    assert c.num_pages == 16 and c.max_slots == 16  # 1000 tokens round up to 16 pages of 64
    k, v = c.kv_layer("kv", 1)
    # value pages are transposed; one page more than sequences can hold is the scratch page of padding rows
    assert k.shape == (17, 2, 64, 16) and v.shape == (17, 2, 16, 64) and c.scratch_page == 16 and c.scratch_slot == 16
    assert c.bytes_per_token() == 2 * 2 * 2 * 16 * 4


def test_slots_are_reused_lowest_first_and_lengths_reset():
    c = _cache()
    a, b, d = c.alloc(), c.alloc(), c.alloc()
    assert (a, b, d) == (0, 1, 2)
    c.reserve([a, b], [70, 3]); c.commit([a, b], [70, 3])
    assert c.length(a) == 70 and len(c.page_list("kv", a)) == 2 and len(c.page_list("kv", b)) == 1
    pages_a = list(c.page_list("kv", a))
    c.free(a)
    assert c.free_pages() == c.num_pages - 1
    again = c.alloc()
    assert again == a and c.length(again) == 0 and c.page_list("kv", again) == []
    c.reserve([again], [1])
    assert c.page_list("kv", again)[0] == min(pages_a)  # freed pages are handed out again
    c.check_consistent()


def test_errors():
    c = _cache(128)
    s = c.alloc()
    with pytest.raises(CacheError, match="not allocated"):
        c.length(5)
    with pytest.raises(CacheError, match="not allocated"):
        c.reserve([5], [1])
    with pytest.raises(CacheError, match="twice"):
        c.reserve([s, s], [1, 1])
    c.free(s)
    with pytest.raises(CacheError, match="not allocated"):
        c.free(s)  # freed twice
    t = c.alloc()
    c.reserve([t], [128]); c.commit([t], [128])
    with pytest.raises(CacheFull, match="needs 1 more pages"):
        c.reserve([t], [1])
    u = c.alloc()
    with pytest.raises(CacheFull):
        c.reserve([u], [1])
    assert c.page_list("kv", u) == []  # a refused reservation takes nothing
    c2 = _cache(128, max_slots=1)
    c2.alloc()
    with pytest.raises(CacheFull, match="no free slot"):
        c2.alloc()
    with pytest.raises(CacheError, match="positive window"):
        _cache(groups=(CacheGroupSpec("w", CACHE_WINDOW, 1, 1, 16),))


def test_reserve_is_all_or_nothing():
    c = _cache(192)  # 3 pages
    a, b = c.alloc(), c.alloc()
    with pytest.raises(CacheFull):
        c.reserve([a, b], [100, 100])  # needs 4
    assert c.free_pages() == 3 and c.page_list("kv", a) == [] and c.page_list("kv", b) == []


def test_state_groups_are_zeroed_on_alloc():
    st = CacheGroupSpec("s", CACHE_STATE, num_layers=2, state_shape=(3, 4))
    c = _cache(256, groups=(KV, st), max_slots=4)
    assert c.state_layer("s", 0).shape == (5, 3, 4)  # four slots and the scratch slot of padding rows
    a = c.alloc()
    c.state_layer("s", 1)[a] += 7.0
    c.free(a)
    b = c.alloc()
    assert b == a and float(c.state_layer("s", 1)[b].abs().sum()) == 0.0
    assert c.paged_groups() == ["kv"]


def test_state_can_be_copied_out_and_put_back():
    """A sequence's fixed-size state as a snapshot: put back into the same slot it undoes what came after, put
    into another slot that one goes on from there; slots that are not allocated and snapshots of another shape
    are refused."""
    st = CacheGroupSpec("s", CACHE_STATE, num_layers=2, state_shape=(3,))
    c = _cache(256, groups=(KV, st), max_slots=4)
    a, b = c.alloc(), c.alloc()
    c.state_layer("s", 0)[a] += 1.0
    c.state_layer("s", 1)[a] += 2.0
    snap = c.snapshot_state(a)
    assert set(snap) == {"s"} and snap["s"].shape == (2, 3)
    c.state_layer("s", 1)[a] += 5.0
    assert float(snap["s"][1, 0]) == 2.0  # a copy, not a view
    c.restore_state(a, snap)
    assert c.state_layer("s", 1)[a].tolist() == [2.0, 2.0, 2.0]
    c.restore_state(b, snap)
    assert c.state_layer("s", 0)[b].tolist() == [1.0, 1.0, 1.0]
    with pytest.raises(CacheError):
        c.snapshot_state(3)
    with pytest.raises(CacheError):
        c.restore_state(b, {"s": snap["s"][:, :2]})
    with pytest.raises(CacheError):
        c.restore_state(b, {})


def test_random_traffic_keeps_the_books_straight():
    rng = random.Random(0)
    c = _cache(64 * 40, max_slots=12)
    live = {}
    for it in range(2000):
        op = rng.random()
        if op < 0.3 and c.free_slots():
            live[c.alloc()] = 0
        elif op < 0.5 and live:
            s = rng.choice(list(live)); c.free(s); del live[s]
        elif live:
            group = rng.sample(list(live), rng.randint(1, min(4, len(live))))
            new = [rng.randint(1, 90) for _ in group]
            try:
                c.reserve(group, new)
            except CacheFull:
                continue
            c.commit(group, new)
            for s, n in zip(group, new):
                live[s] += n
        c.check_consistent()
        assert sorted(live) == c.live_slots()
        assert all(c.length(s) == n for s, n in live.items())
        held = sum(len(c.page_list("kv", s)) for s in live)
        assert held + c.free_pages() == c.num_pages
    for s in list(live):
        c.free(s)
    assert c.free_pages() == c.num_pages and c.free_slots() == 12


def test_plan_step_lays_tokens_end_to_end():
    c = _cache(512)
    a, b = c.alloc(), c.alloc()
    c.reserve([b], [70]); c.commit([b], [70])
    p = plan_step(c, [a, b], [[5, 6, 7], [9]], [[0, 2], [0]], vocab_size=10)
    assert p.token_ids.tolist() == [5, 6, 7, 9] and p.token_seq.tolist() == [0, 0, 0, 1]
    assert p.token_pos.tolist() == [0, 1, 2, 70] and p.cu_tokens.tolist() == [0, 3, 4]
    assert p.logit_rows.tolist() == [0, 2, 3] and p.starts == [0, 70] and not p.is_decode and p.max_len == 71
    assert p.block_tables["kv"].shape == (2, 2) and p.block_tables["kv"][1].tolist() == c.page_list("kv", b)
    assert plan_step(c, [a], [[1]], "last", 10).is_decode
    for args, match in ((([a], [[10]], "last"), "outside the vocabulary"), (([a], [[]], "last"), "no tokens"),
                        (([], [], "last"), "at least one"), (([a], [[1]], [[1]]), "place 1"),
                        (([a, b], [[1]], "last"), "token lists"), (([a], [[1]], "first"), "want must be")):
        with pytest.raises(StepError, match=match):
            plan_step(c, *args, vocab_size=10)


def test_a_window_group_gives_back_the_pages_behind_its_window():
    """A group that keeps the last 100 positions holds two or three pages per sequence however long it grows;
    the full group beside it keeps them all.  Holes in the page list are never below the first page the
    next token reads."""
    c = _cache(64 * 16, groups=(KV, CacheGroupSpec("near", CACHE_WINDOW, 1, 1, 16, window=100)), max_slots=2)
    s = c.alloc()
    c.reserve([s], [300]); c.commit([s], [300])  # a long prompt needs all its pages while it runs
    assert c.page_list("near", s) == [0, 1, 2, 3, 4] and c.page_list("kv", s) == [0, 1, 2, 3, 4]
    c.reserve([s], [1])  # the token at 300 sees 201..300: pages 0, 1, 2 (positions 0..191) are behind it
    assert c.page_list("near", s) == [-1, -1, -1, 3, 4] and c.free_pages("near") == 14 and c.free_pages("kv") == 11
    c.commit([s], [1]); c.check_consistent()
    for _ in range(400):
        c.reserve([s], [1]); c.commit([s], [1])
    c.check_consistent()
    held = [p for p in c.page_list("near", s) if p >= 0]
    assert 2 <= len(held) <= 3 and len(c.page_list("kv", s)) == 11 and c.free_pages("kv") == 5
    assert c.page_list("near", s)[-1] >= 0 and c.length(s) == 701
    t = c.alloc()  # pages that came back are handed out again, lowest first
    c.reserve([t], [10])
    assert c.page_list("near", t) == [0]
    c.free(s); c.free(t)
    assert c.free_pages("near") == 16 and c.free_pages("kv") == 16
    c.check_consistent()
