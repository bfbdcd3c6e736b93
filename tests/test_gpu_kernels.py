"""Each kernel alone against a plain torch computation, at sizes other than the tiny models' (GPU)."""
import math
import os

import pytest
import torch
import torch.nn.functional as F

import plain_falcon as P

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]


def _ops():
    from pytorch_transformers_amd import ops
    return ops


def _rand(*shape, seed=0, dtype=torch.float32, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype).cuda()


def _tol(dtype):
    return dict(rtol=2e-5, atol=2e-5) if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("dtype", DTYPES)
def test_embed(dtype):
    ops = _ops()
    table = _rand(1000, 72, dtype=dtype)
    ids = torch.tensor([0, 999, 5, 5, 123], dtype=torch.int32).cuda()
    assert torch.equal(ops.embed(table, ids), table[ids.long()])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H", [48, 1000, 4544])
def test_layernorm(dtype, H):
    ops = _ops()
    x = _rand(7, H, dtype=dtype, scale=3.0) + 1.5
    w, b, w2, b2 = (_rand(H, seed=s) for s in (1, 2, 3, 4))
    ref = F.layer_norm(x.float(), (H,), w, b, 1e-5)
    torch.testing.assert_close(ops.layernorm(x, w, b, 1e-5).float(), ref, **_tol(dtype))
    o1, o2 = ops.layernorm(x, w, b, 1e-3, w2=w2, b2=b2)
    torch.testing.assert_close(o1.float(), F.layer_norm(x.float(), (H,), w, b, 1e-3), **_tol(dtype))
    torch.testing.assert_close(o2.float(), F.layer_norm(x.float(), (H,), w2, b2, 1e-3), **_tol(dtype))
    rows = torch.tensor([6, 0, 3], dtype=torch.int32).cuda()
    torch.testing.assert_close(ops.layernorm(x, w, b, 1e-5, rows=rows).float(), ref[rows.long()], **_tol(dtype))
    # a row's result does not depend on the rows around it
    assert torch.equal(ops.layernorm(x[2:3].contiguous(), w, b, 1e-5), ops.layernorm(x, w, b, 1e-5)[2:3])


@pytest.mark.parametrize("dtype", DTYPES)
def test_epilogue(dtype):
    ops = _ops()
    y, a1, a2 = (_rand(5, 130, seed=s, dtype=dtype) for s in (0, 1, 2))
    bias = _rand(130, seed=3)
    rnd = (lambda t: t) if dtype == torch.float32 else (lambda t: t.bfloat16().float())
    want = F.gelu(rnd(y.float() + bias)) + a1.float() + a2.float()
    got = ops.epilogue_(y.clone(), bias, "gelu", a1, a2)
    torch.testing.assert_close(got.float(), want, **_tol(dtype))
    torch.testing.assert_close(ops.epilogue_(y.clone(), None, None, a1, None).float(), y.float() + a1.float(), **_tol(dtype))


@pytest.mark.parametrize("M,N,K", [(1, 16, 8), (5, 100, 33), (64, 64, 16), (130, 257, 129), (17, 4544, 300)])
def test_gemm_f32(M, N, K):
    ops = _ops()
    a, w, bias, a1, a2 = _rand(M, K), _rand(N, K, seed=1), _rand(N, seed=2), _rand(M, N, seed=3), _rand(M, N, seed=4)
    want = (a.double() @ w.double().T)
    torch.testing.assert_close(ops.gemm_f32(a, w).double(), want, rtol=1e-5, atol=1e-5 * math.sqrt(K))
    full = F.gelu(want + bias.double()) + a1.double() + a2.double()
    torch.testing.assert_close(ops.gemm_f32(a, w, bias, "gelu", a1, a2).double(), full, rtol=1e-5, atol=1e-5 * math.sqrt(K))
    # bitwise the same for a row alone and in the batch
    r = M // 2
    assert torch.equal(ops.gemm_f32(a[r:r + 1].contiguous(), w, bias), ops.gemm_f32(a, w, bias)[r:r + 1])


@pytest.mark.parametrize("M", [1, 3, 8, 16, 17, 32, 33, 48, 49, 64])
@pytest.mark.parametrize("N,K", [(16, 64), (100, 200), (4544, 4544), (250, 18176 // 4)])
def test_gemm_skinny_bf16(M, N, K):
    ops = _ops()
    x = _rand(M, K, dtype=torch.bfloat16)
    w = _rand(N, K, seed=1, dtype=torch.bfloat16, scale=0.05)
    bias, a1, a2 = _rand(N, seed=2), _rand(M, N, seed=3, dtype=torch.bfloat16), _rand(M, N, seed=4, dtype=torch.bfloat16)
    prod = x.double() @ w.double().T
    scale = float(prod.abs().max())
    got32 = ops.gemm_skinny_bf16(x, w, out_f32=True)
    assert float((got32.double() - prod).abs().max()) <= 2e-5 * scale + 1e-6, "32-bit output: only accumulation error"
    got = ops.gemm_skinny_bf16(x, w, bias, "gelu", a1, a2)
    want = F.gelu((prod.float().bfloat16().float() + bias).bfloat16().float()) + a1.float() + a2.float()
    torch.testing.assert_close(got.float(), want, rtol=2e-2, atol=2e-2 * max(1.0, scale))
    assert ops.gemm_skinny_ok(x, w) == (M <= 16)  # where it is also the faster choice
    # a row alone gives the same bits as in the batch
    r = M - 1
    alone = ops.gemm_skinny_bf16(x[r:r + 1].contiguous(), w, out_f32=True)
    assert torch.equal(alone, got32[r:r + 1])


@pytest.mark.parametrize("M", [1, 9, 17, 32, 33, 50, 64, 65, 81, 96, 100, 128, 129, 200, 256])
@pytest.mark.parametrize("N,K,parts,rt,sb,depth", [(16, 64, 0, 0, 0, 0), (100, 200, 0, 0, 0, 0), (100, 200, 3, 2, 2, 2),
                                                   (4544, 4544, 0, 0, 0, 0), (250, 18176 // 4, 5, 1, 2, 4),
                                                   (1000, 1096, 1, 2, 2, 4), (333, 2056, 4, 1, 2, 2)])
def test_gemm_splitk_bf16(M, N, K, parts, rt, sb, depth):
    """The batch product with x shared through LDS: every row tile count, stage depth and split of K."""
    ops = _ops()
    x = _rand(M, K, dtype=torch.bfloat16)
    w = _rand(N, K, seed=1, dtype=torch.bfloat16, scale=0.05)
    bias, a1, a2 = _rand(N, seed=2), _rand(M, N, seed=3, dtype=torch.bfloat16), _rand(M, N, seed=4, dtype=torch.bfloat16)
    prod = x.double() @ w.double().T
    scale = float(prod.abs().max())
    kw = dict(parts=parts, rt=rt, stage_blocks=sb, depth=depth)
    got32 = ops.gemm_splitk_bf16(x, w, out_f32=True, **kw)
    assert float((got32.double() - prod).abs().max()) <= 2e-5 * scale + 1e-6, "32-bit output: only accumulation error"
    got = ops.gemm_splitk_bf16(x, w, bias, "gelu", a1, a2, **kw)
    want = F.gelu((prod.float().bfloat16().float() + bias).bfloat16().float()) + a1.float() + a2.float()
    torch.testing.assert_close(got.float(), want, rtol=2e-2, atol=2e-2 * max(1.0, scale))
    # a row alone gives the same bits as in the batch: the split of K does not depend on M
    r = M - 1
    alone = ops.gemm_splitk_bf16(x[r:r + 1].contiguous(), w, out_f32=True, **kw)
    assert torch.equal(alone, got32[r:r + 1])


@pytest.mark.parametrize("H", [64, 200, 4544, 8192])
@pytest.mark.parametrize("case", ["plain", "two products", "product and tensors", "rows", "sum only"])
def test_layernorm_sum(H, case):
    """The fused residual sum and LayerNorm against the same steps one by one in 32-bit."""
    ops = _ops()
    M = 5
    bf = lambda t: t.bfloat16()
    pa, pb = _rand(3, M, H, seed=1), _rand(2, M, H, seed=2)
    ba = _rand(H, seed=3)
    x1, x2 = bf(_rand(M, H, seed=4)), bf(_rand(M, H, seed=5))
    w, b, w2, b2 = _rand(H, seed=6) + 1.0, _rand(H, seed=7), _rand(H, seed=8) + 1.0, _rand(H, seed=9)
    value = lambda p, bias: (bf(bf(p.sum(0)).float() + bias).float() if bias is not None else bf(p.sum(0)).float())
    rows = None
    if case == "plain":
        terms, want = [x1], x1.float()
    elif case == "two products":
        terms, want = [(pb, None), (pa, ba), x1], value(pb, None) + value(pa, ba) + x1.float()
    elif case == "product and tensors":
        terms, want = [(pa, ba), x1, x2], value(pa, ba) + x1.float() + x2.float()
    elif case == "rows":
        rows = torch.tensor([4, 0, 4], dtype=torch.int32).cuda()
        terms, want = [(pb, None), x2], (value(pb, None) + x2.float())[rows.long()]
    else:
        terms, want = [(pb, None), x1, x2], value(pb, None) + x1.float() + x2.float()
    want = bf(want)
    if case == "sum only":
        x, o1, o2 = ops.layernorm_sum(terms, H)
        assert o1 is None and o2 is None
        assert torch.equal(x, want)
        return
    x, o1, o2 = ops.layernorm_sum(terms, H, w=w, b=b, eps=1e-5, w2=w2, b2=b2, rows=rows)
    assert torch.equal(x, want), "the sum is formed in the stated order and rounded once"
    for o, (ww, bb) in ((o1, (w, b)), (o2, (w2, b2))):
        ref = F.layer_norm(want.float(), (H,), ww, bb, 1e-5)
        torch.testing.assert_close(o.float(), ref, rtol=1e-2, atol=1e-2)
    x_none, o1b, _ = ops.layernorm_sum(terms, H, w=w, b=b, eps=1e-5, rows=rows, want_x=False)
    assert x_none is None and torch.equal(o1b, o1)


@pytest.mark.parametrize("H", [200, 4544, 5120, 5128, 8192])
@pytest.mark.parametrize("Pb,Pa", [(8, 4), (9, 0), (12, 4), (13, 2), (16, 4), (16, 0), (17, 4), (3, 5)])
def test_layernorm_sum_of_many_ranges(H, Pb, Pa):
    """A decode step's sum with as many ranges of partial sums as the pair launches leave: up to 16 of the first
    product and 4 of the second with the loads in flight at once (at most twelve ranges of the first, the rest behind
    them; rows of up to 5,120 features from 9 ranges on), beyond that one after the other; the ranges are added in their order whichever kernel runs, so the sum is the
    same bits as the additions one by one."""
    ops = _ops()
    M = 6
    bf = lambda t: t.bfloat16()
    pb, pa = _rand(Pb, M, H, seed=1), (_rand(Pa, M, H, seed=2) if Pa else None)
    bb, ba = _rand(H, seed=3), _rand(H, seed=4)
    x1 = bf(_rand(M, H, seed=5))
    w, b = _rand(H, seed=6) + 1.0, _rand(H, seed=7)

    def value(p, bias):
        acc = p[0].clone()
        for u in range(1, p.shape[0]):
            acc = acc + p[u]
        return bf(bf(acc).float() + bias).float()

    terms = [(pb, bb)] + ([(pa, ba)] if Pa else []) + [x1]
    want = bf(value(pb, bb) + (value(pa, ba) if Pa else 0.0) + x1.float())
    x, o1, _ = ops.layernorm_sum(terms, H, w=w, b=b, eps=1e-5)
    assert torch.equal(x, want), "the ranges are added in their order and the sum is rounded once"
    torch.testing.assert_close(o1.float(), F.layer_norm(want.float(), (H,), w, b, 1e-5), rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("H", [64, 200, 4544, 5000, 8192])
@pytest.mark.parametrize("M", [512, 515, 1031])
def test_layernorm_sum_of_many_rows(H, M):
    """From 512 rows on a wave takes a row (the arrangement for prompts): one or two tensors, with and without
    the sum as an output, one or two norms; rows beyond a multiple of four and widths that leave lanes idle."""
    ops = _ops()
    x1, x2 = _rand(M, H, seed=4, dtype=torch.bfloat16), _rand(M, H, seed=5, dtype=torch.bfloat16)
    w, b, w2, b2 = _rand(H, seed=6) + 1.0, _rand(H, seed=7), _rand(H, seed=8) + 1.0, _rand(H, seed=9)
    x3 = _rand(M, H, seed=11, dtype=torch.bfloat16)
    for terms, want in (([x1], x1), ([x1, x2], (x1.float() + x2.float()).bfloat16()),
                        ([x1, x2, x3], (x1.float() + x2.float() + x3.float()).bfloat16())):
        x, o1, o2 = ops.layernorm_sum(terms, H, w=w, b=b, eps=1e-5, w2=w2, b2=b2)
        assert torch.equal(x, want)
        for o, (ww, bb) in ((o1, (w, b)), (o2, (w2, b2))):
            torch.testing.assert_close(o.float(), F.layer_norm(want.float(), (H,), ww, bb, 1e-5), rtol=1e-2, atol=1e-2)
        x_none, o1b, o2b = ops.layernorm_sum(terms, H, w=w, b=b, eps=1e-5, want_x=False)
        assert x_none is None and o2b is None and torch.equal(o1b, o1)
        few = ops.layernorm_sum([t[:7] for t in terms], H, w=w, b=b, eps=1e-5)[1]  # a workgroup per row
        torch.testing.assert_close(o1[:7].float(), few.float(), rtol=1e-2, atol=1e-2)
    assert torch.equal(ops.layernorm_sum([x1, x2], H)[0], (x1.float() + x2.float()).bfloat16())
    assert M >= ops.layernorm_sum_rows_min()
    # three tensors are the sum that a product's epilogue with two additions stores; chosen rows of it (a workgroup per row)
    y = x1.clone()
    ops.epilogue_(y, None, None, x2, x3)
    assert torch.equal(ops.layernorm_sum([x1, x2, x3], H)[0], y)
    rows = torch.tensor([M - 1, 0, 5], dtype=torch.int32).cuda()
    picked = ops.layernorm_sum([x1, x2, x3], H, w=w, b=b, eps=1e-5, rows=rows)
    assert torch.equal(picked[0], y[rows.long()])
    torch.testing.assert_close(picked[1].float(), F.layer_norm(y[rows.long()].float(), (H,), w, b, 1e-5), rtol=1e-2, atol=1e-2)


def test_layernorm_sum_refuses_what_it_cannot_do():
    ops = _ops()
    assert not ops.layernorm_sum_ok(100) and not ops.layernorm_sum_ok(8200) and ops.layernorm_sum_ok(8192)
    x = _rand(2, 100, dtype=torch.bfloat16)
    with pytest.raises(ops.KernelError, match="multiple of 8"):
        ops.layernorm_sum([x], 100)
    x = _rand(2, 64, dtype=torch.bfloat16)
    with pytest.raises(ops.KernelError, match="products must come before"):
        ops.layernorm_sum([x, (_rand(1, 2, 64), None)], 64)


def test_partial_product_equals_the_reduced_one():
    """Partial sums added by the norm kernel give the bits the product's own reduction stores."""
    ops = _ops()
    M, N, K = 9, 328, 2056
    x, w = _rand(M, K, dtype=torch.bfloat16), _rand(N, K, seed=1, dtype=torch.bfloat16, scale=0.05)
    bias, a1 = _rand(N, seed=2), _rand(M, N, seed=3, dtype=torch.bfloat16)
    whole = ops.gemm_splitk_bf16(x, w, bias, None, a1)
    part = ops.gemm_splitk_partial(x, w)
    assert part.shape[0] > 1 and part.shape[1:] == (M, N)
    assert ops.gemm_partial_ok(x, w)  # K is long against N
    formed = ops.layernorm_sum([(part, bias), a1], N)[0]
    assert torch.equal(formed, whole)


def test_gemm_skinny_pair():
    """Two products of one launch equal the products on their own up to summation order."""
    ops = _ops()
    M, K, N1, N2 = 7, 328, 100, 530
    x1, x2 = _rand(M, K, dtype=torch.bfloat16), _rand(M, K, seed=5, dtype=torch.bfloat16)
    w1, w2 = _rand(N1, K, seed=1, dtype=torch.bfloat16, scale=0.05), _rand(N2, K, seed=2, dtype=torch.bfloat16, scale=0.05)
    b2 = _rand(N2, seed=3)
    y1, y2 = ops.gemm_skinny_pair_bf16(x1, w1, x2, w2, None, None, b2, "gelu")
    torch.testing.assert_close(y1.float(), ops.gemm_skinny_bf16(x1, w1).float(), rtol=2e-2, atol=2e-2)
    torch.testing.assert_close(y2.float(), ops.gemm_skinny_bf16(x2, w2, b2, "gelu").float(), rtol=2e-2, atol=2e-2)
    want1 = (x1.double() @ w1.double().T).float()
    torch.testing.assert_close(y1.float(), want1, rtol=2e-2, atol=2e-2 * float(want1.abs().max()))
    # a row alone gives the same bits as in the batch
    a1, a2 = ops.gemm_skinny_pair_bf16(x1[3:4].contiguous(), w1, x2[3:4].contiguous(), w2, None, None, b2, "gelu")
    assert torch.equal(a1, y1[3:4]) and torch.equal(a2, y2[3:4])
    with pytest.raises(ops.KernelError, match="shares M and K"):
        ops.gemm_skinny_pair_bf16(x1, w1, x2[:3].contiguous(), w2)


def test_pair_ranges_are_timed_once_per_shape_and_kept():
    """The ranges of K of a pair: the rule's choice or a timed neighbour of it, the same for every later launch of
    the shape (so the workspace that is asked for fits, and a row alone has the bits it has in the batch), reported
    by gemm_splitk_pair_parts; counts that the kernel does not take are refused; 0, 0 returns to the rule."""
    ops = _ops()
    lib = ops.load_library()
    M, K1, K2, N1, N2 = 48, 2112, 4608, 320, 192
    x1, x2 = _rand(M, K1, dtype=torch.bfloat16), _rand(M, K2, seed=5, dtype=torch.bfloat16)
    w1, w2 = _rand(N1, K1, seed=1, dtype=torch.bfloat16, scale=0.05), _rand(N2, K2, seed=2, dtype=torch.bfloat16, scale=0.05)
    rule = ops.gemm_splitk_pair_parts(N1, K1, N2, K2)
    key = ((N1, K1), (N2, K2))
    ops.gemm_splitk_pair_bf16(x1, w1, x2, w2)
    assert ops.TUNE_LIVE or key not in ops.active().pair_parts, "a launch times nothing unless timing is switched on"
    with ops.live_tuning():
        y1, y2 = ops.gemm_splitk_pair_bf16(x1, w1, x2, w2)
    ops.release_flush()
    if ops.PAIR_TUNE:
        kept = ops.active().pair_parts[key]  # ranges, ranges, row tiles per wave
        assert kept[2] in (1, 2) and 1 <= kept[0] <= 2 * rule[0] + 1 and 1 <= kept[1] <= 2 * rule[1] + 1
        assert ops.gemm_splitk_pair_parts(N1, K1, N2, K2) == kept[:2]
    p1, p2 = ops.gemm_splitk_pair_parts(N1, K1, N2, K2)
    # (what follows is about the kernel that walks K in stages: where the timing has kept the launch with stationary
    # activations for some class of rows, which has ranges of its own, that is set aside)
    for cls in range(len(ops.STATIONARY_CLASS_ROWS)):
        assert lib.pta_gemm_splitk_pair_fix_stationary(N1, K1, N2, K2, cls, 0, 0) == 0
    y1, y2 = ops.gemm_splitk_pair_bf16(x1, w1, x2, w2)
    assert torch.equal(y1, ops.gemm_splitk_bf16(x1, w1, rt=1, parts=p1)) and torch.equal(y2, ops.gemm_splitk_bf16(x2, w2, rt=1, parts=p2))
    for y, x, w in ((y1, x1, w1), (y2, x2, w2)):
        want = (x.double() @ w.double().T).float()
        torch.testing.assert_close(y.float(), want, rtol=2e-2, atol=2e-2 * float(want.abs().max()))
    a1, a2 = ops.gemm_splitk_pair_bf16(x1[20:37].contiguous(), w1, x2[20:37].contiguous(), w2)
    assert torch.equal(a1, y1[20:37]) and torch.equal(a2, y2[20:37])
    assert lib.pta_gemm_splitk_pair_fix_parts(N1, K1, N2, K2, 5, 2) == 1, "2,112 elements are no five ranges of 512 and more"
    assert lib.pta_gemm_splitk_pair_fix_parts(N1, K1, N2, K2, 1, 17) == 1
    try:
        assert lib.pta_gemm_splitk_pair_fix_parts(N1, K1, N2, K2, 1, 3) == 0
        assert ops.gemm_splitk_pair_parts(N1, K1, N2, K2) == (1, 3)
        z1, z2 = ops.gemm_splitk_pair_bf16(x1, w1, x2, w2)
        assert torch.equal(z1, ops.gemm_splitk_bf16(x1, w1, rt=1, parts=1)) and torch.equal(z2, ops.gemm_splitk_bf16(x2, w2, rt=1, parts=3))
        # workgroups of 128 rows of W instead of 64: other workgroups, the same ranges, the same bits
        assert lib.pta_gemm_splitk_pair_fix(N1, K1, N2, K2, 1, 3, 2) == 0
        t1, t2 = ops.gemm_splitk_pair_bf16(x1, w1, x2, w2)
        assert torch.equal(t1, z1) and torch.equal(t2, z2)
        assert lib.pta_gemm_splitk_pair_fix(N1, K1, N2, K2, 1, 3, 3) == 1
    finally:
        assert lib.pta_gemm_splitk_pair_fix_parts(N1, K1, N2, K2, 0, 0) == 0
        assert lib.pta_gemm_splitk_pair_fix_stationary(N1, K1, N2, K2, -1, 0, 0) == 0
        ops.active().pair_parts.pop(key, None)
        ops.active().pair_stationary.pop(key, None)
    assert ops.gemm_splitk_pair_parts(N1, K1, N2, K2) == rule


@pytest.mark.parametrize("M", [1, 8, 16, 17, 32, 33, 47, 48, 49, 64, 65, 96, 100, 128])
@pytest.mark.parametrize("shapes,parts", [(((1000, 520), (344, 1096)), (1, 1)), (((1000, 520), (344, 1096)), (2, 3)),
                                          (((40, 72), (1608, 2304)), (1, 2)), (((4672, 4544), (512, 8192)), (1, 2)),
                                          (((24, 8), (16, 4104)), (1, 16)), (((1000, 4608), (40, 1152)), (1, 1)),
                                          (((200, 1536), (48, 2304)), (1, 1)), (((4672, 4544), (4544, 4544)), (3, 3))])
def test_gemm_stationary_pair(M, shapes, parts):
    """The pair launch with stationary activations, called on its own: every count of sixteen-row tiles of x, K
    that ends inside a block, a phase and a 32-element step, N that ends inside a tile, more row tiles than the
    compute units have waves for, ranges of K that are dropped because they would be empty; against the products
    in 64-bit, and partial sums that nothing has to zero first."""
    import ctypes

    ops = _ops()
    lib = ops.load_library()
    (N1, K1), (N2, K2) = shapes
    x1, x2 = _rand(M, K1, dtype=torch.bfloat16), _rand(M, K2, seed=5, dtype=torch.bfloat16)
    w1, w2 = _rand(N1, K1, seed=1, dtype=torch.bfloat16, scale=0.05), _rand(N2, K2, seed=2, dtype=torch.bfloat16, scale=0.05)
    kept = lambda K, p: -(-((K + 63) // 64) // -(-((K + 63) // 64) // p))
    part1 = torch.full((kept(K1, parts[0]), M, N1), float("nan")).cuda()
    part2 = torch.full((kept(K2, parts[1]), M, N2), float("nan")).cuda()
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    rc = lib.pta_gemm_stationary_pair_bf16(P(part1), P(x1), P(w1), N1, K1, parts[0], P(part2), P(x2), P(w2), N2, K2, parts[1],
                                           M, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == 0, lib.pta_last_error().decode()
    for part, x, w in ((part1, x1, w1), (part2, x2, w2)):
        want = x.double() @ w.double().T
        got = part.double().sum(0)
        assert torch.isfinite(part).all(), "a partial sum was left unwritten"
        assert float((got - want).abs().max()) <= 2e-5 * float(want.abs().max()) + 1e-6


def test_gemm_stationary_pair_refusals_and_dispatch():
    """Rows beyond 128 are refused with a message; a pair launch of up to 128 rows runs with stationary activations
    and the ranges the library reports for the class of its rows; a class can be fixed to other ranges or to the
    staged kernel per shape, and forgotten; partial sums add up to the product either way."""
    import ctypes

    ops = _ops()
    lib = ops.load_library()
    N1, K1, N2, K2 = 328, 2112, 200, 4608
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    stream = lambda: ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    w1, w2 = _rand(N1, K1, seed=1, dtype=torch.bfloat16, scale=0.05), _rand(N2, K2, seed=2, dtype=torch.bfloat16, scale=0.05)
    for M in (0, 129):
        x1, x2 = _rand(max(M, 1), K1, dtype=torch.bfloat16), _rand(max(M, 1), K2, seed=5, dtype=torch.bfloat16)
        part = torch.empty(4, max(M, 1), 328).cuda()
        assert lib.pta_gemm_stationary_pair_bf16(P(part), P(x1), P(w1), N1, K1, 1, P(part), P(x2), P(w2), N2, K2, 1, M, stream()) != 0
        assert "1 to 128 rows" in lib.pta_last_error().decode()
    staged = ops.gemm_splitk_pair_parts(N1, K1, N2, K2)
    rules = [ops.gemm_stationary_rule(N1, K1, N2, K2, cls) for cls in range(4)]
    assert all(q1 >= 1 and q2 >= q1 for q1, q2 in rules), rules  # the longer K has at least as many ranges
    for cls, top in enumerate(ops.STATIONARY_CLASS_ROWS):  # without a fixed choice: from 33 rows on
        assert ops.gemm_splitk_pair_parts(N1, K1, N2, K2, top) == (rules[cls] if cls >= 2 else staged)
    assert ops.gemm_splitk_pair_parts(N1, K1, N2, K2, 129) == staged

    def check(M):
        x1, x2 = _rand(M, K1, dtype=torch.bfloat16), _rand(M, K2, seed=5, dtype=torch.bfloat16)
        a, b = ops.gemm_splitk_pair_partial(x1, w1, x2, w2)
        assert (a.shape[0], b.shape[0]) == ops.gemm_splitk_pair_parts(N1, K1, N2, K2, M)
        for part, x, w in ((a, x1, w1), (b, x2, w2)):
            want = x.double() @ w.double().T
            assert float((part.double().sum(0) - want).abs().max()) <= 2e-5 * float(want.abs().max())

    for M in (1, 8, 16, 17, 48, 64, 100, 128, 129):
        check(M)
    fix = lib.pta_gemm_splitk_pair_fix_stationary
    try:
        assert fix(N1, K1, N2, K2, 1, 2, 4) == 0
        assert ops.gemm_splitk_pair_parts(N1, K1, N2, K2, 20) == (2, 4) and ops.gemm_splitk_pair_parts(N1, K1, N2, K2, 16) == staged
        assert fix(N1, K1, N2, K2, 0, 1, 1) == 0 and ops.gemm_splitk_pair_parts(N1, K1, N2, K2, 8) == (1, 1)
        assert fix(N1, K1, N2, K2, 2, 0, 0) == 0
        assert ops.gemm_splitk_pair_parts(N1, K1, N2, K2, 64) == staged and ops.gemm_splitk_pair_parts(N1, K1, N2, K2, 65) == rules[3]
        for M in (8, 20, 64):
            check(M)
        assert fix(N1, K1, N2, K2, 4, 1, 1) != 0 and fix(N1, K1, N2, K2, 1, 0, 1) != 0 and fix(N1, K1, N2, K2, 1, 17, 1) != 0
    finally:
        fix(N1, K1, N2, K2, -1, 0, 0)
    assert ops.gemm_splitk_pair_parts(N1, K1, N2, K2, 64) == rules[2]


def test_gemm_splitk_pair():
    """Two products of one launch, run to the end, against the products on their own."""
    ops = _ops()
    M, K1, K2, N1, N2 = 100, 328, 264, 100, 530
    x1, x2 = _rand(M, K1, dtype=torch.bfloat16), _rand(M, K2, seed=5, dtype=torch.bfloat16)
    w1, w2 = _rand(N1, K1, seed=1, dtype=torch.bfloat16, scale=0.05), _rand(N2, K2, seed=2, dtype=torch.bfloat16, scale=0.05)
    b2 = _rand(N2, seed=3)
    y1, y2 = ops.gemm_splitk_pair_bf16(x1, w1, x2, w2, None, None, b2, "gelu")
    p1, p2 = ops.gemm_splitk_pair_parts(N1, K1, N2, K2)
    assert torch.equal(y1, ops.gemm_splitk_bf16(x1, w1, rt=1, parts=p1)), "the same ranges in the same order: the same bits"
    assert torch.equal(y2, ops.gemm_splitk_bf16(x2, w2, b2, "gelu", rt=1, parts=p2))
    a1, a2 = ops.gemm_splitk_pair_bf16(x1[17:37].contiguous(), w1, x2[17:37].contiguous(), w2, None, None, b2, "gelu")
    assert torch.equal(a1, y1[17:37]) and torch.equal(a2, y2[17:37])


def test_every_activation_in_every_epilogue():
    """The reference's activations by name, in the epilogue of each product kernel and of the library's product,
    in both types, against the plain table (values out to where relu6 and gelu_10 clip and softplus is linear)."""
    ops = _ops()
    M, N, K = 24, 72, 64
    x = (torch.eye(K)[:M] * 1.0).cuda()  # row m picks column m of W: the product is W's own values
    grid = torch.linspace(-30.0, 30.0, M * N).reshape(N, M).T.contiguous()  # pre-activations, spread over the rows
    w = torch.zeros(N, K)
    w[:, :M] = grid.T
    for name in sorted(k for k in ops.ACT_CODES if k and k != "none"):
        want = P.activation(grid.double(), name)
        got32 = ops.gemm_f32(x, w.cuda(), None, name)
        torch.testing.assert_close(got32.double().cpu(), want, rtol=2e-6, atol=2e-6, msg=lambda m: f"{name} float32: {m}")
        xb, wb = x.bfloat16(), w.bfloat16().cuda()
        wantb = P.activation(w.bfloat16().double().T[:M], name)
        for what, got in (("few rows", ops.gemm_skinny_bf16(xb[:9].contiguous(), wb, None, name)),
                          ("batch", ops.gemm_splitk_bf16(xb, wb, None, name)),
                          ("epilogue", ops.epilogue_(torch.mm(xb, wb.t()), None, name))):
            rows = got.shape[0]
            torch.testing.assert_close(got.double().cpu(), wantb[:rows], rtol=1e-2, atol=1e-2,
                                       msg=lambda m: f"{name} bfloat16 {what}: {m}")


def test_library_mm_in_pieces():
    """The vendor library's product cut along M: forced here by made-up timings, since what is faster is the
    machine's business; the pieces cover every row once and the result is the library's."""
    ops = _ops()
    N, K = 136, 264
    w = _rand(N, K, seed=1, dtype=torch.bfloat16, scale=0.05)
    ops.active().mm_times[(N, K)] = {256: 1.0, 512: 50.0, 1000: 1e6, 1030: 1e6}  # pieces of 256 look cheapest
    try:
        for M in (1000, 1030, 700):
            x = _rand(M, K, seed=M, dtype=torch.bfloat16)
            ops.library_mm(x, w)
            assert ops.TUNE_LIVE or (N, K, (M + 63) // 64) not in ops.active().mm_plans, "no plan is made unless timing is on"
            with ops.live_tuning():
                y = ops.library_mm(x, w)
            plan = ops.active().mm_plans[(N, K, (M + 63) // 64)]
            if M != 700:
                assert len(plan) > 1 and sum(plan) == M and all(p >= 256 for p in plan), plan
            torch.testing.assert_close(y.float(), torch.mm(x, w.t()).float(), rtol=2e-2, atol=2e-2)
        # another row count of the same bucket reuses the plan, its last piece adjusted
        x = _rand(1001, K, seed=7, dtype=torch.bfloat16)
        torch.testing.assert_close(ops.library_mm(x, w).float(), torch.mm(x, w.t()).float(), rtol=2e-2, atol=2e-2)
    finally:
        ops.active().mm_times.pop((N, K), None)
        for key in [k for k in ops.active().mm_plans if k[:2] == (N, K)]:
            ops.active().mm_plans.pop(key)


def test_gemm_skinny_refuses_what_it_cannot_do():
    ops = _ops()
    x, w = _rand(257, 64, dtype=torch.bfloat16), _rand(32, 64, dtype=torch.bfloat16)
    assert not ops.gemm_skinny_ok(x, w) and not ops.gemm_splitk_ok(x, w)
    assert ops.gemm_splitk_ok(x[:17].contiguous(), w) and not ops.gemm_splitk_ok(x[:16].contiguous(), w)
    assert ops.gemm_splitk_ok(x[:min(ops.SPLITK_SURE_ROWS, ops.SPLITK_MAX_ROWS)].contiguous(), w)  # beyond that rows by a timing
    with pytest.raises(ops.KernelError, match="at most 256 rows"):
        ops.gemm_splitk_bf16(x, w)
    with pytest.raises(ops.KernelError, match="at most 64 rows"):
        ops.gemm_skinny_bf16(x[:65].contiguous(), w)
    x, w = _rand(4, 60, dtype=torch.bfloat16), _rand(32, 60, dtype=torch.bfloat16)
    assert not ops.gemm_skinny_ok(x, w)
    with pytest.raises(ops.KernelError, match="multiple of 8"):
        ops.gemm_skinny_bf16(x, w)
    with pytest.raises(ops.KernelError, match="no CPU fallback"):
        ops.gemm_skinny_bf16(x.cpu(), w.cpu())


# --- rotation, head split, cache write, attention ------------------------------------------------------
def _cache_setup(n_seqs, lens, nkv, d, dtype, n_pages=64, seed=0):
    """Scattered pages for every sequence; returns pools, block table and the page lists."""
    g = torch.Generator().manual_seed(seed)
    perm = torch.randperm(n_pages, generator=g).tolist()
    lists, at = [], 0
    for L in lens:
        n = (L + 63) // 64
        lists.append(perm[at:at + n]); at += n
    width = max(len(l) for l in lists)
    bt = torch.zeros(n_seqs, width, dtype=torch.int32)
    for i, l in enumerate(lists):
        bt[i, :len(l)] = torch.tensor(l, dtype=torch.int32)
    # unwritten positions hold NaN: a kernel that lets them into a sum, even with weight zero, shows
    k_pool = torch.full((n_pages, nkv, 64, d), float("nan"), dtype=dtype).cuda()
    v_pool = torch.full((n_pages, nkv, d, 64), float("nan"), dtype=dtype).cuda()  # values: transposed pages
    return k_pool, v_pool, bt.cuda(), lists


def _gather(pool, pages, L, transposed=False):
    """[L, nkv, d] of a sequence from its pages."""
    x = pool[torch.tensor(pages).long().cuda()]  # [p, nkv, 64, d], or [p, nkv, d, 64] for values
    if transposed:
        x = x.transpose(2, 3)
    return x.permute(0, 2, 1, 3).reshape(-1, x.shape[1], x.shape[3])[:L]


def _freq(rotary, d, n_seqs, theta=10000.0, factor=1.0):
    """None, one frequency table, or (rotary == "per sequence") a table per sequence, all rows different."""
    if not rotary:
        return None
    inv = P.rope_inv_freq(d, theta, factor)
    if rotary == "per sequence":
        inv = torch.stack([inv / (1.0 + 0.37 * s) for s in range(n_seqs)])
    return inv.cuda()


def test_rope_dynamic_table():
    """A frequency table per sequence from the lengths after the step, against the plain formula
    (src/transformers/modeling_rope_utils.py:149-158): trained frequencies up to the trained context, stretched
    beyond it, each sequence by its own length."""
    ops = _ops()
    starts, news = [0, 40, 47, 48, 300, 5000], [48, 9, 1, 1, 7, 1]
    seq_start = torch.tensor(starts, dtype=torch.int32).cuda()
    cu = torch.tensor([0] + list(torch.tensor(news).cumsum(0)), dtype=torch.int32).cuda()
    for d, theta, factor, ctx in ((32, 10000.0, 4.0, 48), (128, 500042.0, 10.0, 48), (6, 10000.0, 2.0, 100)):
        got = ops.rope_dynamic_table(seq_start, cu, d, theta, factor, ctx).cpu()
        assert got.shape == (len(starts), d // 2)
        for i, (s, n) in enumerate(zip(starts, news)):
            want = P.rope_dynamic_inv_freq(d, theta, factor, ctx, s + n)
            # the kernel rounds the double-precision value once; the plain formula is the reference's chain of
            # 32-bit operations, each of which may be a unit or two in the last place off (2^-23 = 1.2e-7)
            torch.testing.assert_close(got[i], want, rtol=2e-6, atol=0)
            if s + n <= ctx:
                torch.testing.assert_close(got[i], P.rope_inv_freq(d, theta), rtol=5e-7, atol=0)
    with pytest.raises(ops.KernelError):
        ops.rope_dynamic_table(seq_start, cu, 2, 10000.0, 2.0, 48)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("layout,nh,nkv,d", [("grouped", 6, 2, 32), ("tail", 7, 1, 64), ("interleaved", 5, 5, 24),
                                             ("grouped", 8, 8, 16), ("grouped", 4, 1, 128)])
@pytest.mark.parametrize("rotary", [True, False, "per sequence"])
def test_qkv_rope_cache(dtype, layout, nh, nkv, d, rotary):
    """Against the plain split and rotation; keys and values land at (page, position) of their sequence."""
    ops = _ops()
    starts, news = [70, 0, 127], [3, 66, 1]
    lens = [s + n for s, n in zip(starts, news)]
    k_pool, v_pool, bt, lists = _cache_setup(3, lens, nkv, d, dtype)
    M = sum(news)
    fused = _rand(M, (nh + 2 * nkv) * d, dtype=dtype)
    bias = _rand((nh + 2 * nkv) * d, seed=9)
    token_seq = torch.tensor([i for i, n in enumerate(news) for _ in range(n)], dtype=torch.int32).cuda()
    token_pos = torch.tensor([s + j for s, n in zip(starts, news) for j in range(n)], dtype=torch.int32).cuda()
    inv = _freq(rotary, d, 3, 500042.0, 2.0)
    q = ops.qkv_rope_cache(fused, bias, inv, 1.0, token_pos, token_seq, bt, k_pool, v_pool, nh, nkv, d, layout)

    c = dict(num_attention_heads=nh, hidden_size=nh * d, num_kv_heads=nkv,
             new_decoder_architecture=layout == "grouped", multi_query=layout == "tail")
    rnd = (lambda t: t) if dtype == torch.float32 else (lambda t: t.bfloat16().double())
    x = rnd(fused.double().cpu() + bias.double().cpu())
    wq, wk, wv = P.split_heads(x, c)
    if rotary == "per sequence":  # every token by its own sequence's table
        cs = [P.rope_cos_sin(token_pos.cpu()[t:t + 1], inv.cpu()[int(token_seq[t])]) for t in range(M)]
        cos, sin = torch.cat([c for c, _ in cs]), torch.cat([s_ for _, s_ in cs])
        wq, wk = P.apply_rope(wq, cos, sin), P.apply_rope(wk, cos, sin)
    elif rotary:
        cos, sin = P.rope_cos_sin(token_pos.cpu(), inv.cpu())
        wq, wk = P.apply_rope(wq, cos, sin), P.apply_rope(wk, cos, sin)
    tol = dict(rtol=1e-5, atol=1e-5) if dtype == torch.float32 else dict(rtol=1e-2, atol=1e-2)
    torch.testing.assert_close(q.double().cpu(), wq, **tol)
    at = 0
    for i, (s, n) in enumerate(zip(starts, news)):
        gk, gv = _gather(k_pool, lists[i], lens[i]), _gather(v_pool, lists[i], lens[i], transposed=True)
        torch.testing.assert_close(gk[s:].double().cpu(), wk[at:at + n].contiguous(), **tol)
        torch.testing.assert_close(gv[s:].double().cpu(), wv[at:at + n].contiguous(), **tol)
        assert torch.isnan(gk[:s].float()).all(), "positions before the step's tokens must not be written"
        at += n
    # write_cache=False leaves the cache alone
    k2 = k_pool.clone()
    ops.qkv_rope_cache(fused * 2, bias, inv, 1.0, token_pos, token_seq, bt, k_pool, v_pool, nh, nkv, d, layout, write_cache=False)
    assert torch.equal(torch.nan_to_num(k2.float()), torch.nan_to_num(k_pool.float()))


@pytest.mark.parametrize("layout,nh,nkv,d", [("grouped", 4, 2, 32), ("grouped", 8, 2, 128), ("tail", 7, 1, 64),
                                             ("interleaved", 3, 3, 96), ("tail", 71, 1, 64)])
@pytest.mark.parametrize("rotary,bias", [(True, True), (False, False), (True, False), ("per sequence", True)])
def test_pair_launch_takes_the_fused_qkv_rows_to_their_end(layout, nh, nkv, d, rotary, bias):
    """The pair launch for few rows with the query_key_value tail in its epilogue against the same two products
    followed by the kernel that splits, rotates and writes the cache: the same queries, the same pages (bit for bit
    where K is not a multiple of 2,048, so that both walk K alike), nothing written where no token lies, and
    nothing written at all with write_cache off."""
    ops = _ops()
    if not ops.QKV_TAIL:
        pytest.skip("switched off by PTA_QKV_TAIL=0")
    K, N2 = 264, 200
    starts = [70, 0, 127, 5, 63]
    M = len(starts)
    lens = [s + 1 for s in starts]
    N1 = (nh + 2 * nkv) * d
    x = _rand(M, K, dtype=torch.bfloat16)
    w1, w2 = _rand(N1, K, seed=1, dtype=torch.bfloat16, scale=0.05), _rand(N2, K, seed=2, dtype=torch.bfloat16, scale=0.05)
    b1, b2 = (_rand(N1, seed=3) if bias else None), _rand(N2, seed=4)
    token_seq = torch.arange(M, dtype=torch.int32).cuda()
    token_pos = torch.tensor(starts, dtype=torch.int32).cuda()
    inv = _freq(rotary, d, M)
    assert ops.gemm_skinny_pair_qkv_ok(x, w1, w2, d)
    pools = []
    for fused_way in (False, True):
        k_pool, v_pool, bt, lists = _cache_setup(M, lens, nkv, d, torch.bfloat16)
        if fused_way:
            q, y2 = ops.gemm_skinny_pair_qkv(x, w1, b1, inv, 0.9, token_pos, token_seq, bt, k_pool, v_pool, nh, nkv, d,
                                             layout, True, x, w2, b2, "gelu")
        else:
            fused, y2 = ops.gemm_skinny_pair_bf16(x, w1, x, w2, None, None, b2, "gelu")
            q = ops.qkv_rope_cache(fused, b1, inv, 0.9, token_pos, token_seq, bt, k_pool, v_pool, nh, nkv, d, layout)
        pools.append((q, y2, k_pool, v_pool))
    (q0, y0, k0, v0), (q1, y1, k1, v1) = pools
    assert torch.equal(y0, y1), "the second product does not know about the first one's tail"
    assert torch.equal(q0, q1)
    same = lambda a, b: torch.equal(torch.nan_to_num(a.float(), nan=-7.0), torch.nan_to_num(b.float(), nan=-7.0))
    assert same(k0, k1) and same(v0, v1), "the same values at the same places of the pages, and nothing anywhere else"
    before = k1.clone()
    q2, _ = ops.gemm_skinny_pair_qkv(x, w1 * 2, b1, inv, 0.9, token_pos, token_seq, bt, k1, v1, nh, nkv, d, layout, False,
                                     x, w2, b2, "gelu")
    assert same(before, k1) and not torch.equal(q2, q1)


@pytest.mark.parametrize("layout,nh,nkv,d,M", [("grouped", 4, 2, 24, 40), ("grouped", 8, 2, 128, 17), ("tail", 7, 1, 64, 150),
                                               ("interleaved", 3, 3, 96, 64)])
@pytest.mark.parametrize("rotary,bias", [(True, True), (False, False), ("per sequence", False)])
def test_batch_pair_launch_takes_the_fused_qkv_rows_to_their_end(layout, nh, nkv, d, M, rotary, bias):
    """The same for a decode batch of 17 to 256 rows, where the launch that adds the partial sums carries the
    tail: the queries and pages of the two products followed by the kernel of its own, bit for bit."""
    ops = _ops()
    K1, K2, N2 = 264, 328, 200
    g = torch.Generator().manual_seed(M)
    starts = torch.randint(0, 190, (M,), generator=g).tolist()
    lens = [s + 1 for s in starts]
    N1 = (nh + 2 * nkv) * d
    x1, x2 = _rand(M, K1, dtype=torch.bfloat16), _rand(M, K2, seed=7, dtype=torch.bfloat16)
    w1, w2 = _rand(N1, K1, seed=1, dtype=torch.bfloat16, scale=0.05), _rand(N2, K2, seed=2, dtype=torch.bfloat16, scale=0.05)
    b1, b2 = (_rand(N1, seed=3) if bias else None), _rand(N2, seed=4)
    token_seq = torch.arange(M, dtype=torch.int32).cuda()
    token_pos = torch.tensor(starts, dtype=torch.int32).cuda()
    inv = _freq(rotary, d, M)
    pools = []
    for fused_way in (False, True):
        k_pool, v_pool, bt, lists = _cache_setup(M, lens, nkv, d, torch.bfloat16, n_pages=3 * M + 8)
        if fused_way:
            q, y2 = ops.gemm_splitk_pair_qkv(x1, w1, b1, inv, 1.0, token_pos, token_seq, bt, k_pool, v_pool, nh, nkv, d,
                                             layout, True, x2, w2, b2, "gelu")
        else:
            fused, y2 = ops.gemm_splitk_pair_bf16(x1, w1, x2, w2, None, None, b2, "gelu")
            q = ops.qkv_rope_cache(fused, b1, inv, 1.0, token_pos, token_seq, bt, k_pool, v_pool, nh, nkv, d, layout)
        pools.append((q, y2, k_pool, v_pool))
    (q0, y0, k0, v0), (q1, y1, k1, v1) = pools
    same = lambda a, b: torch.equal(torch.nan_to_num(a.float(), nan=-7.0), torch.nan_to_num(b.float(), nan=-7.0))
    assert torch.equal(y0, y1) and torch.equal(q0, q1)
    assert same(k0, k1) and same(v0, v1), "the same values at the same places of the pages, and nothing anywhere else"
    before = k1.clone()
    ops.gemm_splitk_pair_qkv(x1, w1 * 2, b1, inv, 1.0, token_pos, token_seq, bt, k1, v1, nh, nkv, d, layout, False, x2, w2,
                             b2, "gelu")
    assert same(before, k1)


@pytest.mark.parametrize("layout,nh,nkv,d,M,K", [("grouped", 4, 2, 24, 40, 264), ("grouped", 8, 2, 128, 17, 2560),
                                                 ("tail", 7, 1, 64, 150, 1032), ("interleaved", 3, 3, 96, 256, 4104)])
@pytest.mark.parametrize("rotary,bias", [(True, True), (False, False), ("per sequence", True)])
def test_batch_launch_takes_the_fused_qkv_rows_to_their_end(layout, nh, nkv, d, M, K, rotary, bias):
    """A query_key_value projection on its own, 17 to 256 rows, one range of K and several: the launch that adds
    the partial sums carries the tail, and gives the queries and pages of the product followed by the kernel of
    its own, bit for bit; with write_cache off the pages stay as they are."""
    ops = _ops()
    g = torch.Generator().manual_seed(M)
    starts = torch.randint(0, 190, (M,), generator=g).tolist()
    lens = [s + 1 for s in starts]
    N = (nh + 2 * nkv) * d
    x = _rand(M, K, dtype=torch.bfloat16)
    w = _rand(N, K, seed=1, dtype=torch.bfloat16, scale=0.05)
    b = _rand(N, seed=3) if bias else None
    token_seq = torch.arange(M, dtype=torch.int32).cuda()
    token_pos = torch.tensor(starts, dtype=torch.int32).cuda()
    inv = _freq(rotary, d, M)
    pools = []
    for fused_way in (False, True):
        k_pool, v_pool, bt, lists = _cache_setup(M, lens, nkv, d, torch.bfloat16, n_pages=3 * M + 8)
        if fused_way:
            q = ops.gemm_splitk_qkv(x, w, b, inv, 1.0, token_pos, token_seq, bt, k_pool, v_pool, nh, nkv, d, layout, True)
        else:
            fused = ops.gemm_splitk_bf16(x, w)
            q = ops.qkv_rope_cache(fused, b, inv, 1.0, token_pos, token_seq, bt, k_pool, v_pool, nh, nkv, d, layout)
        pools.append((q, k_pool, v_pool))
    (q0, k0, v0), (q1, k1, v1) = pools
    same = lambda a, b: torch.equal(torch.nan_to_num(a.float(), nan=-7.0), torch.nan_to_num(b.float(), nan=-7.0))
    assert torch.equal(q0, q1)
    assert same(k0, k1) and same(v0, v1), "the same values at the same places of the pages, and nothing anywhere else"
    before = k1.clone()
    q2 = ops.gemm_splitk_qkv(x, w * 2, b, inv, 1.0, token_pos, token_seq, bt, k1, v1, nh, nkv, d, layout, False)
    assert same(before, k1) and not torch.equal(q2, q1)
    with pytest.raises(ops.KernelError, match="w_qkv"):
        ops.gemm_splitk_qkv(x, w[:-8], b, inv, 1.0, token_pos, token_seq, bt, k1, v1, nh, nkv, d, layout, False)


def _rotate_plain(x, pos, inv_freq, scale, rotary_dim, pairing):
    """The rotation spelled out element by element: x [T, heads, d], the first ``rotary_dim`` elements of a head in
    pairs (i, i + rotary_dim / 2) ("half") or (2i, 2i + 1) ("interleaved"), pair i by position * inv_freq[i] (the
    angle in 32-bit); the other elements as they are."""
    out = x.clone()
    ang = pos.float()[:, None] * inv_freq.float()  # [T, rotary_dim / 2], one row of frequencies or one per token
    cos, sin = (ang.cos() * scale).double()[:, None, :], (ang.sin() * scale).double()[:, None, :]
    first = slice(0, rotary_dim, 2) if pairing == "interleaved" else slice(0, rotary_dim // 2)
    second = slice(1, rotary_dim, 2) if pairing == "interleaved" else slice(rotary_dim // 2, rotary_dim)
    a, b = x[..., first], x[..., second]
    out[..., first] = a * cos - b * sin
    out[..., second] = b * cos + a * sin
    return out


ARRANGEMENTS = [dict(rotary_dim=None, pairing="interleaved"), dict(rotary_dim=0.5, pairing="half"),
                dict(rotary_dim=0.5, pairing="interleaved"), dict(rotary_dim=0.25, pairing="half"),
                dict(rotary_dim=0.75, pairing="interleaved")]


def _how(arrangement, d):
    """Keywords of the launches that rotate, the table of frequencies' length, for a head size."""
    r = d if arrangement["rotary_dim"] is None else max(2, int(d * arrangement["rotary_dim"]) // 2 * 2)
    return dict(rotary_dim=r, pairing=arrangement["pairing"]), r


def test_the_whole_head_in_half_split_pairs_is_what_the_reference_rotates():
    """The spelling above with the whole head and half-split pairs is the reference's rotate_half form."""
    x = torch.randn(5, 3, 16, dtype=torch.float64)
    pos, inv = torch.tensor([0, 3, 9, 70, 71]), P.rope_inv_freq(16, 10000.0)
    cos, sin = P.rope_cos_sin(pos, inv)
    torch.testing.assert_close(_rotate_plain(x, pos, inv[None, :], 1.0, 16, "half"), P.apply_rope(x, cos, sin), rtol=1e-12, atol=1e-12)
    # interleaved pairs are the same rotation of a head whose elements are laid out pair by pair
    order = torch.stack([torch.arange(8), torch.arange(8) + 8], dim=1).reshape(-1)  # 0, 8, 1, 9, ...
    torch.testing.assert_close(_rotate_plain(x[..., order], pos, inv[None, :], 1.0, 16, "interleaved"),
                               P.apply_rope(x, cos, sin)[..., order], rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("layout,nh,nkv,d", [("grouped", 6, 2, 32), ("tail", 7, 1, 64), ("interleaved", 5, 5, 24),
                                             ("grouped", 4, 1, 128)])
@pytest.mark.parametrize("arrangement", ARRANGEMENTS)
@pytest.mark.parametrize("rotary", [True, "per sequence"])
def test_rotation_of_part_of_the_head_and_of_interleaved_pairs(dtype, layout, nh, nkv, d, arrangement, rotary):
    """The kernel that splits, rotates and writes the cache with a rotation given as data: part of the head or all
    of it, half-split or interleaved pairs, against the spelling above; what is not rotated passes as it is."""
    ops = _ops()
    how, r = _how(arrangement, d)
    starts, news = [70, 0, 127], [3, 66, 1]
    lens = [s + n for s, n in zip(starts, news)]
    k_pool, v_pool, bt, lists = _cache_setup(3, lens, nkv, d, dtype)
    M = sum(news)
    fused = _rand(M, (nh + 2 * nkv) * d, dtype=dtype)
    bias = _rand((nh + 2 * nkv) * d, seed=9)
    token_seq = torch.tensor([i for i, n in enumerate(news) for _ in range(n)], dtype=torch.int32).cuda()
    token_pos = torch.tensor([s + j for s, n in zip(starts, news) for j in range(n)], dtype=torch.int32).cuda()
    inv = _freq(rotary, r, 3, 500042.0, 2.0)
    q = ops.qkv_rope_cache(fused, bias, inv, 0.8, token_pos, token_seq, bt, k_pool, v_pool, nh, nkv, d, layout, **how)
    c = dict(num_attention_heads=nh, hidden_size=nh * d, num_kv_heads=nkv,
             new_decoder_architecture=layout == "grouped", multi_query=layout == "tail")
    rnd = (lambda t: t) if dtype == torch.float32 else (lambda t: t.bfloat16().double())
    wq, wk, wv = P.split_heads(rnd(fused.double().cpu() + bias.double().cpu()), c)
    per_token = inv.cpu()[token_seq.cpu().long()] if rotary == "per sequence" else inv.cpu()[None, :]
    wq, wk = (_rotate_plain(t, token_pos.cpu(), per_token, 0.8, r, how["pairing"]) for t in (wq, wk))
    tol = dict(rtol=1e-5, atol=1e-5) if dtype == torch.float32 else dict(rtol=1e-2, atol=1e-2)
    torch.testing.assert_close(q.double().cpu(), wq, **tol)
    if r < d and dtype == torch.bfloat16:  # what lies past rotary_dim is the fused row's value (and bias), bit for bit
        assert torch.equal(q[..., r:].double().cpu(), wq[..., r:])
    at = 0
    for i, (s_, n) in enumerate(zip(starts, news)):
        gk, gv = _gather(k_pool, lists[i], lens[i]), _gather(v_pool, lists[i], lens[i], transposed=True)
        torch.testing.assert_close(gk[s_:].double().cpu(), wk[at:at + n].contiguous(), **tol)
        torch.testing.assert_close(gv[s_:].double().cpu(), wv[at:at + n].contiguous(), **tol)
        at += n
    for bad, match in ((dict(rotary_dim=d + 2), "rotary_dim"), (dict(rotary_dim=5), "rotary_dim"), (dict(pairing="thirds"), "pairing")):
        with pytest.raises(ops.KernelError, match=match):
            ops.qkv_rope_cache(fused, bias, inv, 1.0, token_pos, token_seq, bt, k_pool, v_pool, nh, nkv, d, layout, **bad)


@pytest.mark.parametrize("layout,nh,nkv,d", [("grouped", 4, 2, 32), ("tail", 7, 1, 64), ("interleaved", 3, 3, 96), ("grouped", 8, 2, 128)])
@pytest.mark.parametrize("arrangement", ARRANGEMENTS)
def test_fused_launches_rotate_as_the_kernel_of_its_own_in_every_arrangement(layout, nh, nkv, d, arrangement):
    """The three launches that take fused query_key_value rows to their end (the pair launch for few rows, the pair
    launch of a decode batch, the batch product on its own) with a rotation of part of the head or of interleaved
    pairs: queries and pages bit for bit those of the product followed by the kernel of its own."""
    ops = _ops()
    how, r = _how(arrangement, d)
    K, N2 = 264, 200
    N1 = (nh + 2 * nkv) * d
    w1, w2 = _rand(N1, K, seed=1, dtype=torch.bfloat16, scale=0.05), _rand(N2, K, seed=2, dtype=torch.bfloat16, scale=0.05)
    b1, b2 = _rand(N1, seed=3), _rand(N2, seed=4)
    same = lambda a, b: torch.equal(torch.nan_to_num(a.float(), nan=-7.0), torch.nan_to_num(b.float(), nan=-7.0))
    for M in (5, 40):
        g = torch.Generator().manual_seed(M)
        starts = torch.randint(0, 190, (M,), generator=g).tolist()
        lens = [s_ + 1 for s_ in starts]
        x = _rand(M, K, dtype=torch.bfloat16)
        token_seq = torch.arange(M, dtype=torch.int32).cuda()
        token_pos = torch.tensor(starts, dtype=torch.int32).cuda()
        inv = _freq("per sequence", r, M)
        results = {}
        for way in ("own kernel", "pair") + (("single",) if M > 16 else ()):
            k_pool, v_pool, bt, _ = _cache_setup(M, lens, nkv, d, torch.bfloat16, n_pages=3 * M + 8)
            tail_args = (inv, 0.9, token_pos, token_seq, bt, k_pool, v_pool, nh, nkv, d, layout)
            if way == "own kernel":
                fused = (ops.gemm_skinny_pair_bf16 if M <= 16 else ops.gemm_splitk_pair_bf16)(x, w1, x, w2, None, None, b2, "gelu")[0]
                q = ops.qkv_rope_cache(fused, b1, *tail_args, **how)
            elif way == "pair":
                fn = ops.gemm_skinny_pair_qkv if M <= 16 else ops.gemm_splitk_pair_qkv
                q = fn(x, w1, b1, *tail_args, True, x, w2, b2, "gelu", **how)[0]
            else:
                q = ops.gemm_splitk_qkv(x, w1, b1, *tail_args, True, **how)
            results[way] = (q, k_pool, v_pool)
        q0, k0, v0 = results["own kernel"]
        for way, (q, k_pool, v_pool) in results.items():
            if way == "single":  # the product on its own cuts K by its own rule: its own bits, the same rotation
                fused = ops.gemm_splitk_bf16(x, w1)
                k_pool2, v_pool2, bt2, _ = _cache_setup(M, lens, nkv, d, torch.bfloat16, n_pages=3 * M + 8)
                q0 = ops.qkv_rope_cache(fused, b1, inv, 0.9, token_pos, token_seq, bt2, k_pool2, v_pool2, nh, nkv, d, layout, **how)
                k0, v0 = k_pool2, v_pool2
            assert torch.equal(q, q0), (way, M)
            assert same(k_pool, k0) and same(v_pool, v0), (way, M)


@pytest.mark.parametrize("dtype", DTYPES)
def test_score_bias_of_the_distance_and_with_another_scale(dtype):
    """The bias on scores as data: slopes times the key's position or times its distance from the query (equal
    under softmax), exact or rounded as the reference rounds, with any scale; prompts, chunks and decode steps of
    both attention kernels against plain attention with the bias spelled out."""
    ops = _ops()
    nh, nkv, d = 6, 2, 32
    slopes = (0.5 ** torch.arange(1, nh + 1).float()).cuda()
    starts, news = [0, 63, 200, 0, 127], [70, 1, 5, 1, 2]

    def case(fn, bias_scale, **kw):
        def run(q, k_pool, v_pool, bt, token_seq, token_pos, slopes_, scale, starts_, news_, window=0):
            return fn(q, k_pool, v_pool, bt, token_seq, token_pos, slopes_, scale, starts_, news_, bias_scale=bias_scale, **kw)
        return run

    def generic(q, k_pool, v_pool, bt, token_seq, token_pos, slopes_, scale, starts_, news_, **kw):
        return ops.attn_generic(q, k_pool, v_pool, bt, token_seq, token_pos, slopes_, scale, 0, **kw)

    def mfma(q, k_pool, v_pool, bt, token_seq, token_pos, slopes_, scale, starts_, news_, **kw):
        cu = torch.tensor([0] + list(torch.tensor(news_).cumsum(0)), dtype=torch.int32).cuda()
        st = torch.tensor(starts_, dtype=torch.int32).cuda()
        return ops.attn_mfma(q, k_pool, v_pool, bt, cu, st, slopes_, scale, max_new=max(news_), **kw)

    kernels = [generic] + ([mfma] if dtype == torch.bfloat16 else [])
    for fn in kernels:
        for bias_scale in (1.0, 0.3):
            for kw in (dict(alibi_exact=True), dict(alibi_exact=True, bias_of="distance")):
                _attn_case(ops, case(fn, bias_scale, **kw), dtype, nh, nkv, d, starts, news, slopes=slopes,
                           plain_bias=lambda L: (slopes.cpu().double()[:, None] * torch.arange(L).double()[None, :]) * bias_scale)
        # the reference's rounding (bfloat16 slopes, position and product), with the scale it has there
        from pytorch_transformers_amd.parts import AlibiPositions
        _attn_case(ops, case(fn, d ** -0.5), dtype, nh, nkv, d, starts, news, slopes=AlibiPositions(nh).slopes.cuda())
    with pytest.raises(ops.KernelError, match="not built"):
        ops._score_bias_arg(slopes, nh, "query")
    assert ops.score_bias_problem("distance", True) and ops.score_bias_problem("key", True) is None


def _windowed_attention(q, k, v, window):
    """Plain attention in which query t sees keys t - window + 1 .. t; q [T, nh, d], k, v [T, nkv, d]."""
    T, nh, d = q.shape
    g = nh // k.shape[1]
    t = torch.arange(T)
    seen = (t[None, :] <= t[:, None]) & (t[None, :] > t[:, None] - window)
    out = torch.empty_like(q)
    for h in range(nh):
        s = (q[:, h] @ k[:, h // g].T / math.sqrt(d)).masked_fill(~seen, float("-inf"))
        out[:, h] = torch.softmax(s, dim=-1) @ v[:, h // g]
    return out.reshape(T, nh * d)


def _attn_case(ops, fn, dtype, nh, nkv, d, starts, news, slopes=None, seed=0, boost=None, window=0, plain_bias=None):
    """Fill a cache with random keys and values, run ``fn`` for the new tokens, compare with plain attention.
    With a window, the pages that lie wholly behind every new token's window hold NaN: they may be gone."""
    lens = [s + n for s, n in zip(starts, news)]
    n_pages = sum((L + 63) // 64 for L in lens) + 3
    k_pool, v_pool, bt, lists = _cache_setup(len(lens), lens, nkv, d, dtype, n_pages=n_pages, seed=seed)
    g = torch.Generator().manual_seed(seed + 1)
    ks, vs, qs = [], [], []
    for i, L in enumerate(lens):
        k = torch.randn(L, nkv, d, generator=g).to(dtype)
        v = torch.randn(L, nkv, d, generator=g).to(dtype)
        q = torch.randn(news[i], nh, d, generator=g).to(dtype)
        if boost is not None and boost[i] is not None:
            # one far key stands out for the last query: the output must be (almost) that key's value
            j = boost[i]
            k[j] = 0
            k[j, :, 0] = 6.0
            q[-1] = 0
            q[-1, :, 0] = 6.0 * math.sqrt(d)
        ks.append(k); vs.append(v); qs.append(q)
        for p, page in enumerate(lists[i]):
            n = min(64, L - p * 64)
            if window and (p + 1) * 64 <= starts[i] - window + 1:
                continue  # behind the window of the first new token: left as NaN
            k_pool[page, :, :n] = k[p * 64:p * 64 + n].transpose(0, 1).cuda()
            v_pool[page, :, :, :n] = v[p * 64:p * 64 + n].permute(1, 2, 0).cuda()
    q_all = torch.cat(qs).cuda()
    token_seq = torch.tensor([i for i, n in enumerate(news) for _ in range(n)], dtype=torch.int32).cuda()
    token_pos = torch.tensor([s + j for s, n in zip(starts, news) for j in range(n)], dtype=torch.int32).cuda()
    kw = {"window": window} if window else {}
    got = fn(q_all, k_pool, v_pool, bt, token_seq, token_pos, slopes, 1.0 / math.sqrt(d), starts, news, **kw)
    at = 0
    worst = 0.0
    for i, (s, n) in enumerate(zip(starts, news)):
        L = lens[i]
        bias = None
        if plain_bias is not None:  # [heads, keys] for a sequence of L keys
            bias = plain_bias(L)
        elif slopes is not None:
            bias = P.alibi_bias(nh, L, d)
        # plain attention of the whole sequence needs a query per position: only the new rows are compared
        q_full = torch.zeros(L, nh, d, dtype=torch.float64)
        q_full[s:] = qs[i].double()
        if window:
            want = _windowed_attention(q_full, ks[i].double(), vs[i].double(), window)[s:]
        else:
            want = P.attention_scores_softmax(q_full, ks[i].double(), vs[i].double(), bias)[s:]
        g_ = got[at:at + n].double().cpu()
        tol = 2e-5 if dtype == torch.float32 else 2e-2
        err = float((g_ - want).abs().max())
        assert err <= tol * max(1.0, float(want.abs().max())), f"sequence {i} (start {s}, {n} new): max diff {err:.3e}"
        worst = max(worst, err)
        if boost is not None and boost[i] is not None:
            far = vs[i][boost[i]].double().repeat_interleave(nh // nkv, 0).reshape(-1)
            assert float((g_[-1] - far).abs().max()) < 0.05, "the boosted far key does not dominate"
        at += n
    return worst


def _generic(ops):
    def fn(q, k_pool, v_pool, bt, token_seq, token_pos, slopes, scale, starts, news, window=0):
        return ops.attn_generic(q, k_pool, v_pool, bt, token_seq, token_pos, slopes, scale, window)
    return fn


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nh,nkv,d", [(7, 1, 64), (6, 2, 32), (3, 3, 24), (4, 2, 128), (2, 1, 256)])
def test_attn_generic(dtype, nh, nkv, d):
    """Prompts, single tokens and chunks over an existing cache in one launch; page edges at 64, 128."""
    ops = _ops()
    _attn_case(ops, _generic(ops), dtype, nh, nkv, d, starts=[0, 63, 200, 0, 127], news=[70, 1, 5, 1, 2])


@pytest.mark.parametrize("dtype", DTYPES)
def test_attn_generic_far_key_and_alibi(dtype):
    ops = _ops()
    _attn_case(ops, _generic(ops), dtype, 4, 2, 32, starts=[700, 0, 300], news=[1, 650, 3], boost=[5, 64, 299])
    from pytorch_transformers_amd.parts import AlibiPositions
    for nh in (6, 20):
        slopes = AlibiPositions(nh).slopes.cuda()
        _attn_case(ops, _generic(ops), dtype, nh, nh, 16, starts=[0, 290], news=[40, 30], slopes=slopes)


def _mfma(ops, n_splits_for=None, tiles=0, waves=1, wide=None):
    def fn(q, k_pool, v_pool, bt, token_seq, token_pos, slopes, scale, starts, news, window=0):
        cu = torch.tensor([0] + list(torch.tensor(news).cumsum(0)), dtype=torch.int32).cuda()
        st = torch.tensor(starts, dtype=torch.int32).cuda()
        n_splits = 1
        if n_splits_for is not None:
            n_splits = (max(s + n for s, n in zip(starts, news)) + n_splits_for - 1) // n_splits_for
        return ops.attn_mfma(q, k_pool, v_pool, bt, cu, st, slopes, scale, max_new=max(news), n_splits=n_splits,
                             split_size=n_splits_for or 256, window=window, decode_tiles=tiles, decode_waves=waves,
                             prompt_wide=wide)
    return fn


@pytest.mark.parametrize("nh,nkv,d", [(71, 1, 64), (7, 1, 64), (6, 2, 32), (3, 3, 16), (4, 2, 128), (2, 1, 256),
                                      (5, 5, 48), (8, 2, 80), (4, 4, 96), (2, 2, 112), (32, 8, 128)])
def test_attn_mfma_prefill_and_chunks(nh, nkv, d):
    """Whole prompts, single tokens and chunks over an existing cache in one launch (bfloat16 matrix cores)."""
    ops = _ops()
    assert ops.attn_mfma_ok(torch.empty(1, nh, d, dtype=torch.bfloat16).cuda())
    _attn_case(ops, _mfma(ops), torch.bfloat16, nh, nkv, d, starts=[0, 63, 200, 0, 127, 31], news=[70, 1, 5, 1, 2, 40])


@pytest.mark.parametrize("nh,nkv,d", [(71, 1, 64), (16, 2, 64), (8, 2, 128), (6, 1, 48)])
def test_attn_mfma_long_prompts(nh, nkv, d):
    """A prompt of 1,300 tokens and 500 new tokens over 900 cached ones in one launch: many stages of keys per
    workgroup, column groups of every length, with one far key that stands out for the last query of each."""
    ops = _ops()
    _attn_case(ops, _mfma(ops), torch.bfloat16, nh, nkv, d, starts=[0, 900, 3], news=[1300, 500, 61], boost=[7, 1390, None])
    if d <= 64:
        # workgroups of eight waves, which launches with four such workgroups a compute unit and more choose by themselves
        eight = _mfma(ops, wide=True)
        _attn_case(ops, eight, torch.bfloat16, nh, nkv, d, starts=[0, 900, 3], news=[1300, 500, 61], boost=[7, 1390, None])
        _attn_case(ops, eight, torch.bfloat16, nh, nkv, d, starts=[0, 63, 200, 0, 127, 31], news=[70, 1, 5, 1, 2, 40])
        _attn_case(ops, eight, torch.bfloat16, nh, nkv, d, starts=[0, 700], news=[800, 300], window=200, seed=4)
    slopes = None
    if nh == 16:
        from pytorch_transformers_amd.parts import AlibiPositions
        slopes = AlibiPositions(nh).slopes.cuda()
        _attn_case(ops, _mfma(ops), torch.bfloat16, nh, nkv, d, starts=[0, 700], news=[800, 300], slopes=slopes, seed=3)
        _attn_case(ops, _mfma(ops), torch.bfloat16, nh, nkv, d, starts=[0, 700], news=[800, 300], window=200, seed=4)


@pytest.mark.parametrize("nh,nkv,d", [(71, 1, 64), (6, 2, 32), (3, 3, 16), (8, 2, 128), (2, 1, 256)])
@pytest.mark.parametrize("split", [64, 256])
def test_attn_mfma_decode_split(nh, nkv, d, split):
    """One token per sequence, contexts of very different lengths, keys split over waves and merged."""
    ops = _ops()
    _attn_case(ops, _mfma(ops, split), torch.bfloat16, nh, nkv, d, starts=[0, 63, 64, 700, 255, 256, 1], news=[1] * 7)


@pytest.mark.parametrize("nh,nkv,d", [(3, 3, 16), (6, 2, 32), (5, 5, 48), (7, 1, 64), (8, 2, 80), (2, 2, 112), (4, 2, 128),
                                      (2, 1, 256)])
def test_attn_mfma_many_ranges(nh, nkv, d):
    """One token per sequence over contexts of up to 4,500 keys cut into ranges of 64: up to 71 partial results a
    row, which four waves merge (groups of 4 to 64 lanes per result, some lanes idle where the head size is no
    power of two), ranges past a shorter sequence's end, and a far key in a range of its own."""
    ops = _ops()
    starts = [4499, 130, 2100, 63, 1025]
    _attn_case(ops, _mfma(ops, 64), torch.bfloat16, nh, nkv, d, starts=starts, news=[1] * 5, boost=[70, None, 2000, 5, None])
    _attn_case(ops, _mfma(ops, 128), torch.bfloat16, nh, nkv, d, starts=starts, news=[1] * 5, boost=[4490, 129, None, None, 1])


@pytest.mark.parametrize("nh,nkv,d,tiles", [(71, 1, 64, 1), (71, 1, 64, 2), (71, 1, 64, 3), (71, 1, 64, 5), (40, 1, 32, 3),
                                            (128, 2, 128, 4), (128, 2, 128, 3), (66, 2, 16, 2), (17, 1, 256, 1)])
def test_attn_mfma_decode_tiles(nh, nkv, d, tiles):
    """One token per sequence with many heads on a KV head: a wave holds `tiles` groups of sixteen of them,
    the last group partly filled; with split ranges and without, with and without ALiBi and a window."""
    ops = _ops()
    from pytorch_transformers_amd.parts import AlibiPositions
    starts = [0, 63, 64, 700, 255, 256, 1]
    for split in (None, 128):
        _attn_case(ops, _mfma(ops, split, tiles), torch.bfloat16, nh, nkv, d, starts=starts, news=[1] * 7)
    if d == 64:
        slopes = AlibiPositions(nh).slopes.cuda()
        _attn_case(ops, _mfma(ops, 128, tiles), torch.bfloat16, nh, nkv, d, starts=starts, news=[1] * 7, slopes=slopes)
        _attn_case(ops, _mfma(ops, 128, tiles), torch.bfloat16, nh, nkv, d, starts=starts, news=[1] * 7, window=100)
    most = min((nh // nkv + 15) // 16, 5 if d <= 64 else 4 if d <= 128 else 1)
    with pytest.raises(ops.KernelError, match="column tiles per decode wave"):
        _attn_case(ops, _mfma(ops, None, most + 1), torch.bfloat16, nh, nkv, d, starts=[5], news=[1])


@pytest.mark.parametrize("nh,nkv,d,tiles", [(71, 1, 64, 1), (71, 1, 64, 2), (6, 2, 32, 1), (3, 3, 16, 1), (32, 8, 128, 1),
                                            (40, 2, 128, 2), (17, 1, 256, 1), (5, 5, 48, 1), (20, 1, 80, 2), (9, 3, 112, 1)])
@pytest.mark.parametrize("waves", [4, 8])
def test_attn_mfma_decode_waves(nh, nkv, d, tiles, waves):
    """One token per sequence, a workgroup of four or eight waves that take the keys block by block in turn and
    merge in LDS: the whole context in one workgroup (no second launch), and ranges of 256 and 512 keys merged
    afterwards as well; contexts shorter than the waves have blocks for, page edges, ALiBi, a window, and one
    far key that must dominate whichever wave it falls to."""
    ops = _ops()
    from pytorch_transformers_amd.parts import AlibiPositions
    assert ops.load_library().pta_attn_decode_waves_ok(d, tiles, waves)
    starts = [0, 63, 64, 700, 255, 256, 1, 31, 32, 1500]
    boost = [0, 40, None, 333, None, 17, None, None, 31, 1203]
    for split in (None, 256, 512):
        _attn_case(ops, _mfma(ops, split, tiles, waves), torch.bfloat16, nh, nkv, d, starts=starts, news=[1] * 10, boost=boost)
    slopes = AlibiPositions(nh).slopes.cuda()
    _attn_case(ops, _mfma(ops, None, tiles, waves), torch.bfloat16, nh, nkv, d, starts=starts, news=[1] * 10, slopes=slopes)
    for window in (33, 100):
        for split in (None, 256):
            _attn_case(ops, _mfma(ops, split, tiles, waves), torch.bfloat16, nh, nkv, d, starts=starts, news=[1] * 10,
                       window=window)


def test_attn_mfma_decode_waves_refusals():
    ops = _ops()
    lib = ops.load_library()
    assert not lib.pta_attn_decode_waves_ok(64, 3, 4) and not lib.pta_attn_decode_waves_ok(64, 1, 2)
    assert not lib.pta_attn_decode_waves_ok(64, 1, 16) and lib.pta_attn_decode_waves_ok(64, 5, 1)
    assert not lib.pta_attn_decode_waves_ok(256, 2, 4) and lib.pta_attn_decode_waves_ok(256, 1, 8)
    with pytest.raises(ops.KernelError, match="waves on the keys of a workgroup"):
        _attn_case(ops, _mfma(ops, None, 3, 4), torch.bfloat16, 71, 1, 64, starts=[5], news=[1])
    with pytest.raises(ops.KernelError, match="waves on the keys of a workgroup"):
        _attn_case(ops, _mfma(ops, None, 1, 2), torch.bfloat16, 71, 1, 64, starts=[5], news=[1])


@pytest.mark.parametrize("nh,nkv,d", [(71, 1, 64), (64, 1, 64), (100, 1, 64), (130, 2, 128), (56, 1, 128), (128, 1, 128)])
def test_attn_mfma_decode_shared_keys(nh, nkv, d):
    """One token per sequence, the heads of a KV head on the waves of one workgroup that shares its keys through
    LDS (four and five waves of one tile, four of two): the whole context in one workgroup and ranges of 128, 256
    and 512 keys merged afterwards; contexts shorter than a stage, page edges, ALiBi, a window, and one far key
    that must dominate in whichever range it lies."""
    ops = _ops()
    from pytorch_transformers_amd.parts import AlibiPositions
    assert ops.attn_decode_shared_ok(d, nh // nkv)
    starts = [0, 63, 64, 700, 255, 256, 1, 31, 32, 1500]
    boost = [0, 40, None, 333, None, 17, None, None, 31, 1203]
    shared = ops.SHARED_KEYS
    for split in (None, 128, 256, 512):
        _attn_case(ops, _mfma(ops, split, 0, shared), torch.bfloat16, nh, nkv, d, starts=starts, news=[1] * 10, boost=boost)
    slopes = AlibiPositions(nh).slopes.cuda()
    for split in (None, 256):
        _attn_case(ops, _mfma(ops, split, 0, shared), torch.bfloat16, nh, nkv, d, starts=starts, news=[1] * 10, slopes=slopes)
    for window in (33, 100):
        for split in (None, 256):
            _attn_case(ops, _mfma(ops, split, 0, shared), torch.bfloat16, nh, nkv, d, starts=starts, news=[1] * 10,
                       window=window)


def test_attn_mfma_decode_shared_keys_refusals():
    ops = _ops()
    assert ops.attn_decode_shared_ok(64, 71) and ops.attn_decode_shared_ok(128, 49) and ops.attn_decode_shared_ok(64, 128)
    assert not ops.attn_decode_shared_ok(64, 48) and not ops.attn_decode_shared_ok(64, 129)
    assert not ops.attn_decode_shared_ok(48, 71) and not ops.attn_decode_shared_ok(256, 71)
    for nh, nkv, d in ((32, 8, 128), (71, 1, 48)):
        with pytest.raises(ops.KernelError, match="keys shared through LDS is not built"):
            _attn_case(ops, _mfma(ops, None, 0, ops.SHARED_KEYS), torch.bfloat16, nh, nkv, d, starts=[5], news=[1])


def test_decode_plan():
    """The cut of a decode launch: whole tiles within what the head size allows, a range size that is a
    multiple of the page, the same for every batch and context of one captured step's bucket."""
    ops = _ops()
    bucket_keys = lambda n, length: (1 << (n - 1).bit_length()) * ((length + 1023) // 1024 * 1024)
    assert ops.decode_plan(64, 71, 1, 64, 1100)[2] == ops.SHARED_KEYS and ops.decode_plan(8, 71, 1, 64, 1100)[2] == 1
    for nh, nkv, d in ((71, 1, 64), (32, 8, 128), (128, 8, 64), (6, 2, 32), (2, 1, 256)):
        groups = (nh // nkv + 15) // 16
        for n in (1, 3, 8, 33, 64, 128, 300, 512):
            for length in (1, 100, 1024, 1025, 2049, 8192, 32768, 65536, 100000, 300000):
                tiles, size, waves = ops.decode_plan(n, nh, nkv, d, length)
                # the rule: one wave a workgroup, or, with many heads on a KV head and keys enough, shared keys
                assert 1 <= tiles <= groups and size % 64 == 0 and size >= 128
                assert waves == 1 or (waves == ops.SHARED_KEYS and ops.attn_decode_shared_ok(d, nh // nkv)
                                      and bucket_keys(n, length) >= 20000)
                assert (length + size - 1) // size <= 1024
                bucket_n = 1 << (n - 1).bit_length()
                # the launch has one workgroup row per (sequence of the padded batch, range): the grid's limit
                assert bucket_n * ((((length + 1023) // 1024 * 1024) + size - 1) // size) <= 65535
                bucket_len = (length + 1023) // 1024 * 1024
                assert (tiles, size, waves) == ops.decode_plan(bucket_n, nh, nkv, d, bucket_len)
                for mean in (1, length // 3 + 1, length):
                    cut = ops.decode_plan(n, nh, nkv, d, length, mean)
                    assert cut == ops.decode_plan(bucket_n, nh, nkv, d, bucket_len, min(bucket_len, (mean + 511) // 512 * 512))
                    assert 1 <= cut[0] <= groups and cut[1] % 64 == 0 and (length + cut[1] - 1) // cut[1] <= 1024


@pytest.mark.parametrize("nh,nkv,d", [(71, 1, 64), (32, 8, 128), (128, 8, 64)])
@pytest.mark.parametrize("n,lengths", [(8, "equal"), (64, "equal"), (16, "unequal"), (33, "unequal")])
def test_decode_attention_as_planned(nh, nkv, d, n, lengths):
    """A decode step's attention the way the engine cuts it at the published models' head shapes (groups of
    heads per wave, keys per wave, with and without partial sums), against plain attention over each sequence's keys
    and values as the pages hold them (float64, on the GPU)."""
    from types import SimpleNamespace

    from pytorch_transformers_amd.engine.model import _len_bound, mean_len_bound

    ops = _ops()
    g = torch.Generator().manual_seed(n * 1000 + nh)
    lens = [1100] * n if lengths == "equal" else [int(x) for x in torch.randint(100, 4400, (n,), generator=g)]
    pages = [(L + 63) // 64 for L in lens]
    width = max(pages)
    k_pool = torch.randn(sum(pages), nkv, 64, d, generator=g).bfloat16().cuda()
    v_pool = torch.randn(sum(pages), nkv, d, 64, generator=g).bfloat16().cuda()
    bt = torch.zeros(n, width, dtype=torch.int32)
    at = 0
    for i, p in enumerate(pages):
        bt[i, :p] = torch.arange(at, at + p, dtype=torch.int32)
        at += p
    q = torch.randn(n, nh, d, generator=g).bfloat16().cuda()
    q[0] = 0
    q[0, :, 0] = 6.0 * math.sqrt(d)          # sequence 0 looks at one far key only
    k_pool[int(bt[0, 0]), :, 5] = 0
    k_pool[int(bt[0, 0]), :, 5, 0] = 6.0
    starts = [L - 1 for L in lens]
    ctx = SimpleNamespace(is_decode=True, n_seqs=n, max_len=max(lens), new_tokens=[1] * n,
                          mean_len=mean_len_bound(sum(lens), n, _len_bound(max(lens))),
                          cu_tokens=torch.arange(n + 1, dtype=torch.int32).cuda(),
                          seq_start=torch.tensor(starts, dtype=torch.int32).cuda(),
                          token_seq=torch.arange(n, dtype=torch.int32).cuda(),
                          token_pos=torch.tensor(starts, dtype=torch.int32).cuda())
    scale = 1.0 / math.sqrt(d)
    got = ops.attention(q, k_pool, v_pool, bt.cuda(), ctx, None, scale).float()
    rows = []
    for i, L in enumerate(lens):
        mine = bt[i, :pages[i]].long().cuda()
        k = k_pool[mine].permute(0, 2, 1, 3).reshape(-1, nkv, d)[:L].double()  # [page, kv head, 64, d] -> [keys, kv head, d]
        v = v_pool[mine].permute(0, 3, 1, 2).reshape(-1, nkv, d)[:L].double()  # [page, kv head, d, 64] -> the same
        q_full = torch.zeros(L, nh, d, dtype=torch.float64, device="cuda")
        q_full[-1] = q[i].double()  # plain attention wants a query per position: the last one is the step's
        rows.append(P.attention_scores_softmax(q_full, k, v)[-1])
    want = torch.stack(rows).float()
    assert float((got - want).abs().max()) <= 2e-2 * max(1.0, float(want.abs().max()))
    far = v_pool[int(bt[0, 0]), :, :, 5].float().repeat_interleave(nh // nkv, 0).reshape(-1)
    assert float((got[0] - far).abs().max()) < 0.05, "the far key does not dominate"
    tiles, size, waves = ops.decode_plan(n, nh, nkv, d, ctx.max_len, ctx.mean_len)
    assert 1 <= tiles <= (nh // nkv + 15) // 16 and size % 64 == 0 and waves in (1, ops.SHARED_KEYS)
    # the same launch with every other cut that may be timed against the rule's: the same result within rounding;
    # a fixed cut holds for the step's bucket and for no other, travels in the tuning table, and is forgotten with it
    key = ops.decode_key(n, nh, nkv, d, ctx.max_len, ctx.mean_len)
    cuts = ops.decode_plan_candidates(key)
    assert cuts[0] == (tiles, size, waves) and len(set(cuts)) == len(cuts) > 3 and any(c[2] > 1 for c in cuts)
    assert any(c[2] == ops.SHARED_KEYS for c in cuts) == ops.attn_decode_shared_ok(d, nh // nkv)
    try:
        with ops.live_tuning():
            ops.take_decode_keys()
            ops.attention(q, k_pool, v_pool, bt.cuda(), ctx, None, scale)
            assert ops.take_decode_keys() == [key] and ops.take_decode_keys() == []
        for cut in cuts[1:]:
            assert cut[1] % 64 == 0 and (ops.attn_decode_shared_ok(d, nh // nkv) if cut[2] == ops.SHARED_KEYS
                                         else ops.load_library().pta_attn_decode_waves_ok(d, cut[0], cut[2]))
            ops.set_decode_plan(key, cut)
            assert ops.decode_plan(n, nh, nkv, d, ctx.max_len, ctx.mean_len) == cut
            fixed = ops.attention(q, k_pool, v_pool, bt.cuda(), ctx, None, scale).float()
            assert float((fixed - want).abs().max()) <= 2e-2 * max(1.0, float(want.abs().max())), cut
            assert float((fixed[0] - far).abs().max()) < 0.05, cut
        other = ops.decode_plan(n, nh, nkv, d, ctx.max_len + 2048, ctx.mean_len)  # another bucket: the rule
        assert other == ops.decode_plan_candidates(ops.decode_key(n, nh, nkv, d, ctx.max_len + 2048, ctx.mean_len))[0]
        table = ops.tuning_table()
        assert table["decode_plans"][",".join(str(v) for v in key)] == list(cuts[-1])
        ops.clear_tuning()
        assert ops.decode_plan(n, nh, nkv, d, ctx.max_len, ctx.mean_len) == cuts[0]
        ops.load_tuning(table)
        assert ops.decode_plan(n, nh, nkv, d, ctx.max_len, ctx.mean_len) == cuts[-1]
        ops.set_decode_plan(key, None)
        assert ops.decode_plan(n, nh, nkv, d, ctx.max_len, ctx.mean_len) == cuts[0]
    finally:
        ops.clear_tuning()


@pytest.mark.parametrize("window", [1, 33, 64, 100, 200])
def test_attention_with_a_window(window):
    """Each token sees its last `window` positions only; pages behind the window hold NaN and are not read.
    Prompts longer than the window, chunks over a cache, decode steps with and without split ranges."""
    ops = _ops()
    starts, news = [0, 63, 300, 0, 127, 500], [70, 1, 5, 1, 2, 150]
    for dtype in DTYPES:
        _attn_case(ops, _generic(ops), dtype, 6, 2, 32, starts, news, window=window)
    for nh, nkv, d in ((6, 2, 32), (71, 1, 64), (4, 4, 128)):
        _attn_case(ops, _mfma(ops), torch.bfloat16, nh, nkv, d, starts, news, window=window)
        _attn_case(ops, _mfma(ops, 64), torch.bfloat16, nh, nkv, d, [0, 63, 64, 700, 255, 256, 1], [1] * 7, window=window)
        _attn_case(ops, _mfma(ops, 256), torch.bfloat16, nh, nkv, d, [900, 30], [1, 1], window=window)


def test_attn_mfma_far_key_alibi_and_refusals():
    ops = _ops()
    _attn_case(ops, _mfma(ops), torch.bfloat16, 4, 2, 32, starts=[700, 0, 300], news=[1, 650, 3], boost=[5, 64, 299])
    _attn_case(ops, _mfma(ops, 128), torch.bfloat16, 4, 2, 32, starts=[700, 900, 300], news=[1, 1, 1], boost=[5, 64, 299])
    from pytorch_transformers_amd.parts import AlibiPositions
    for nh in (6, 20):
        slopes = AlibiPositions(nh).slopes.cuda()
        _attn_case(ops, _mfma(ops), torch.bfloat16, nh, nh, 16, starts=[0, 290], news=[40, 30], slopes=slopes)
        _attn_case(ops, _mfma(ops, 64), torch.bfloat16, nh, nh, 16, starts=[39, 319], news=[1, 1], slopes=slopes)
    assert not ops.attn_mfma_ok(torch.empty(1, 2, 24, dtype=torch.bfloat16).cuda())  # head size 24: the 32-bit kernel runs
    assert not ops.attn_mfma_ok(torch.empty(1, 2, 64, dtype=torch.float32).cuda())
    with pytest.raises(ops.KernelError, match="head size 144 is not built"):
        q = torch.zeros(1, 1, 144, dtype=torch.bfloat16).cuda()
        ops.attn_mfma(q, torch.zeros(1, 1, 64, 144, dtype=torch.bfloat16).cuda(), torch.zeros(1, 1, 144, 64, dtype=torch.bfloat16).cuda(),
                      torch.zeros(1, 1, dtype=torch.int32).cuda(), torch.tensor([0, 1], dtype=torch.int32).cuda(),
                      torch.zeros(1, dtype=torch.int32).cuda(), None, 1.0, max_new=1)
