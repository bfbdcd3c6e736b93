"""What pins the plain implementation besides the reference's text (no GPU).

Vectors that the reference's own tests hold, special cases that reduce to a torch routine, and
invariants; each is chosen so that a plausible mistake fails it (named in the test's docstring).
"""
import math

import pytest
import torch
import torch.nn.functional as F

import plain_falcon as P
from tiny import TINY, write_model

D = torch.float64


def rnd(*shape, seed=0):
    return torch.randn(*shape, dtype=D, generator=torch.Generator().manual_seed(seed))


# --- norm, activation ----------------------------------------------------------------------
def test_layer_norm_is_torchs():
    """Fails for unbiased variance, eps outside the root, or a missing affine term."""
    x, w, b = rnd(5, 48) * 3 + 1, rnd(48, seed=1), rnd(48, seed=2)
    for eps in (1e-5, 1e-2):
        torch.testing.assert_close(P.layer_norm(x, w, b, eps), F.layer_norm(x, (48,), w, b, eps))
    torch.testing.assert_close(P.layer_norm(x + 7.5, w, b, 1e-5), P.layer_norm(x, w, b, 1e-5))
    y = P.layer_norm(x, torch.ones(48, dtype=D), torch.zeros(48, dtype=D), 1e-12)
    torch.testing.assert_close(y.mean(-1), torch.zeros(5, dtype=D), atol=1e-12, rtol=0)
    torch.testing.assert_close((y ** 2).mean(-1), torch.ones(5, dtype=D))


def test_gelu_is_the_erf_form():
    """The reference's vector (tests/utils/test_activations.py:29-33); fails for the tanh form."""
    x = torch.tensor([-100, -1, -0.1, 0, 0.1, 1.0, 100], dtype=D)
    torch.testing.assert_close(P.gelu(x), F.gelu(x))
    assert not torch.allclose(P.gelu(x), F.gelu(x, approximate="tanh"), atol=1e-6, rtol=0)


def test_hand_written_activations_against_torchs_own():
    """The activations that the plain table spells out by hand, on the reference's vector
    (tests/utils/test_activations.py:29-33) and on a denser one, each against a torch routine or an
    independent spelling; fails for a wrong constant (1.702, 0.044715, sqrt(2/pi)), a missing clip, a cube
    taken of the wrong term or a square in front of the relu."""
    for x in (torch.tensor([-100, -1, -0.1, 0, 0.1, 1.0, 100], dtype=D), torch.linspace(-6, 6, 97, dtype=D)):
        tanh_form = F.gelu(x, approximate="tanh")
        for name in ("gelu_new", "gelu_pytorch_tanh", "gelu_accurate", "gelu_fast"):
            torch.testing.assert_close(P.activation(x, name), tanh_form, rtol=1e-8, atol=1e-9)
        torch.testing.assert_close(P.activation(x, "gelu_python"), F.gelu(x))
        torch.testing.assert_close(P.activation(x, "quick_gelu"), x / (1 + torch.exp(-1.702 * x)))
        torch.testing.assert_close(P.activation(x, "gelu_10"), torch.clamp(F.gelu(x), -10, 10))
        torch.testing.assert_close(P.activation(x, "relu2"), torch.where(x > 0, x * x, torch.zeros_like(x)))
        torch.testing.assert_close(P.activation(x, "silu"), x * torch.sigmoid(x))
        torch.testing.assert_close(P.activation(x, "swish"), F.silu(x))
        torch.testing.assert_close(P.activation(x, "mish"), x * torch.tanh(F.softplus(x)))
        torch.testing.assert_close(P.activation(x, "leaky_relu"), torch.where(x > 0, x, 0.01 * x))
        torch.testing.assert_close(P.activation(x, "relu6"), torch.clamp(x, 0, 6))
        # the Laplace activation is the normal distribution function with mean 0.707107 and deviation 0.282095
        # (src/transformers/activations.py:176-178)
        normal = torch.distributions.Normal(torch.tensor(0.707107, dtype=D), torch.tensor(0.282095, dtype=D))
        torch.testing.assert_close(P.activation(x, "laplace"), normal.cdf(x), rtol=1e-7, atol=1e-12)
    x = torch.tensor([-100, -1, -0.1, 0, 0.1, 1.0, 100], dtype=D)
    # tests/utils/test_activations.py:35-47: clipped at 10, equal to the exact form below the clip
    y, y10 = P.activation(x, "gelu"), P.activation(x, "gelu_10")
    assert float(y10.max()) == 10.0 and float(y.max()) == 100.0
    torch.testing.assert_close(y10[:-1], y[:-1])
    assert not torch.allclose(P.activation(x, "gelu_new"), y, atol=1e-6, rtol=0)  # :29-33
    assert not torch.allclose(P.activation(x, "quick_gelu"), y, atol=1e-4, rtol=0)


# --- rotary ---------------------------------------------------------------------------------
def test_rope_inv_freq_vector():
    """tests/utils/test_modeling_rope_utils.py:133-166: d=128, theta=1e4."""
    inv = P.rope_inv_freq(128, 10000.0)
    expected = torch.tensor([10.0 ** (-i / 16.0) for i in range(64)])
    torch.testing.assert_close(inv, expected, rtol=1e-4, atol=0)
    assert inv.dtype == torch.float32 and abs(float(inv[1]) - 8.6596e-01) < 1e-4 and abs(float(inv[63]) - 1.1548e-04) < 1e-7
    torch.testing.assert_close(P.rope_inv_freq(128, 10000.0, 4.0), inv / 4.0)  # linear scaling (:168-194)


YARN_SNAPSHOT = [  # tests/utils/test_modeling_rope_utils.py:235-252: d=128, theta=1e4, context 2048, factor 10
    1.0000e+00, 8.6596e-01, 7.4989e-01, 6.4938e-01, 5.6234e-01, 4.8697e-01, 4.2170e-01, 3.6517e-01, 3.1623e-01, 2.7384e-01,
    2.3714e-01, 2.0535e-01, 1.7783e-01, 1.5399e-01, 1.3335e-01, 1.1548e-01, 1.0000e-01, 8.3479e-02, 6.9590e-02, 5.7925e-02,
    4.8136e-02, 3.9931e-02, 3.3061e-02, 2.7315e-02, 2.2515e-02, 1.8512e-02, 1.5177e-02, 1.2403e-02, 1.0101e-02, 8.1924e-03,
    6.6143e-03, 5.3120e-03, 4.2400e-03, 3.3599e-03, 2.6396e-03, 2.0520e-03, 1.5746e-03, 1.1882e-03, 8.7713e-04, 6.2810e-04,
    4.3007e-04, 2.7384e-04, 2.3714e-04, 2.0535e-04, 1.7783e-04, 1.5399e-04, 1.3335e-04, 1.1548e-04, 1.0000e-04, 8.6596e-05,
    7.4989e-05, 6.4938e-05, 5.6234e-05, 4.8697e-05, 4.2170e-05, 3.6517e-05, 3.1623e-05, 2.7384e-05, 2.3714e-05, 2.0535e-05,
    1.7783e-05, 1.5399e-05, 1.3335e-05, 1.1548e-05]
LLAMA3_SNAPSHOT = [  # :372-389: the same, original context 2048, low 1, high 4, factor 10
    1.0000e+00, 8.6596e-01, 7.4989e-01, 6.4938e-01, 5.6234e-01, 4.8697e-01, 4.2170e-01, 3.6517e-01, 3.1623e-01, 2.7384e-01,
    2.3714e-01, 2.0535e-01, 1.7783e-01, 1.5399e-01, 1.3335e-01, 1.1548e-01, 1.0000e-01, 8.6596e-02, 7.4989e-02, 6.4938e-02,
    5.6234e-02, 4.8697e-02, 4.2170e-02, 3.6517e-02, 3.1623e-02, 2.7384e-02, 2.3714e-02, 2.0535e-02, 1.7783e-02, 1.5399e-02,
    1.3335e-02, 1.0730e-02, 7.7785e-03, 5.6009e-03, 3.9991e-03, 2.8248e-03, 1.9675e-03, 1.3449e-03, 8.9549e-04, 5.7363e-04,
    3.4539e-04, 2.7384e-04, 2.3714e-04, 2.0535e-04, 1.7783e-04, 1.5399e-04, 1.3335e-04, 1.1548e-04, 1.0000e-04, 8.6596e-05,
    7.4989e-05, 6.4938e-05, 5.6234e-05, 4.8697e-05, 4.2170e-05, 3.6517e-05, 3.1623e-05, 2.7384e-05, 2.3714e-05, 2.0535e-05,
    1.7783e-05, 1.5399e-05, 1.3335e-05, 1.1548e-05]


def test_yarn_and_llama3_frequencies_against_the_reference_snapshots():
    """The plain tables and the engine's, both against the vectors the reference's tests hold, and the factor on
    cosines and sines that yarn asks for (tests/utils/test_modeling_rope_utils.py:262-272, :401-412)."""
    from pytorch_transformers_amd.parts.positions import llama3_frequencies, yarn_frequencies

    base = dict(hidden_size=4096, num_attention_heads=32, rope_theta=10000.0, max_position_embeddings=2048)
    yarn = {"rope_type": "yarn", "factor": 10.0, "beta_fast": 32, "beta_slow": 1}
    l3 = {"rope_type": "llama3", "factor": 10.0, "original_max_position_embeddings": 2048, "low_freq_factor": 1,
          "high_freq_factor": 4}
    inv, scale = P.rope_parameters(dict(base, rope_scaling=yarn))
    torch.testing.assert_close(inv, torch.tensor(YARN_SNAPSHOT), rtol=2e-4, atol=0)
    assert scale == 0.1 * math.log(10.0) + 1.0
    assert P.rope_parameters(dict(base, rope_scaling=dict(yarn, attention_factor=0.5)))[1] == 0.5
    got, got_scale = yarn_frequencies(128, 10000.0, 10.0, 2048)
    torch.testing.assert_close(got, inv, rtol=1e-6, atol=0)
    assert got_scale == scale and yarn_frequencies(128, 10000.0, 10.0, 2048, attention_factor=0.5)[1] == 0.5
    inv, scale = P.rope_parameters(dict(base, rope_scaling=l3))
    torch.testing.assert_close(inv, torch.tensor(LLAMA3_SNAPSHOT), rtol=2e-4, atol=0)
    assert scale == 1.0
    torch.testing.assert_close(llama3_frequencies(128, 10000.0, 10.0, 1, 4, 2048), inv, rtol=1e-6, atol=0)
    # every frequency lies between the trained one and the trained one divided by the factor (:279-287, :420-430)
    plain = P.rope_inv_freq(128, 10000.0)
    for table in (torch.tensor(YARN_SNAPSHOT), torch.tensor(LLAMA3_SNAPSHOT)):
        assert bool(((table <= plain * (1 + 2e-4)) & (table >= plain / 10.0 * (1 - 2e-4))).all())
    # a very large beta_fast leaves only the first frequency as trained (:289-298)
    inv, _ = P.rope_parameters(dict(base, rope_scaling=dict(yarn, beta_fast=1000)))
    assert float(inv[0]) == 1.0 and bool((inv[1:] < plain[1:]).all())
    torch.testing.assert_close(inv[-20:], plain[-20:] / 10.0)


DYNAMIC_SNAPSHOT = [  # tests/utils/test_modeling_rope_utils.py:184-199: d=128, theta=1e4, context 2048, factor 10, length 16384
    1.0000e+00, 8.0931e-01, 6.5498e-01, 5.3008e-01, 4.2900e-01, 3.4720e-01, 2.8099e-01, 2.2741e-01, 1.8404e-01, 1.4895e-01,
    1.2055e-01, 9.7558e-02, 7.8955e-02, 6.3899e-02, 5.1714e-02, 4.1853e-02, 3.3872e-02, 2.7413e-02, 2.2185e-02, 1.7955e-02,
    1.4531e-02, 1.1760e-02, 9.5176e-03, 7.7027e-03, 6.2339e-03, 5.0451e-03, 4.0831e-03, 3.3045e-03, 2.6744e-03, 2.1644e-03,
    1.7517e-03, 1.4176e-03, 1.1473e-03, 9.2852e-04, 7.5146e-04, 6.0817e-04, 4.9220e-04, 3.9834e-04, 3.2238e-04, 2.6091e-04,
    2.1115e-04, 1.7089e-04, 1.3830e-04, 1.1193e-04, 9.0585e-05, 7.3312e-05, 5.9332e-05, 4.8018e-05, 3.8861e-05, 3.1451e-05,
    2.5453e-05, 2.0600e-05, 1.6672e-05, 1.3492e-05, 1.0920e-05, 8.8374e-06, 7.1522e-06, 5.7883e-06, 4.6845e-06, 3.7912e-06,
    3.0683e-06, 2.4832e-06, 2.0097e-06, 1.6265e-06]


def test_dynamic_and_longrope_frequencies_against_the_references_tests():
    """Dynamic NTK: the trained table up to the trained context whatever the factor, the reference's snapshot beyond
    it, no plain division by the factor (tests/utils/test_modeling_rope_utils.py:201-225).  LongRoPE: the short
    factors divide the trained table, and the factor on cosines and sines has the paper's default
    (:300-365); fails for the long factors, a missing logarithm or the wrong context length in it."""
    from pytorch_transformers_amd.parts.positions import longrope_frequencies

    base = dict(hidden_size=4096, num_attention_heads=32, rope_theta=10000.0, max_position_embeddings=2048)
    plain = P.rope_inv_freq(128, 10000.0)
    for factor in (2.0, 10.0, 20.0):
        c = dict(base, rope_scaling={"rope_type": "dynamic", "factor": factor})
        for n in (None, 1, 2048):
            inv, scale = P.rope_parameters(c, n)
            assert scale == 1.0
            torch.testing.assert_close(inv, plain)
    inv, _ = P.rope_parameters(dict(base, rope_scaling={"rope_type": "dynamic", "factor": 10.0}), 16384)
    torch.testing.assert_close(inv, torch.tensor(DYNAMIC_SNAPSHOT), rtol=2e-4, atol=0)
    assert not torch.allclose(inv, plain / 10.0, rtol=1e-3)
    assert bool((inv <= plain).all())  # tests/models/falcon/test_modeling_falcon.py:503
    # cosines of a short range are the trained ones, of a long range not (:493-502 there)
    c10 = dict(base, rope_scaling={"type": "dynamic", "factor": 10.0})
    cs_short, _ = P.rope_cos_sin(torch.arange(10), P.rope_parameters(c10, 10)[0])
    cs_plain, _ = P.rope_cos_sin(torch.arange(10), plain)
    torch.testing.assert_close(cs_short, cs_plain)
    cs_long, _ = P.rope_cos_sin(torch.arange(3072), P.rope_parameters(c10, 3072)[0])
    assert not torch.allclose(cs_long, P.rope_cos_sin(torch.arange(3072), plain)[0], atol=1e-3)

    short, long_ = [2.0] * 64, [float(i + 1) for i in range(64)]
    for factor in (2.0, 10.0, 20.0):
        rs = {"rope_type": "longrope", "factor": factor, "short_factor": short, "long_factor": long_}
        inv, scale = P.rope_parameters(dict(base, rope_scaling=rs))
        assert scale == math.sqrt(1 + math.log(factor) / math.log(2048))
        torch.testing.assert_close(inv, plain / 2.0)
        assert P.rope_parameters(dict(base, rope_scaling=dict(rs, attention_factor=0.5)))[1] == 0.5
        got, got_scale = longrope_frequencies(128, 10000.0, short, factor, 2048)
        torch.testing.assert_close(got, inv, rtol=1e-6, atol=0)
        assert got_scale == scale and longrope_frequencies(128, 10000.0, short, factor, 2048, attention_factor=0.5)[1] == 0.5
    rs = {"rope_type": "longrope", "factor": 1.0, "short_factor": short, "long_factor": long_}
    assert P.rope_parameters(dict(base, rope_scaling=rs))[1] == 1.0
    # a configuration that names the trained context takes the ratio of the two lengths as its factor
    c = dict(base, max_position_embeddings=8192, original_max_position_embeddings=2048,
             rope_scaling={"rope_type": "longrope", "short_factor": short, "long_factor": long_})
    assert P.rope_parameters(c)[1] == math.sqrt(1 + math.log(4.0) / math.log(2048))
    assert longrope_frequencies(128, 10000.0, short, None, 8192, 2048)[1] == P.rope_parameters(c)[1]


def test_dynamic_frequencies_in_the_model(models_dynamic):
    """Falcon's own test of scaling from the configuration (tests/models/falcon/test_modeling_falcon.py:424-455):
    up to the trained context a model with dynamic scaling gives what it gives without, beyond it not; and fed in
    pieces, every piece is rotated by the table of the length reached with it, earlier pieces staying as they were."""
    cfg, w = models_dynamic
    unscaled = dict(cfg, rope_scaling=None)
    ctx = cfg["max_position_embeddings"]
    short = [(5 * i + 1) % cfg["vocab_size"] for i in range(ctx)]
    long_ = [(3 * i + 2) % cfg["vocab_size"] for i in range(ctx + ctx // 2)]
    torch.testing.assert_close(P.forward(cfg, w, short), P.forward(unscaled, w, short))
    whole = P.forward(cfg, w, long_)
    assert not torch.allclose(whole, P.forward(unscaled, w, long_), atol=1e-5)
    # the first `ctx` tokens as one piece, then one token at a time
    lens = [ctx] * ctx + list(range(ctx + 1, len(long_) + 1))
    pieces = P.forward(cfg, w, long_, seq_lens=lens)
    torch.testing.assert_close(pieces[:ctx], P.forward(unscaled, w, long_[:ctx]))  # nothing was scaled yet
    assert not torch.allclose(pieces[ctx:], whole[ctx:], atol=1e-5)  # the prompt's keys kept their rotation
    torch.testing.assert_close(P.forward(cfg, w, long_, seq_lens=[len(long_)] * len(long_)), whole)


def test_rope_hand_case_pairs_and_sign():
    """Pairs are (i, i + d/2), not (2i, 2i+1); the lower half gets -sin.  d=4, position 1."""
    x = torch.tensor([[[1.0, 2.0, 3.0, 4.0]]], dtype=D)
    inv = torch.tensor([1.0, 0.5])
    cos, sin = P.rope_cos_sin(torch.tensor([1]), inv)
    out = P.apply_rope(x, cos, sin)[0, 0]
    c0, s0, c1, s1 = math.cos(1.0), math.sin(1.0), math.cos(0.5), math.sin(0.5)
    want = torch.tensor([1 * c0 - 3 * s0, 2 * c1 - 4 * s1, 3 * c0 + 1 * s0, 4 * c1 + 2 * s1], dtype=D)
    torch.testing.assert_close(out, want, rtol=1e-6, atol=1e-7)


def test_rope_is_a_complex_multiplication_of_half_split_pairs():
    """An independent spelling: z_i = x[i] + j x[i + d/2] times e^{j pos inv_freq[i]}.  Fails for a flipped sign
    of the sine (the conjugate rotation) and for interleaved pairs (2i, 2i + 1)."""
    d, T = 16, 5
    x = rnd(T, 3, d)
    inv = P.rope_inv_freq(d, 10000.0)
    pos = torch.tensor([0, 1, 7, 30, 200])
    cos, sin = P.rope_cos_sin(pos, inv)
    got = P.apply_rope(x, cos, sin)
    ang = pos.float()[:, None] * inv[None, :]  # 32-bit angles, as the reference forms them
    turn = torch.complex(torch.cos(ang).double(), torch.sin(ang).double())[:, None, :]
    z = torch.complex(x[..., :d // 2], x[..., d // 2:]) * turn
    torch.testing.assert_close(got, torch.cat((z.real, z.imag), dim=-1), rtol=1e-9, atol=1e-12)
    z_conj = torch.complex(x[..., :d // 2], x[..., d // 2:]) * turn.conj()
    assert not torch.allclose(got[1:], torch.cat((z_conj.real, z_conj.imag), dim=-1)[1:], atol=1e-3)
    zi = torch.complex(x[..., 0::2], x[..., 1::2]) * turn  # the interleaved convention, which this is not
    inter = torch.stack((zi.real, zi.imag), dim=-1).reshape(T, 3, d)
    assert not torch.allclose(got[1:], inter[1:], atol=1e-3)
    torch.testing.assert_close(got[0], x[0])


def test_rope_invariants():
    """Position 0 is the identity; pair norms are kept; <R_m q, R_n k> depends on m - n only; the
    cos/sin of a short range are the prefix of a long one (tests/models/falcon/test_modeling_falcon.py:470-475);
    linear scaling by f maps position x to x / f (:485-488)."""
    d = 32
    inv = P.rope_inv_freq(d, 10000.0)
    q, k = rnd(1, 3, d), rnd(1, 3, d, seed=1)
    c0, s0 = P.rope_cos_sin(torch.tensor([0]), inv)
    torch.testing.assert_close(P.apply_rope(q, c0, s0), q)
    pos = torch.tensor([0, 3, 4, 10, 11, 17])
    cos, sin = P.rope_cos_sin(pos, inv)
    qq = P.apply_rope(q.expand(6, 3, d), cos, sin)
    kk = P.apply_rope(k.expand(6, 3, d), cos, sin)
    pair_norm = lambda t: t[..., :d // 2] ** 2 + t[..., d // 2:] ** 2
    torch.testing.assert_close(pair_norm(qq), pair_norm(q.expand(6, 3, d)), rtol=1e-6, atol=1e-9)
    dot = lambda a, b: float((qq[a, 0] * kk[b, 0]).sum())
    assert abs(dot(2, 1) - dot(4, 3)) < 1e-5 and abs(dot(3, 1) - dot(5, 3)) < 1e-5  # distances 1 and 7
    assert abs(dot(2, 1) - dot(1, 2)) > 1e-3  # ... and the sign of the distance matters
    cl, sl = P.rope_cos_sin(torch.arange(40), inv)
    cs, ss = P.rope_cos_sin(torch.arange(9), inv)
    assert torch.equal(cl[:9], cs) and torch.equal(sl[:9], ss)
    c2, s2 = P.rope_cos_sin(torch.tensor([10]), P.rope_inv_freq(d, 10000.0, 2.0))
    c1, s1 = P.rope_cos_sin(torch.tensor([5]), inv)
    torch.testing.assert_close(c2, c1, rtol=1e-6, atol=1e-7)
    torch.testing.assert_close(s2, s1, rtol=1e-6, atol=1e-7)


# --- ALiBi -----------------------------------------------------------------------------------
def test_alibi_slopes():
    """Power-of-two head counts: 2^(-8(i+1)/n).  Six heads: the four of n=4, then odd powers of the
    n=8 base.  Fails for a wrong base or for taking the extra slopes at even powers."""
    for n in (4, 8, 16):
        torch.testing.assert_close(P.alibi_slopes(n), torch.tensor([2.0 ** (-8.0 * (i + 1) / n) for i in range(n)]))
    torch.testing.assert_close(P.alibi_slopes(6), torch.tensor([1 / 4, 1 / 16, 1 / 64, 1 / 256, 1 / 2, 1 / 8]))
    s20 = P.alibi_slopes(20)
    torch.testing.assert_close(s20[16:], torch.tensor([2.0 ** (-0.25 * p) for p in (1, 3, 5, 7)]))


def test_alibi_bias_is_rounded_like_the_reference():
    """slope x position is formed in bfloat16 (modeling_falcon.py:196-198): exact for 6 heads at
    small positions, visibly rounded for 20 heads and for positions past 256."""
    b6 = P.alibi_bias(6, 10, 24)
    torch.testing.assert_close(b6[4], torch.arange(10, dtype=D) * 0.5 / math.sqrt(24))
    b20 = P.alibi_bias(20, 400, 16)
    exact = P.alibi_slopes(20).double()[:, None] * torch.arange(400, dtype=D)[None, :] / 4.0
    assert float((b20 - exact).abs().max()) > 1e-3
    s_bf = P.alibi_slopes(20).bfloat16().double()
    p_bf = torch.arange(400).bfloat16().double()
    prod = (s_bf[:, None] * p_bf[None, :]).bfloat16().double()  # each product has <= 16 significant bits: exact in float64
    torch.testing.assert_close(b20, prod / 4.0)
    assert float(p_bf[301]) != 301.0  # positions past 256 are themselves rounded


def test_alibi_key_bias_equals_relative_bias():
    """Softmax ignores a per-query constant: slope*j == -slope*(t - j).  Zero slopes: no positions."""
    T, d = 7, 8
    q, k, v = rnd(T, 1, d), rnd(T, 1, d, seed=1), rnd(T, 1, d, seed=2)
    slope = 0.3
    key_bias = (slope * torch.arange(T, dtype=D))[None, :]
    out_key = P.attention_scores_softmax(q, k, v, key_bias)
    rel = torch.stack([-slope * (t - torch.arange(T, dtype=D)) for t in range(T)])  # [T, T]
    s = (q[:, 0] @ k[:, 0].T) / math.sqrt(d) + rel + torch.full((T, T), float("-inf"), dtype=D).triu(1)
    torch.testing.assert_close(out_key, torch.softmax(s, -1) @ v[:, 0])
    torch.testing.assert_close(P.attention_scores_softmax(q, k, v, torch.zeros(1, T, dtype=D)),
                               P.attention_scores_softmax(q, k, v, None))


# --- fused projection layouts, attention ---------------------------------------------------------
def _cfg(**kw):
    return P.cfg_defaults(dict(kw))


def test_split_heads_three_layouts():
    """Hand-indexed rows for each order; fails if k and v are swapped or groups are interleaved wrongly."""
    T, d = 3, 4
    # grouped: 6 heads in 2 groups of 3: [q0 q1 q2 k0 v0 | q3 q4 q5 k1 v1]
    c = _cfg(hidden_size=24, num_attention_heads=6, num_kv_heads=2, new_decoder_architecture=True)
    fused = torch.arange(T * 10 * d, dtype=D).view(T, 10 * d)
    q, k, v = P.split_heads(fused, c)
    blocks = fused.view(T, 10, d)
    assert torch.equal(q, blocks[:, [0, 1, 2, 5, 6, 7]]) and torch.equal(k, blocks[:, [3, 8]]) and torch.equal(v, blocks[:, [4, 9]])
    # tail: [q0..q5 k v]
    c = _cfg(hidden_size=24, num_attention_heads=6, multi_query=True)
    fused = torch.arange(T * 8 * d, dtype=D).view(T, 8 * d)
    q, k, v = P.split_heads(fused, c)
    blocks = fused.view(T, 8, d)
    assert torch.equal(q, blocks[:, :6]) and torch.equal(k, blocks[:, [6]]) and torch.equal(v, blocks[:, [7]])
    # interleaved: [q0 k0 v0 q1 k1 v1 ...]
    c = _cfg(hidden_size=24, num_attention_heads=6, multi_query=False)
    fused = torch.arange(T * 18 * d, dtype=D).view(T, 18 * d)
    q, k, v = P.split_heads(fused, c)
    blocks = fused.view(T, 18, d)
    assert torch.equal(q, blocks[:, 0::3]) and torch.equal(k, blocks[:, 1::3]) and torch.equal(v, blocks[:, 2::3])


def test_attention_is_sdpa_and_groups_are_repeated_heads():
    """No rotation, no bias: one sequence equals torch's scaled_dot_product_attention(is_causal=True);
    grouped KV equals full heads on repeated keys and values (modeling_falcon.py:286-289)."""
    T, nh, nkv, d = 9, 6, 2, 8
    q, k, v = rnd(T, nh, d), rnd(T, nkv, d, seed=1), rnd(T, nkv, d, seed=2)
    out = P.attention_scores_softmax(q, k, v)
    kr, vr = k.repeat_interleave(nh // nkv, 1), v.repeat_interleave(nh // nkv, 1)
    ref = F.scaled_dot_product_attention(q.transpose(0, 1)[None], kr.transpose(0, 1)[None], vr.transpose(0, 1)[None],
                                         is_causal=True)[0].transpose(0, 1).reshape(T, nh * d)
    torch.testing.assert_close(out, ref)
    torch.testing.assert_close(P.attention_scores_softmax(q, kr, vr), out)
    # one token: the output is its value; equal keys: the running mean of values
    torch.testing.assert_close(P.attention_scores_softmax(q[:1], k[:1], v[:1]).view(nh, d), vr[0])
    same_k = k[:1].expand(T, nkv, d)
    mean = torch.cumsum(vr, 0) / torch.arange(1, T + 1, dtype=D)[:, None, None]
    torch.testing.assert_close(P.attention_scores_softmax(q, same_k, v), mean.reshape(T, nh * d))


# --- the whole model ----------------------------------------------------------------------------
@pytest.fixture(scope="module")
def models(tmp_path_factory):
    root = str(tmp_path_factory.mktemp("plain"))
    return {n: P.read_model(write_model(n, root)) for n in TINY}


@pytest.fixture(scope="module")
def models_dynamic(tmp_path_factory):
    from tiny import DYNAMIC, write_config

    return P.read_model(write_config(DYNAMIC, str(tmp_path_factory.mktemp("plain-dyn")), "dyn", seed=6))


@pytest.mark.parametrize("name", sorted(TINY))
def test_causality_and_prefix(models, name):
    """Logits at a position do not change with later tokens; fails for a mask off by one."""
    cfg, w = models[name]
    ids = [(7 * i + 3) % cfg["vocab_size"] for i in range(20)]
    full = P.forward(cfg, w, ids)
    torch.testing.assert_close(P.forward(cfg, w, ids[:11]), full[:11], rtol=1e-9, atol=1e-9)
    changed = list(ids)
    changed[15] = (changed[15] + 1) % cfg["vocab_size"]
    other = P.forward(cfg, w, changed)
    torch.testing.assert_close(other[:15], full[:15], rtol=1e-9, atol=1e-9)
    assert not torch.allclose(other[15:], full[15:], atol=1e-6)
    assert full.shape == (20, cfg["vocab_size"])


def test_residual_arrangements(models):
    """Parallel block with the feed-forward's output matrix zeroed is x + attention; with the
    attention's output matrix zeroed it is x + feed-forward (fails for a norm in the wrong branch)."""
    cfg, w = models["C"]
    c = P.cfg_defaults(cfg)
    x = rnd(6, c["hidden_size"])
    pos = torch.arange(6)
    p = "transformer.h.0."
    ln = P.layer_norm(x, w[p + "input_layernorm.weight"], w[p + "input_layernorm.bias"], c["layer_norm_epsilon"])
    attn = P.self_attention(ln, w, p + "self_attention.", c, pos)
    w0 = dict(w); w0[p + "mlp.dense_4h_to_h.weight"] = torch.zeros_like(w[p + "mlp.dense_4h_to_h.weight"])
    torch.testing.assert_close(P.decoder_layer(x, w0, 0, c, pos), x + attn)
    w1 = dict(w); w1[p + "self_attention.dense.weight"] = torch.zeros_like(w[p + "self_attention.dense.weight"])
    torch.testing.assert_close(P.decoder_layer(x, w1, 0, c, pos), x + P.mlp(ln, w, p + "mlp."))
    # sequential (B): the feed-forward reads the norm of x + attention, with the second norm's parameters
    cfg, w = models["B"]
    c = P.cfg_defaults(cfg)
    x = rnd(5, c["hidden_size"])
    pos = torch.arange(5)
    a = P.self_attention(P.layer_norm(x, w[p + "input_layernorm.weight"], w[p + "input_layernorm.bias"], 1e-6), w,
                         p + "self_attention.", c, pos)
    r = x + a
    want = r + P.mlp(P.layer_norm(r, w[p + "post_attention_layernorm.weight"], w[p + "post_attention_layernorm.bias"], 1e-6),
                     w, p + "mlp.")
    torch.testing.assert_close(P.decoder_layer(x, w, 0, c, pos), want)


def test_sequential_block_by_special_cases(models):
    """The sequential arrangement (modeling_falcon.py:652-659, :676) pinned without recomputing it the same way:
    a silent attention (output matrix and bias zero) leaves x + mlp(post_norm(x)); a silent feed-forward leaves
    x + attention(input_norm(x)), with no trace of the second norm; and the two norms are not interchangeable
    (fails for a post norm applied to x instead of x + attention, or for the norms swapped)."""
    cfg, w = models["B"]
    c = P.cfg_defaults(cfg)
    assert not c["parallel_attn"] and not c["new_decoder_architecture"]
    p = "transformer.h.1."
    eps = c["layer_norm_epsilon"]
    x = rnd(7, c["hidden_size"], seed=5)
    pos = torch.arange(7)
    ln_in = lambda t, ww=w: P.layer_norm(t, ww[p + "input_layernorm.weight"], ww[p + "input_layernorm.bias"], eps)
    ln_post = lambda t, ww=w: P.layer_norm(t, ww[p + "post_attention_layernorm.weight"], ww[p + "post_attention_layernorm.bias"], eps)

    def silenced(*names):
        out = dict(w)
        for n in names:
            out[p + n] = torch.zeros_like(w[p + n])
        return out

    no_attn = silenced("self_attention.dense.weight", "self_attention.dense.bias")
    torch.testing.assert_close(P.decoder_layer(x, no_attn, 1, c, pos), x + P.mlp(ln_post(x), w, p + "mlp."))
    no_ffn = silenced("mlp.dense_4h_to_h.weight", "mlp.dense_4h_to_h.bias")
    attn = P.self_attention(ln_in(x), w, p + "self_attention.", c, pos)
    torch.testing.assert_close(P.decoder_layer(x, no_ffn, 1, c, pos), x + attn)
    changed = dict(no_ffn)  # ... whatever the second norm holds
    changed[p + "post_attention_layernorm.weight"] = w[p + "post_attention_layernorm.weight"] * 3 + 1
    torch.testing.assert_close(P.decoder_layer(x, changed, 1, c, pos), x + attn)
    # the feed-forward reads the norm of x + attention: with attention on, the result is not
    # x + attention + mlp(post_norm(x)) ...
    full = P.decoder_layer(x, w, 1, c, pos)
    assert not torch.allclose(full, x + attn + P.mlp(ln_post(x), w, p + "mlp."), atol=1e-6)
    torch.testing.assert_close(full, (x + attn) + P.mlp(ln_post(x + attn), w, p + "mlp."))
    # ... and swapping the two norms' parameters changes it
    swapped = dict(w)
    for s_ in ("weight", "bias"):
        swapped[p + "input_layernorm." + s_] = w[p + "post_attention_layernorm." + s_]
        swapped[p + "post_attention_layernorm." + s_] = w[p + "input_layernorm." + s_]
    assert not torch.allclose(P.decoder_layer(x, swapped, 1, c, pos), full, atol=1e-6)


def test_two_equal_norms_are_one_norm(models):
    """New architecture with ln_attn == ln_mlp equals the one-norm variant with that norm."""
    cfg, w = models["A"]
    w2 = dict(w)
    for i in range(cfg["num_hidden_layers"]):
        for s in ("weight", "bias"):
            w2[f"transformer.h.{i}.ln_mlp.{s}"] = w[f"transformer.h.{i}.ln_attn.{s}"]
            w2[f"transformer.h.{i}.input_layernorm.{s}"] = w[f"transformer.h.{i}.ln_attn.{s}"]
    ids = list(range(3, 15))
    one = dict(cfg, num_ln_in_parallel_attn=1)
    torch.testing.assert_close(P.forward(cfg, w2, ids), P.forward(one, w2, ids))
    assert not torch.allclose(P.forward(cfg, w, ids), P.forward(cfg, w2, ids), atol=1e-6)


def test_tied_head(models):
    cfg, w = models["A"]
    ids = list(range(10))
    untied = dict(w); untied["lm_head.weight"] = w["transformer.word_embeddings.weight"].clone()
    torch.testing.assert_close(P.forward(cfg, w, ids), P.forward(dict(cfg, tie_word_embeddings=False), untied, ids))


# --- processors and the choice -----------------------------------------------------------------------
def test_processors_on_the_references_vectors():
    """tests/generation/test_logits_process.py: :183-205 penalty, :235-271 top-k, :273-309 top-p, :311-355 min-p."""
    s = torch.full((10,), 0.1); s[0] = -0.1
    out = P.repetition_penalty(s, [0, 1], 2.0)
    assert abs(float(out[0]) + 0.2) < 1e-7 and abs(float(out[1]) - 0.05) < 1e-7 and float(out[2]) == pytest.approx(0.1)
    s = torch.full((10,), 0.1); s[5] = 0.4
    out = P.repetition_penalty(s, [5, 0], 2.0)
    assert float(out[0]) == pytest.approx(0.05) and float(out[5]) == pytest.approx(0.2)
    assert float(s[5]) == pytest.approx(0.4)  # inputs are not changed in place

    ramp = torch.arange(10.0)
    assert torch.isinf(P.top_k(ramp, 3)).tolist() == 7 * [True] + 3 * [False]
    ramp2 = ramp.clone(); ramp2[:5] += 10
    assert torch.isinf(P.top_k(ramp2, 3)).tolist() == 2 * [True] + 3 * [False] + 5 * [True]
    assert int(torch.isinf(P.top_k(torch.arange(5.0), 1, min_tokens_to_keep=3)).sum()) == 2

    dist = torch.log(torch.tensor([[0.3, 0.1, 0.1, 0.5], [0.15, 0.3, 0.3, 0.25]]))
    torch.testing.assert_close(torch.exp(P.top_p(dist[1], 0.8)), torch.tensor([0.0, 0.3, 0.3, 0.25]), atol=1e-3, rtol=0)
    torch.testing.assert_close(torch.exp(P.top_p(dist[0], 0.79)), torch.tensor([0.3, 0.0, 0.0, 0.5]), atol=1e-3, rtol=0)
    # of two equal scores at the cut, the first in ascending stable order goes
    torch.testing.assert_close(torch.exp(P.top_p(dist[0], 0.85)), torch.tensor([0.3, 0.0, 0.1, 0.5]), atol=1e-3, rtol=0)
    ramp = torch.arange(10.0) - 5
    assert int((P.top_p(ramp, 0.9, min_tokens_to_keep=2) != float("-inf")).sum()) == 3
    assert int((P.top_p(ramp * 100, 0.9, min_tokens_to_keep=2) != float("-inf")).sum()) == 2

    dist = torch.log(torch.tensor([[0.9, 0.0274, 0.047, 0.0274], [0.15, 0.3, 0.3, 0.25], [0.97, 0.01, 0.01, 0.01]]))
    want = torch.tensor([[0.9, 0.0, 0.047, 0.0], [0.15, 0.3, 0.3, 0.25], [0.97, 0.0, 0.0, 0.0]])
    for r in range(3):
        torch.testing.assert_close(torch.exp(P.min_p(dist[r], 0.05)), want[r], atol=1e-3, rtol=0)
    assert int((P.min_p(ramp, 0.9, min_tokens_to_keep=2) != float("-inf")).sum()) == 2

    # typical-p, epsilon and eta cut-offs (:357-378, :405-428, :445-468)
    dist = torch.log(torch.tensor([[0.97, 0.01, 0.01, 0.01], [0.4, 0.2, 0.2, 0.2]]))
    want = torch.tensor([[0.97, 0.0, 0.0, 0.0], [0.0, 0.2, 0.2, 0.2]])  # the likeliest token is not the typical one
    for r in range(2):
        torch.testing.assert_close(torch.exp(P.typical_p(dist[r], 0.5)), want[r], atol=1e-3, rtol=0)
    dist = torch.log(torch.tensor([[0.87, 0.099, 0.001, 0.03], [0.4, 0.299, 0.101, 0.2]]))
    want = torch.tensor([[0.87, 0.0, 0.0, 0.0], [0.4, 0.299, 0.101, 0.2]])
    for r in range(2):
        torch.testing.assert_close(torch.exp(P.epsilon_cutoff(dist[r], 0.1)), want[r], atol=1e-3, rtol=0)
    dist = torch.log(torch.tensor([[0.0, 0.1, 0.8, 0.1], [0.01, 0.04, 0.9, 0.05]]))
    want = torch.tensor([[0.0, 0.1, 0.8, 0.1], [0.0, 0.0, 0.9, 0.0]])
    for r in range(2):
        torch.testing.assert_close(torch.exp(P.eta_cutoff(dist[r], 0.0625)), want[r], atol=1e-3, rtol=0)

    # no-repeat n-grams and bad words (:485-508, :576-601)
    flat = torch.zeros(3)
    for ids, n, gone in (([1, 1, 2, 1], 2, [False, True, True]), ([0, 1, 0, 1], 2, [True, False, False]),
                         ([1, 1, 2, 1], 3, [False, False, False]), ([0, 1, 0, 1], 3, [True, False, False])):
        assert torch.isinf(P.no_repeat_ngram(flat, ids, n)).tolist() == gone
    words = [[1], [4], [1, 0], [0, 1, 2], [1, 3, 1, 3]]
    assert torch.isinf(P.no_bad_words(torch.zeros(5), [0, 1, 3, 1], words, eos_ids=[4])).tolist() == [True, True, False, True, False]
    assert torch.isinf(P.no_bad_words(torch.zeros(5), [0, 1, 0, 1], words, eos_ids=[4])).tolist() == [True, True, True, False, False]

    # temperature (:148-181): uniform stays uniform, peaks sharpen below 1 and flatten above
    s = torch.full((20,), 0.05); s[5] = 0.15; s[10] = -0.35
    p, sharp, smooth = (torch.softmax(t, -1) for t in (s, P.temperature(s, 0.5), P.temperature(s, 1.3)))
    assert sharp.max() > p.max() > smooth.max() and sharp.min() < p.min() < smooth.min()

    assert torch.isinf(P.suppress(torch.zeros(6), [2, 4])).tolist() == [False, False, True, False, True, False]


def test_bias_forced_token_and_bonus_on_eos_on_the_references_vectors():
    """tests/generation/test_logits_process.py: :604-629 sequence bias, :766-791 forced last token, :820-855 the bonus
    on EOS that grows with the length."""
    entries = {(1,): 100.0, (4,): 100.0, (1, 0): -100.0, (0, 1, 2): -100.0, (1, 3, 1, 3): -100.0,
               (1, 3, 1, 3, 1, 3): -100.0}
    flat = torch.zeros(5)
    assert P.sequence_bias(flat, [0, 1, 3, 1], entries).tolist() == [-100.0, 100.0, 0.0, -100.0, 100.0]
    assert P.sequence_bias(flat, [0, 1, 0, 1], entries).tolist() == [-100.0, 100.0, -100.0, 0.0, 100.0]
    assert flat.abs().sum() == 0  # inputs are not changed in place
    # two entries that end in one token add up; a one-token entry adds to whatever else the token gets
    both = {(3, 1): 1.5, (2, 3, 1): 2.0, (1,): 0.25}
    assert P.sequence_bias(flat, [9, 2, 3], both).tolist() == [0, 3.75, 0, 0, 0]
    # an entry longer than the ids so far never applies, although the ids end in the tokens before its last (:1122)
    assert P.sequence_bias(flat, [2, 3], both).tolist() == [0, 1.75, 0, 0, 0]
    assert not torch.isinf(P.no_bad_words(flat, [2, 3], [[2, 3, 1]])).any()
    assert torch.isinf(P.no_bad_words(flat, [9, 2, 3], [[2, 3, 1]])).tolist() == [False, True, False, False, False]

    uniform = torch.full((20,), 1.0 / 20)
    forced = P.forced_eos(uniform, 4, 5, [0])
    assert float(forced[0]) == 0 and torch.isneginf(forced[1:]).all()
    assert torch.equal(P.forced_eos(uniform, 3, 5, [0]), uniform)

    # a prompt of 2 ids, start index 5, factor 1.1: nothing up to 7 ids, then |score| * (1.1 ** (ids - 7) - 1) on top
    assert torch.equal(P.exponential_decay(uniform, 2, 2, 5, 1.1, [0]), uniform)
    assert torch.equal(P.exponential_decay(uniform, 7, 2, 5, 1.1, [0]), uniform)
    after = P.exponential_decay(uniform, 20, 2, 5, 1.1, [0])
    assert float(after[0]) == pytest.approx(0.05 * 1.1 ** 13) and torch.equal(after[1:], uniform[1:])
    negative = P.exponential_decay(-uniform, 20, 2, 5, 1.1, [0])
    assert float(negative[0]) == pytest.approx(-0.05 + 0.05 * (1.1 ** 13 - 1)) and float(negative[0]) > -0.05

    # their places in the order (generation/utils.py:898-1005): the bias before the penalty, the forced token over
    # everything before it, the bonus after it
    s = torch.tensor([2.0, 1.0, -1.0])
    out = P.process(s, [0], do_sample=False, sequence_bias_={(0,): -4.0}, repetition_penalty_=2.0)
    assert out.tolist() == [-4.0, 1.0, -1.0]  # (2 - 4) * 2; the penalty first would have given 2 / 2 - 4 = -3
    out = P.process(s, [0, 1], do_sample=False, forced_eos_=(3, [2]), exponential_decay_=(1, 0, 2.0), eos_ids_=[2],
                    suppress_ids=[2])
    assert out.tolist() == [float("-inf"), float("-inf"), 0.0]  # the forced token undoes the suppression; |0| gains nothing


def test_processing_order_and_pick():
    """Penalty before temperature, top-k before top-p (generation/utils.py:926-1097); argmax and
    inverse-CDF choice."""
    s = torch.tensor([2.0, 1.0, 0.75, -1.0])
    out = P.process(s, [0], do_sample=True, temperature_=0.5, top_k_=2, repetition_penalty_=4.0)
    # 2.0 / 4 = 0.5 falls behind 0.75 before top-k looks; top-k first would have kept token 0
    assert out.tolist() == [float("-inf"), 2.0, 1.5, float("-inf")]
    assert P.pick(s, None) == 0
    probs = torch.softmax(s.double(), -1).cumsum(-1)
    assert P.pick(s, 0.0) == 0 and P.pick(s, float(probs[0]) + 1e-9) == 1 and P.pick(s, 0.999999) == 3
    greedy = P.process(s, [], do_sample=False, temperature_=0.5, top_k_=1)
    assert torch.equal(greedy, s)  # warpers are not applied without sampling


def test_generate_stops_at_eos_and_keeps_it(models):
    cfg, w = models["A"]
    free = P.generate(cfg, w, [1, 2, 3], 8)
    assert len(free) == 8
    eos = free[3]
    first = free.index(eos)
    stopped = P.generate(cfg, w, [1, 2, 3], 8, eos_ids=(eos,))
    assert stopped == free[:first + 1]
    held = P.generate(cfg, w, [1, 2, 3], 8, eos_ids=(eos,), min_new_tokens=first + 2)
    assert len(held) > first + 1 and eos not in held[:first + 2]
