"""Each part alone against the plain functions, and a toy architecture with a state-holding mixer that
is defined here, registered, built and stepped without touching the framework's files (GPU)."""
import dataclasses
import math

import pytest
import torch

import helpers
import plain_falcon as P

pytestmark = pytest.mark.gpu

DTYPES = [(torch.float32, 3e-5), (torch.bfloat16, 3e-2)]


def _rand(*shape, seed=0, scale=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * scale


def _fill(part, dtype, seed=0, std=0.05):
    """Random tensors for a part, as the device would hold them; returns (device dict, float64 dict)."""
    from pytorch_transformers_amd.weights.loader import device_dtype_for
    from pytorch_transformers_amd.weights.random_init import init_tensor

    dev, ref = {}, {}
    for s in part.all_tensor_specs():
        t = init_tensor(s, seed, std, noise=0.2, dtype=torch.bfloat16)
        dev[s.name] = t.to(device_dtype_for(s, dtype)).cuda()
        ref[s.name] = t.double()
    part.load_all(dev)
    return dev, ref


def _ctx(cache, slots, new_tokens, dtype):
    """A StepContext for sequences that bring ``new_tokens`` tokens each (pages reserved, not committed)."""
    import numpy as np

    from pytorch_transformers_amd.engine.step import plan_step
    from pytorch_transformers_amd.parts.base import StepContext

    plan = plan_step(cache, slots, [[0] * n for n in new_tokens], "all", 10)
    i32 = lambda a: torch.as_tensor(np.asarray(a), dtype=torch.int32).cuda()
    return StepContext(dtype=dtype, device=torch.device("cuda:0"), n_seqs=plan.n_seqs, n_tokens=plan.n_tokens,
                       token_seq=i32(plan.token_seq), token_pos=i32(plan.token_pos), cu_tokens=i32(plan.cu_tokens),
                       seq_start=i32(plan.starts), seq_slot=i32(plan.slots),
                       block_tables={g: i32(t) for g, t in plan.block_tables.items()}, cache=cache, slots=plan.slots,
                       new_tokens=plan.new_tokens, starts=plan.starts, is_decode=plan.is_decode, max_len=plan.max_len), plan


def _close(got, want, rel, what):
    got, want = got.double().cpu(), want.double()
    scale = max(1.0, float(want.abs().max()))
    err = float((got - want).abs().max())
    assert err <= rel * scale, f"{what}: max |diff| {err:.3e} > {rel} x {scale:.3e}"


@pytest.mark.parametrize("dtype,rel", DTYPES)
def test_layernorm_linear_embedding_head(dtype, rel):
    from pytorch_transformers_amd.parts import Embedding, LayerNorm, Linear, OutputHead

    H = 200
    x = _rand(9, H).bfloat16()
    ln, ln2 = LayerNorm("n1", H, 1e-5), LayerNorm("n2", H, 1e-5)
    (_, r1), (_, r2) = _fill(ln, dtype, 1), _fill(ln2, dtype, 2)
    want1 = P.layer_norm(x.double(), r1["n1.weight"], r1["n1.bias"], 1e-5)
    _close(ln.forward(x.to(dtype).cuda()), want1, rel, "LayerNorm")
    a, b = ln.forward_pair(x.to(dtype).cuda(), ln2)
    _close(a, want1, rel, "LayerNorm pair, first")
    _close(b, P.layer_norm(x.double(), r2["n2.weight"], r2["n2.bias"], 1e-5), rel, "LayerNorm pair, second")
    rows = torch.tensor([8, 0], dtype=torch.int32).cuda()
    _close(ln.forward(x.to(dtype).cuda(), rows=rows), want1[[8, 0]], rel, "LayerNorm on chosen rows")

    for M in (3, 100):  # few rows: the decode kernel in bfloat16; many: the library product plus epilogue
        x = _rand(M, H, seed=M).bfloat16()
        lin = Linear("lin", H, 72, bias=True)
        _, r = _fill(lin, dtype, 3)
        add = _rand(M, 72, seed=5).bfloat16()
        want = P.gelu(P.linear(x.double(), r["lin.weight"], r["lin.bias"])) + add.double()
        _close(lin(x.to(dtype).cuda(), act="gelu", add1=add.to(dtype).cuda()), want, rel, f"Linear, {M} rows")
        _close(lin(x.to(dtype).cuda(), apply_bias=False), x.double() @ r["lin.weight"].T, rel, "Linear without bias")

    emb = Embedding("emb", 50, H)
    _, r = _fill(emb, dtype, 4)
    ids = torch.tensor([3, 49, 0, 3], dtype=torch.int32).cuda()
    _close(emb.forward(ids), r["emb.weight"][[3, 49, 0, 3]], 0.0, "Embedding")
    head = OutputHead("head", 50, H, tied_to=None)
    _, r = _fill(head, dtype, 5)
    for M in (2, 70):
        h = _rand(M, H, seed=7).bfloat16()
        out = head.forward(h.to(dtype).cuda())
        assert out.dtype == torch.float32
        _close(out, h.double() @ r["head.weight"].T, rel, f"OutputHead, {M} rows")


def test_joined_matrices_give_one_product_for_many_rows(monkeypatch):
    """Two linear layers of one input whose matrices are laid out side by side: a prompt's rows can go through
    one library product; the two results are blocks of columns of its output, each with its own epilogue, and
    what reads them (the next product, the rotation kernel) takes rows that lie apart."""
    from pytorch_transformers_amd import ops
    from pytorch_transformers_amd.parts import Linear

    H, N1, N2, M = 200, 72, 136, 600
    first, second = Linear("a", H, N1, bias=True), Linear("b", H, N2, bias=False)
    (_, r1), (_, r2) = _fill(first, torch.bfloat16, 1), _fill(second, torch.bfloat16, 2)
    w1, w2 = first.weight.clone(), second.weight.clone()
    assert Linear.join(first, second) and Linear.join(first, second)
    assert torch.equal(first.weight, w1) and torch.equal(second.weight, w2)
    assert first.weight.data_ptr() + first.weight.numel() * 2 == second.weight.data_ptr()
    x = _rand(M, H, seed=3).bfloat16().cuda()
    want1 = P.linear(x.double().cpu(), r1["a.weight"], r1["a.bias"])
    want2 = P.gelu(x.double().cpu() @ r2["b.weight"].T)
    for pays in (True, False):
        monkeypatch.setattr(ops, "joined_mm_pays", lambda *a, **k: pays)
        both = Linear.pair(first, x, {}, second, x, {"act": "gelu"})
        if not pays:
            assert both is None  # the block then runs the two on their own
            continue
        y1, y2 = both
        assert y1.shape == (M, N1) and y2.shape == (M, N2) and not y2.is_contiguous()
        _close(y1, want1, 2e-2, "first of the joined product")
        _close(y2, want2, 2e-2, "second of the joined product, with its activation")
        down = Linear("c", N2, 64, bias=False)
        _, r3 = _fill(down, torch.bfloat16, 4)
        _close(down(y2), y2.double().cpu() @ r3["c.weight"].T, 2e-2, "a product whose input rows lie apart")
    monkeypatch.undo()
    assert ops.TUNE_LIVE or ops.joined_mm_pays(x, first.joined[0], N1) is False  # nothing is timed unless asked
    with ops.live_tuning():
        assert ops.joined_mm_pays(x, first.joined[0], N1) in (True, False)  # measured, either way


def test_rows_beyond_one_chunk_take_the_way_that_was_timed_faster(monkeypatch):
    """129 to 256 rows: the decode batch kernel (two chunks of rows per launch) or the library's product, by a
    timing per weight shape; both ways give the plain result, alone and as a pair launch."""
    from pytorch_transformers_amd import ops, tuning
    from pytorch_transformers_amd.parts import Linear

    if ops.SPLITK_MAX_ROWS < 256:
        pytest.skip("capped by PTA_SPLITK_MAX_ROWS")
    H, N1, N2, M = 264, 136, 200, 200
    first, second = Linear("a", H, N1, bias=True), Linear("b", H, N2, bias=False)
    (_, r1), (_, r2) = _fill(first, torch.bfloat16, 1), _fill(second, torch.bfloat16, 2)
    x = _rand(M, H, seed=3).bfloat16().cuda()
    want1 = P.linear(x.double().cpu(), r1["a.weight"], r1["a.bias"])
    want2 = P.gelu(x.double().cpu() @ r2["b.weight"].T)
    assert ops.TUNE_LIVE or ops.splitk_row_limit(first.weight) == 128  # nothing is timed unless asked
    with ops.live_tuning():
        assert ops.splitk_row_limit(first.weight) in (128, 192, 256)  # measured, whichever
    ops.release_flush()
    for limit in (256, 128):
        monkeypatch.setattr(tuning, "splitk_row_limit", lambda *ws: limit)
        assert ops.gemm_splitk_ok(x, first.weight) == (limit == 256)
        _close(first(x), want1, 2e-2, f"alone, limit {limit}")
        both = Linear.pair(first, x, {}, second, x, {"act": "gelu"})
        assert (both is not None) == (limit == 256)
        if both is not None:
            _close(both[0], want1, 2e-2, "first of the pair")
            _close(both[1], want2, 2e-2, "second of the pair")
    # at 128 rows and below nothing is timed: the kernel takes them
    monkeypatch.setattr(tuning, "splitk_row_limit", lambda *ws: 1 / 0)
    assert ops.gemm_splitk_ok(x[:128].contiguous(), first.weight)


def test_library_product_over_ranges_of_k():
    """A few hundred rows with K long against N: the library's batched product over ranges of K, its 32-bit
    partial sums added in order by the kernel that applies bias, activation and additions.  Which way is
    faster is the machine's business, so the ranges are set by hand here; rows of x may lie apart."""
    from pytorch_transformers_amd import ops
    from pytorch_transformers_amd.parts import Linear

    if not ops.MM_KSPLIT:
        pytest.skip("switched off by PTA_MM_KSPLIT=0")
    K, N, M = 640, 136, 300
    lin = Linear("a", K, N, bias=True)
    _, ref = _fill(lin, torch.bfloat16, 1)
    wide = _rand(M, K + 64, seed=3).bfloat16().cuda()
    x = wide[:, 64:]  # rows that lie apart, as a block of columns of a joined product
    a1, a2 = _rand(M, N, seed=4).bfloat16().cuda(), _rand(M, N, seed=5).bfloat16().cuda()
    want = P.gelu(P.linear(x.double().cpu(), ref["a.weight"], ref["a.bias"])) + a1.double().cpu() + a2.double().cpu()
    key = (N, K, (M + 63) // 64)
    try:
        for S in (2, 4, 1):
            ops.active().mm_ksplit[key] = S
            got = ops.library_mm_ksplit(x, lin.weight, lin.bias, "gelu", a1, a2)
            assert (got is None) == (S == 1)
            _close(lin(x, act="gelu", add1=a1, add2=a2), want, 2e-2, f"{S} ranges of K")
    finally:
        ops.active().mm_ksplit.pop(key, None)
    assert ops.library_mm_ksplit(x[:64], lin.weight) is None  # few rows go to the decode kernels
    lin(x, act="gelu", add1=a1, add2=a2)
    assert ops.TUNE_LIVE or key not in ops.active().mm_ksplit  # nothing is timed unless asked
    with ops.live_tuning():
        lin(x, act="gelu", add1=a1, add2=a2)  # timed, whichever way
    ops.release_flush()
    assert ops.active().mm_ksplit.pop(key) in (1, 2, 4)


def test_positions():
    from pytorch_transformers_amd.parts import AlibiPositions, NoPositions, RotaryPositions

    from pytorch_transformers_amd.parts.positions import Rotation, ScoreBias, as_rotation, as_score_bias

    r = RotaryPositions(64, 500042.0, scaling_factor=4.0)
    rot = r.rotation()
    assert torch.equal(rot.inv_freq, P.rope_inv_freq(64, 500042.0, 4.0)) and r.score_bias() is None
    assert (rot.scale, rot.rotary_dim, rot.pairing) == (1.0, None, "half")  # the whole head, half-split pairs
    for nh in (6, 20, 64):
        a = AlibiPositions(nh, scale=0.125)
        bias = a.score_bias()
        assert torch.equal(bias.slopes, P.alibi_slopes(nh).bfloat16().float()) and a.rotation() is None
        assert (bias.of, bias.bf16, bias.scale) == ("key", True, 0.125)
        assert not AlibiPositions(nh, bf16_compat=False).score_bias().bf16
    assert NoPositions().rotation() is None and NoPositions().score_bias() is None
    # what a position encoding may hand out in place of the two classes: a pair for a rotation of whole heads, a
    # tensor of slopes for the reference's bias
    inv = torch.ones(8)
    assert as_rotation((None, 1.0)) is None and as_rotation((inv, 0.5)) == Rotation(inv, 0.5)
    assert as_score_bias(inv, 64) == ScoreBias(inv, "key", True, 0.125) and as_score_bias(None, 64) is None


@pytest.mark.parametrize("dtype,rel", DTYPES)
@pytest.mark.parametrize("layout,nh,nkv,d,alibi,bias", [("grouped", 6, 2, 32, False, False), ("tail", 5, 1, 64, False, True),
                                                        ("interleaved", 3, 3, 24, True, True)])
def test_attention_mixer_and_blocks(dtype, rel, layout, nh, nkv, d, alibi, bias):
    """The mixer alone (whole prompt, then a chunk, then single tokens), and both block arrangements around it."""
    from pytorch_transformers_amd.cache import PagedCache
    from pytorch_transformers_amd.engine.spec import CACHE_FULL, CacheGroupSpec, LayerCall
    from pytorch_transformers_amd.parts.base import as_tensor
    from pytorch_transformers_amd.parts import (AlibiPositions, AttentionMixer, DenseFeedForward, LayerNorm, ParallelBlock,
                                                RotaryPositions, SequentialBlock)

    H, F, T = nh * d, 3 * nh * d + 8, 75
    pos = AlibiPositions(nh, scale=d ** -0.5) if alibi else RotaryPositions(d, 10000.0)  # the scale of modeling_falcon.py:1081
    pos.to("cuda:0")
    mixer = AttentionMixer("transformer.h.0.self_attention", H, nh, nkv, d, layout, bias, pos)
    ffn = DenseFeedForward("transformer.h.0.mlp", H, F, bias)
    n1, n2 = LayerNorm("transformer.h.0.input_layernorm", H, 1e-5), LayerNorm("transformer.h.0.post_attention_layernorm", H, 1e-5)
    n3, n4 = LayerNorm("transformer.h.0.ln_attn", H, 1e-5), LayerNorm("transformer.h.0.ln_mlp", H, 1e-5)
    ref = {}
    for i, part in enumerate((mixer, ffn, n1, n2, n3, n4)):
        ref.update(_fill(part, dtype, 10 + i)[1])
    c = P.cfg_defaults(dict(hidden_size=H, num_attention_heads=nh, num_kv_heads=nkv, alibi=alibi, bias=bias,
                            new_decoder_architecture=layout == "grouped", multi_query=layout == "tail",
                            ffn_hidden_size=F))
    x = _rand(T, H, seed=1).bfloat16()
    positions = torch.arange(T)
    want_mixer = P.self_attention(x.double(), ref, "transformer.h.0.self_attention.", c, positions)
    call = LayerCall(0, "kv", 0)

    def run(fn, cuts):
        cache = PagedCache([CacheGroupSpec("kv", CACHE_FULL, 1, nkv, d)], 256, dtype, "cuda:0")
        slot = cache.alloc()
        outs, at = [], 0
        for n in cuts:
            ctx, plan = _ctx(cache, [slot], [n], dtype)
            outs.append(fn(x[at:at + n].to(dtype).cuda(), ctx))
            cache.commit([slot], [n])
            at += n
        return torch.cat(outs)

    cuts = [40, 30, 1, 1, 1, 1, 1]
    _close(run(lambda xs, ctx: mixer.forward(xs, ctx, call), [T]), want_mixer, rel, "mixer, whole")
    _close(run(lambda xs, ctx: mixer.forward(xs, ctx, call), cuts), want_mixer, rel, "mixer, cut")
    res = run(lambda xs, ctx: mixer.forward(xs, ctx, call, residual=xs), cuts)
    _close(res, want_mixer + x.double(), rel, "mixer with residual")

    # which way the 40-row step above went: its product's launch carries the tail where that product is the
    # split-K kernel's (bfloat16, fewer fused rows than twice the width), else the tail is a kernel of its own
    from pytorch_transformers_amd import ops
    from pytorch_transformers_amd.parts.linear import TailDone
    cache = PagedCache([CacheGroupSpec("kv", CACHE_FULL, 1, nkv, d)], 256, dtype, "cuda:0")
    ctx, _ = _ctx(cache, [cache.alloc()], [40], dtype)
    done = mixer.qkv.with_tail(x[:40].to(dtype).cuda(), mixer.projection_tail(ctx, call))
    carried = dtype == torch.bfloat16 and ops.QKV_TAIL and (nh + 2 * nkv) * d < 2 * H
    assert isinstance(done, TailDone) if carried else done is None

    # blocks: each arrangement is a decoder layer of the plain implementation with the matching flags
    for block, flags in ((ParallelBlock(mixer, ffn, n1), dict(parallel_attn=True, new_decoder_architecture=False)),
                         (SequentialBlock(mixer, ffn, n1, n2), dict(parallel_attn=False, new_decoder_architecture=False)),
                         (ParallelBlock(mixer, ffn, n3, n4), dict(parallel_attn=True, new_decoder_architecture=True,
                                                                  num_ln_in_parallel_attn=2))):
        if flags["new_decoder_architecture"] != (layout == "grouped"):
            continue  # the fused row order belongs to the architecture flag in the plain code
        cc = P.cfg_defaults(dict(c, **flags))
        want = P.decoder_layer(x.double(), ref, 0, cc, positions)
        _close(run(lambda xs, ctx: as_tensor(block.forward(xs, ctx, call)), cuts), want, rel, f"{type(block).__name__} {flags}")


# --- a toy architecture, defined in the test -------------------------------------------------------------
def _define_toy(device_decode: bool = False):
    """``device_decode``: in steps of one token per sequence the mixer reads nothing but the step's device
    arrays, so that such steps can be captured and replayed; the model then says ``supports_graphs=True``."""
    from pytorch_transformers_amd.config.base import ModelConfig
    from pytorch_transformers_amd.engine.spec import (CACHE_FULL, CACHE_STATE, INIT_NORMAL, MATRIX, CacheGroupSpec,
                                                      LayerCall, ModelSpec, TensorSpec)
    from pytorch_transformers_amd.parts import (AttentionMixer, DenseFeedForward, Embedding, LayerNorm, NoPositions,
                                                OutputHead, ParallelBlock, Part, SequentialBlock, register_part)

    @dataclasses.dataclass
    class ToyConfig(ModelConfig):
        model_type = "toy-decay"
        vocab_size: int = 97
        width: int = 48
        layers: int = 3
        decay: float = 0.8

    class DecayMixer(Part):
        """y_t = s_t @ W, s_t = decay * s_{t-1} + x_t: a running state per sequence instead of keys and values."""

        def __init__(self, name, width, decay):
            self.name, self.width, self.decay = name, width, decay

        def tensor_specs(self):
            return [TensorSpec(self.name + ".weight", (self.width, self.width), MATRIX, INIT_NORMAL)]

        def load(self, tensors):
            self.weight = tensors[self.name + ".weight"]

        def forward(self, x, ctx, call, residual=None):
            table = ctx.cache.state_layer(call.cache_group, call.cache_layer)  # [slots, width], 32-bit
            if device_decode and ctx.is_decode:
                rows = ctx.seq_slot.long()  # one token per sequence: token t belongs to sequence t
                s = self.decay * table.index_select(0, rows) + x.float()
                table.index_copy_(0, rows, s)
                out = (s @ self.weight.float().T).to(x.dtype)
                return out if residual is None else out + residual
            out = torch.empty_like(x)
            at = 0
            for slot, n in zip(ctx.slots, ctx.new_tokens):
                s = table[slot].clone()
                for t in range(at, at + n):
                    s = self.decay * s + x[t].float()
                    out[t] = (s @ self.weight.float().T).to(x.dtype)
                table[slot] = s
                at += n
            return out if residual is None else out + residual

    register_part("mixer", "decay", DecayMixer, exist_ok=True)

    def build_toy(cfg):
        blocks, order = [], []
        for i in range(cfg.layers):
            p = f"toy.h.{i}"
            ffn = DenseFeedForward(f"{p}.mlp", cfg.width, 2 * cfg.width, bias=False)
            if i == 1:  # one attention layer among the state layers: two cache groups in one model
                mixer = AttentionMixer(f"{p}.attn", cfg.width, 3, 1, 16, "tail", False, NoPositions())
                blocks.append(ParallelBlock(mixer, ffn, LayerNorm(f"{p}.norm", cfg.width, 1e-5)))
                order.append(LayerCall(i, "kv", 0))
            else:
                mixer = DecayMixer(f"{p}.decay", cfg.width, cfg.decay)
                blocks.append(SequentialBlock(mixer, ffn, LayerNorm(f"{p}.n1", cfg.width, 1e-5), LayerNorm(f"{p}.n2", cfg.width, 1e-5)))
                order.append(LayerCall(i, "state", len([c for c in order if c.cache_group == "state"])))
        order.append(LayerCall(0, "state", cfg.layers - 1))  # block 0 runs a second time, on a state layer of its own
        return ModelSpec(config=cfg, embedding=Embedding("toy.embed", cfg.vocab_size, cfg.width), blocks=blocks, order=order,
                         final_norm=LayerNorm("toy.final", cfg.width, 1e-5),
                         head=OutputHead("toy.head", cfg.vocab_size, cfg.width, "toy.embed.weight"),
                         cache_groups=[CacheGroupSpec("kv", CACHE_FULL, 1, 1, 16),
                                       CacheGroupSpec("state", CACHE_STATE, cfg.layers, state_shape=(cfg.width,))],
                         supports_graphs=device_decode)  # else the toy mixer reads the step's host lists

    return ToyConfig, build_toy


def _plain_toy(cfg, w, ids):
    """The toy model whole, in float64, from the same tensors."""
    x = w["toy.embed.weight"][torch.as_tensor(ids)]
    T = len(ids)

    def decay_mixer(h, name):
        s, out = torch.zeros(cfg.width, dtype=torch.float64), []
        for t in range(T):
            s = cfg.decay * s + h[t]
            out.append(s @ w[name + ".weight"].T)
        return torch.stack(out)

    def ffn(h, p):
        return P.gelu(h @ w[p + ".mlp.dense_h_to_4h.weight"].T) @ w[p + ".mlp.dense_4h_to_h.weight"].T

    def ln(h, name):
        return P.layer_norm(h, w[name + ".weight"], w[name + ".bias"], 1e-5)

    def state_block(h, i):
        p = f"toy.h.{i}"
        r = h + decay_mixer(ln(h, p + ".n1"), p + ".decay")
        return r + ffn(ln(r, p + ".n2"), p)

    for i in list(range(cfg.layers)) + [0]:
        p = f"toy.h.{i}"
        if i == 1:
            a = ln(x, p + ".norm")
            fused = a @ w[p + ".attn.query_key_value.weight"].T
            qkv = fused.view(T, 5, 16)
            o = P.attention_scores_softmax(qkv[:, :3], qkv[:, [3]], qkv[:, [4]])
            x = x + (ffn(a, p) + o @ w[p + ".attn.dense.weight"].T)
        else:
            x = state_block(x, i)
    return ln(x, "toy.final") @ w["toy.embed.weight"].T


@pytest.mark.parametrize("dtype,rel", [("float32", helpers.REL_F32), ("bfloat16", helpers.REL_BF16)])
def test_toy_architecture_with_a_state_mixer(tmp_path, dtype, rel):
    """Register, write random weights, load, replay whole / one by one / in unequal batches with slot
    reuse, and generate: all through the framework's own entry points."""
    from safetensors.torch import load_file

    from pytorch_transformers_amd import AutoModelForCausalLM
    from pytorch_transformers_amd.config import AutoConfig, register, unregister
    from pytorch_transformers_amd.engine.replay import Replayer
    from pytorch_transformers_amd.weights import write_random_model

    ToyConfig, build_toy = _define_toy()
    register("toy-decay", ToyConfig, build_toy, exist_ok=True)
    try:
        cfg = ToyConfig(decay=0.7, layers=3)
        folder = write_random_model(str(tmp_path / "toy"), cfg, seed=5, std=0.08, noise=0.1)
        assert isinstance(AutoConfig.from_pretrained(folder), ToyConfig)
        model = AutoModelForCausalLM.from_pretrained(folder, dtype=dtype)
        assert not model.use_graphs
        w = {k: v.double() for k, v in load_file(f"{folder}/model.safetensors").items()}
        reqs = helpers.make_requests(cfg.vocab_size, [9, 30, 70, 3, 41], seed=2)
        want = {rid: _plain_toy(cfg, w, toks).float() for rid, toks in reqs.items()}
        rp = Replayer(model, 1024, max_slots=8)
        for name, records in (("whole", helpers.schedule_whole(reqs)), ("tail", helpers.schedule_tail(reqs, 8)),
                              ("batches", helpers.schedule_batches(reqs, 3)), ("batches again", helpers.schedule_batches(reqs, 2))):
            got = helpers.run_schedule(rp, records)
            for rid in reqs:
                helpers.assert_close(got[rid], want[rid], rel, f"toy {dtype} {name} {rid}")
        # a slot that is used again starts from zero state: a stale state would change these logits
        assert not rp.cache.live_slots()
        if dtype == "float32":
            out = model.generate([reqs["r0"], reqs["r3"]], max_new_tokens=5, do_sample=False, eos_token_id=None)
            for seq, rid in zip(out, ("r0", "r3")):
                toks = list(reqs[rid])
                for _ in range(5):
                    toks.append(int(_plain_toy(cfg, w, toks)[-1].argmax()))
                assert seq == toks
    finally:
        unregister("toy-decay")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_state_mixer_decodes_under_captured_steps(tmp_path, dtype):
    """A model with a state group whose decode steps are captured and replayed gives the bits of the same steps
    launched one by one: the first step of a shape runs once (not once to warm up and once as a replay), and the
    rows that pad a batch to the captured size advance the scratch slot's state, never a sequence's.  Batches of
    3, 5 and 11 sequences use padded shapes (4 rows; 8; 16), and sequences leave on the way."""
    from pytorch_transformers_amd import AutoModelForCausalLM
    from pytorch_transformers_amd.config import register, unregister
    from pytorch_transformers_amd.engine.replay import Replayer
    from pytorch_transformers_amd.weights import write_random_model

    ToyConfig, build_toy = _define_toy(device_decode=True)
    register("toy-decay", ToyConfig, build_toy, exist_ok=True)
    try:
        cfg = ToyConfig(decay=0.6, layers=3)
        folder = write_random_model(str(tmp_path / "toy"), cfg, seed=6, std=0.08, noise=0.1)
        reqs = helpers.make_requests(cfg.vocab_size, [9, 30, 70, 3, 41, 12, 25, 8, 19, 33, 50], seed=4)
        records = helpers.schedule_batches(reqs, 3, decode=(5, 2, 8)) + \
            [dict(r, step=r["step"] + 1000) for r in helpers.schedule_batches(reqs, 5, decode=(3, 7, 2, 6, 4))] + \
            [dict(r, step=r["step"] + 2000) for r in helpers.schedule_batches(reqs, 11, decode=(2, 9, 4))]
        outs = {}
        for graphs in (False, True):
            model = AutoModelForCausalLM.from_pretrained(folder, dtype=dtype)
            assert model.use_graphs
            model.use_graphs = graphs
            rp = Replayer(model, 2048, max_slots=16)
            outs[graphs] = [rp.run(rec) for rec in records]
            torch.cuda.synchronize()
            if graphs:
                shapes = sorted(g.n for g in rp.cache._decode_graphs.values() if g.graph is not None)
                assert len(shapes) >= 3 and shapes[-1] == 16, f"captured shapes: {shapes}"
        for rec, a, b in zip(records, outs[False], outs[True]):
            assert (a is None) == (b is None)
            if a is not None:
                assert torch.equal(a, b), f"step {rec['step']}: a captured step differs from the same step launched directly"
    finally:
        unregister("toy-decay")


# --- a second toy: a routed feed-forward and a position encoding of its own, both defined here ------------
def _define_routed_toy():
    from pytorch_transformers_amd.config.base import ModelConfig
    from pytorch_transformers_amd.engine.spec import (CACHE_FULL, INIT_NORMAL, MATRIX, CacheGroupSpec, LayerCall, ModelSpec,
                                                      TensorSpec)
    from pytorch_transformers_amd.parts import (AttentionMixer, DenseFeedForward, Embedding, LayerNorm, NoPositions,
                                                OutputHead, ParallelBlock, Part, SequentialBlock, register_part)

    @dataclasses.dataclass
    class RoutedConfig(ModelConfig):
        model_type = "toy-routed"
        vocab_size: int = 131
        width: int = 64
        experts: int = 3
        heads: int = 4

    class HarmonicPositions(NoPositions):
        """Rotation with frequencies 1/(j+1) instead of a geometric ladder: another position encoding that
        feeds the same seam (``rotation()``), read by the framework's rotary kernel unchanged."""

        def __init__(self, head_dim):
            self.inv_freq = (1.0 / torch.arange(1, head_dim // 2 + 1, dtype=torch.float32)).contiguous()

        def to(self, device):
            self.inv_freq = self.inv_freq.to(device)

        def rotation(self):
            return self.inv_freq, 1.0

    class RoutedFeedForward(Part):
        """Each token goes to the expert its router scores highest (scores and softmax in 32-bit), and the
        expert's output is weighted by that probability.  Experts are the framework's dense feed-forwards."""

        def __init__(self, name, width, experts):
            self.name, self.width = name, width
            self.experts = [DenseFeedForward(f"{name}.experts.{e}", width, 2 * width, bias=True) for e in range(experts)]

        def tensor_specs(self):
            return [TensorSpec(self.name + ".router.weight", (len(self.experts), self.width), MATRIX, INIT_NORMAL)]

        def load(self, tensors):
            self.router = tensors[self.name + ".router.weight"]

        def children(self):
            return tuple(self.experts)

        def forward(self, x, ctx, add1=None, add2=None):
            probs = torch.softmax(x.float() @ self.router.float().T, dim=-1)
            gate, pick = probs.max(dim=-1)
            out = torch.zeros_like(x, dtype=torch.float32)
            for e, expert in enumerate(self.experts):
                rows = torch.nonzero(pick == e).flatten()
                if rows.numel():
                    y = expert.forward(x.index_select(0, rows).contiguous(), ctx)
                    out.index_copy_(0, rows, y.float() * gate[rows, None])
            for a in (add1, add2):
                if a is not None:
                    out = out + a.float()
            return out.to(x.dtype)

    register_part("positions", "harmonic", HarmonicPositions, exist_ok=True)
    register_part("feed_forward", "routed", RoutedFeedForward, exist_ok=True)

    def build(cfg):
        d = cfg.width // cfg.heads
        blocks = [
            ParallelBlock(AttentionMixer("t.h.0.attn", cfg.width, cfg.heads, 2, d, "grouped", False, HarmonicPositions(d)),
                          RoutedFeedForward("t.h.0.moe", cfg.width, cfg.experts), LayerNorm("t.h.0.norm", cfg.width, 1e-5)),
            SequentialBlock(AttentionMixer("t.h.1.attn", cfg.width, cfg.heads, cfg.heads, d, "interleaved", True, NoPositions()),
                            RoutedFeedForward("t.h.1.moe", cfg.width, cfg.experts), LayerNorm("t.h.1.n1", cfg.width, 1e-5),
                            LayerNorm("t.h.1.n2", cfg.width, 1e-5)),
        ]
        return ModelSpec(config=cfg, embedding=Embedding("t.embed", cfg.vocab_size, cfg.width), blocks=blocks,
                         order=[LayerCall(0, "grouped", 0), LayerCall(1, "full", 0)],
                         final_norm=LayerNorm("t.final", cfg.width, 1e-5),
                         head=OutputHead("t.head", cfg.vocab_size, cfg.width, "t.embed.weight"),
                         # the two layers keep different numbers of heads: a cache group each, pages of their own
                         cache_groups=[CacheGroupSpec("grouped", CACHE_FULL, 1, 2, d),
                                       CacheGroupSpec("full", CACHE_FULL, 1, cfg.heads, d)],
                         supports_graphs=False)  # routing looks at the data on the host

    return RoutedConfig, build


def _plain_routed(cfg, w, ids):
    T, H, nh = len(ids), cfg.width, cfg.heads
    d = H // nh
    x = w["t.embed.weight"][torch.as_tensor(ids)]
    ln = lambda h, n: P.layer_norm(h, w[n + ".weight"], w[n + ".bias"], 1e-5)

    def moe(h, p):
        probs = torch.softmax(h @ w[p + ".router.weight"].T, dim=-1)
        gate, pick = probs.max(dim=-1)
        out = torch.zeros_like(h)
        for t in range(T):
            e = f"{p}.experts.{int(pick[t])}"
            u = P.gelu(h[t] @ w[e + ".dense_h_to_4h.weight"].T + w[e + ".dense_h_to_4h.bias"])
            out[t] = gate[t] * (u @ w[e + ".dense_4h_to_h.weight"].T + w[e + ".dense_4h_to_h.bias"])
        return out

    # layer 0: parallel, grouped rows (2 groups of 2 heads), rotation with harmonic frequencies
    a = ln(x, "t.h.0.norm")
    f = (a @ w["t.h.0.attn.query_key_value.weight"].T).view(T, 2, 4, d)
    q, k, v = f[:, :, :2].reshape(T, nh, d), f[:, :, 2], f[:, :, 3]
    cos, sin = P.rope_cos_sin(torch.arange(T), 1.0 / torch.arange(1, d // 2 + 1, dtype=torch.float32))
    o = P.attention_scores_softmax(P.apply_rope(q, cos, sin), P.apply_rope(k, cos, sin), v)
    x = x + (moe(a, "t.h.0.moe") + o @ w["t.h.0.attn.dense.weight"].T)
    # layer 1: sequential, interleaved rows with bias, no positions
    a = ln(x, "t.h.1.n1")
    f = (a @ w["t.h.1.attn.query_key_value.weight"].T + w["t.h.1.attn.query_key_value.bias"]).view(T, nh, 3, d)
    o = P.attention_scores_softmax(f[:, :, 0], f[:, :, 1], f[:, :, 2])
    r = x + o @ w["t.h.1.attn.dense.weight"].T + w["t.h.1.attn.dense.bias"]
    x = r + moe(ln(r, "t.h.1.n2"), "t.h.1.moe")
    return ln(x, "t.final") @ w["t.embed.weight"].T


def test_toy_architecture_with_routing_and_its_own_positions(tmp_path):
    """A feed-forward with a router and experts and a position encoding that the framework does not have,
    both defined in this file, registered, built, loaded and stepped through every schedule (32-bit, where a
    token that changed its expert would show)."""
    from safetensors.torch import load_file

    from pytorch_transformers_amd import AutoModelForCausalLM
    from pytorch_transformers_amd.config import register, unregister
    from pytorch_transformers_amd.engine.replay import Replayer
    from pytorch_transformers_amd.parts import registered_parts
    from pytorch_transformers_amd.weights import write_random_model

    RoutedConfig, build = _define_routed_toy()
    assert "routed" in registered_parts("feed_forward") and "harmonic" in registered_parts("positions")
    register("toy-routed", RoutedConfig, build, exist_ok=True)
    try:
        cfg = RoutedConfig()
        folder = write_random_model(str(tmp_path / "routed"), cfg, seed=9, std=0.2, noise=0.1)
        w = {k: v.double() for k, v in load_file(f"{folder}/model.safetensors").items()}
        assert sum(".experts." in k for k in w) == 2 * cfg.experts * 4 and "t.h.0.moe.router.weight" in w
        model = AutoModelForCausalLM.from_pretrained(folder, dtype="float32")
        reqs = helpers.make_requests(cfg.vocab_size, [11, 40, 70, 5], seed=4)
        want = {rid: _plain_routed(cfg, w, toks).float() for rid, toks in reqs.items()}
        rp = Replayer(model, 1024, max_slots=4)
        for name, records in (("whole", helpers.schedule_whole(reqs)), ("tail", helpers.schedule_tail(reqs, 16)),
                              ("batches", helpers.schedule_batches(reqs, 3))):
            got = helpers.run_schedule(rp, records)
            for rid in reqs:
                helpers.assert_close(got[rid], want[rid], 5e-5, f"routed toy {name} {rid}")
    finally:
        unregister("toy-routed")


# --- a third toy: a layer that attends to a window of the last positions, with a cache group of its own ---
def _define_window_toy(window):
    from pytorch_transformers_amd.config.base import ModelConfig
    from pytorch_transformers_amd.engine.spec import CACHE_FULL, CACHE_WINDOW, CacheGroupSpec, LayerCall, ModelSpec
    from pytorch_transformers_amd.parts import (AttentionMixer, DenseFeedForward, Embedding, LayerNorm, OutputHead,
                                                ParallelBlock, RotaryPositions)

    @dataclasses.dataclass
    class WindowConfig(ModelConfig):
        model_type = "toy-window"
        vocab_size: int = 113
        width: int = 64
        heads: int = 2

    def build(cfg):
        d = cfg.width // cfg.heads
        def block(i, win):
            mixer = AttentionMixer(f"t.h.{i}.attn", cfg.width, cfg.heads, 1, d, "tail", False, RotaryPositions(d, 10000.0),
                                   window=win)
            return ParallelBlock(mixer, DenseFeedForward(f"t.h.{i}.mlp", cfg.width, 2 * cfg.width, bias=False),
                                 LayerNorm(f"t.h.{i}.norm", cfg.width, 1e-5))
        return ModelSpec(config=cfg, embedding=Embedding("t.embed", cfg.vocab_size, cfg.width),
                         blocks=[block(0, window), block(1, 0)], order=[LayerCall(0, "near", 0), LayerCall(1, "all", 0)],
                         final_norm=LayerNorm("t.final", cfg.width, 1e-5),
                         head=OutputHead("t.head", cfg.vocab_size, cfg.width, "t.embed.weight"),
                         cache_groups=[CacheGroupSpec("near", CACHE_WINDOW, 1, 1, d, window=window),
                                       CacheGroupSpec("all", CACHE_FULL, 1, 1, d)])

    return WindowConfig, build


def _plain_window_toy(cfg, w, ids, window):
    T, H, nh = len(ids), cfg.width, cfg.heads
    d = H // nh
    x = w["t.embed.weight"][torch.as_tensor(ids)]
    cos, sin = P.rope_cos_sin(torch.arange(T), P.rope_inv_freq(d, 10000.0))
    t = torch.arange(T)
    for i, win in ((0, window), (1, 0)):
        p = f"t.h.{i}"
        a = P.layer_norm(x, w[p + ".norm.weight"], w[p + ".norm.bias"], 1e-5)
        f = (a @ w[p + ".attn.query_key_value.weight"].T).view(T, nh + 2, d)
        q, k, v = P.apply_rope(f[:, :nh], cos, sin), P.apply_rope(f[:, nh:nh + 1], cos, sin), f[:, nh + 1:]
        seen = t[None, :] <= t[:, None]
        if win:
            seen = seen & (t[None, :] > t[:, None] - win)
        o = torch.empty(T, nh, d, dtype=x.dtype)
        for h in range(nh):
            s = (q[:, h] @ k[:, 0].T / math.sqrt(d)).masked_fill(~seen, float("-inf"))
            o[:, h] = torch.softmax(s, dim=-1) @ v[:, 0]
        mlp = P.gelu(a @ w[p + ".mlp.dense_h_to_4h.weight"].T) @ w[p + ".mlp.dense_4h_to_h.weight"].T
        x = x + (mlp + o.reshape(T, H) @ w[p + ".attn.dense.weight"].T)
    return P.layer_norm(x, w["t.final.weight"], w["t.final.bias"], 1e-5) @ w["t.embed.weight"].T


@pytest.mark.parametrize("dtype,rel", [("float32", helpers.REL_F32), ("bfloat16", helpers.REL_BF16)])
def test_toy_architecture_with_a_window_layer(tmp_path, dtype, rel):
    """One layer sees the last 40 positions and keeps them in a cache group of kind `window`, the other sees
    everything: every schedule against the plain model, and the window group gives its pages back."""
    from safetensors.torch import load_file

    from pytorch_transformers_amd import AutoModelForCausalLM
    from pytorch_transformers_amd.config import register, unregister
    from pytorch_transformers_amd.engine.replay import Replayer
    from pytorch_transformers_amd.weights import write_random_model

    window = 40
    WindowConfig, build = _define_window_toy(window)
    register("toy-window", WindowConfig, build, exist_ok=True)
    try:
        cfg = WindowConfig()
        folder = write_random_model(str(tmp_path / "window"), cfg, seed=3, std=0.15, noise=0.1)
        w = {k: v.double() for k, v in load_file(f"{folder}/model.safetensors").items()}
        model = AutoModelForCausalLM.from_pretrained(folder, dtype=dtype)
        reqs = helpers.make_requests(cfg.vocab_size, [9, 150, 70, 41, 230], seed=6)
        want = {rid: _plain_window_toy(cfg, w, toks, window).float() for rid, toks in reqs.items()}
        rp = Replayer(model, 1024, max_slots=4)
        for name, records in (("whole", helpers.schedule_whole(reqs)), ("tail", helpers.schedule_tail(reqs, 32)),
                              ("batches", helpers.schedule_batches(reqs, 3, decode=(3, 60, 1)))):
            got = helpers.run_schedule(rp, records)
            for rid in reqs:
                helpers.assert_close(got[rid], want[rid], rel, f"window toy {dtype} {name} {rid}")
        # decoding far past the window (as captured graphs where the model allows them): the window group holds
        # a page or two, the full group all of them
        cache = model.new_cache(1024, max_slots=1)
        slot = cache.alloc()
        toks = reqs["r4"]
        model.step(cache, [slot], [toks[:50]], "none")
        for t in toks[50:]:
            logits = model.step(cache, [slot], [[t]], "last")
        helpers.assert_close(logits[0].float().cpu()[None], want["r4"][-1:], rel, f"window toy {dtype} long decode")
        held = [p for p in cache.page_list("near", slot) if p >= 0]
        assert len(held) <= 2 and len(cache.page_list("all", slot)) == 4
        cache.check_consistent()
    finally:
        unregister("toy-window")


# --- a fourth toy: position encodings of its own, said in the data that the kernels take ---
def _define_positions_toy():
    from pytorch_transformers_amd.config.base import ModelConfig
    from pytorch_transformers_amd.engine.spec import CACHE_FULL, CacheGroupSpec, LayerCall, ModelSpec
    from pytorch_transformers_amd.parts import (AttentionMixer, DenseFeedForward, Embedding, LayerNorm, NoPositions,
                                                OutputHead, ParallelBlock, Rotation, ScoreBias, SequentialBlock,
                                                register_part)

    @dataclasses.dataclass
    class PositionsConfig(ModelConfig):
        model_type = "toy-positions"
        vocab_size: int = 157
        width: int = 256
        heads: int = 4
        rotary_fraction: float = 0.5
        theta: float = 1000.0
        slope_base: float = 0.25

    class PartialInterleavedRotary(NoPositions):
        """Rotates the first part of every head only, in pairs of neighbouring elements (2i, 2i + 1): a rotation that
        the framework's own position encoding does not have, said in the fields of ``Rotation``."""

        def __init__(self, head_dim, fraction, theta):
            self.rotary_dim = int(head_dim * fraction) // 2 * 2
            self.inv_freq = (1.0 / theta ** (torch.arange(0, self.rotary_dim, 2, dtype=torch.float32) / self.rotary_dim)).contiguous()

        def to(self, device):
            self.inv_freq = self.inv_freq.to(device)

        def rotation(self):
            return Rotation(self.inv_freq, 1.0, rotary_dim=self.rotary_dim, pairing="interleaved")

    class DistanceBias(NoPositions):
        """A bias on the scores that falls with the distance between query and key, ``-slope_h * (t - j)``, exact and
        with no further scale: another bias function of (head, query position, key position)."""

        def __init__(self, heads, base):
            self.slopes = (base ** torch.arange(1, heads + 1, dtype=torch.float32)).contiguous()

        def to(self, device):
            self.slopes = self.slopes.to(device)

        def score_bias(self):
            return ScoreBias(self.slopes, of="distance", bf16=False, scale=1.0)

    register_part("positions", "partial-interleaved", PartialInterleavedRotary, exist_ok=True)
    register_part("positions", "distance-bias", DistanceBias, exist_ok=True)

    def build(cfg):
        d = cfg.width // cfg.heads
        rotary = PartialInterleavedRotary(d, cfg.rotary_fraction, cfg.theta)
        blocks = [
            # one norm, so that decode steps run the fused query_key_value rows through the pair launches' tails
            ParallelBlock(AttentionMixer("t.h.0.attn", cfg.width, cfg.heads, 2, d, "grouped", True, rotary),
                          DenseFeedForward("t.h.0.mlp", cfg.width, 2 * cfg.width, bias=False), LayerNorm("t.h.0.norm", cfg.width, 1e-5)),
            SequentialBlock(AttentionMixer("t.h.1.attn", cfg.width, cfg.heads, 1, d, "tail", False, DistanceBias(cfg.heads, cfg.slope_base)),
                            DenseFeedForward("t.h.1.mlp", cfg.width, 2 * cfg.width, bias=False), LayerNorm("t.h.1.n1", cfg.width, 1e-5),
                            LayerNorm("t.h.1.n2", cfg.width, 1e-5)),
        ]
        return ModelSpec(config=cfg, embedding=Embedding("t.embed", cfg.vocab_size, cfg.width), blocks=blocks,
                         order=[LayerCall(0, "two", 0), LayerCall(1, "one", 0)],
                         final_norm=LayerNorm("t.final", cfg.width, 1e-5),
                         head=OutputHead("t.head", cfg.vocab_size, cfg.width, "t.embed.weight"),
                         cache_groups=[CacheGroupSpec("two", CACHE_FULL, 1, 2, d), CacheGroupSpec("one", CACHE_FULL, 1, 1, d)])

    return PositionsConfig, build


def _plain_positions_toy(cfg, w, ids):
    T, H, nh = len(ids), cfg.width, cfg.heads
    d = H // nh
    r = int(d * cfg.rotary_fraction) // 2 * 2
    x = w["t.embed.weight"][torch.as_tensor(ids)]
    ln = lambda h, n: P.layer_norm(h, w[n + ".weight"], w[n + ".bias"], 1e-5)
    ffn = lambda h, p: P.gelu(h @ w[p + ".dense_h_to_4h.weight"].T) @ w[p + ".dense_4h_to_h.weight"].T
    pos = torch.arange(T)

    def rotate(t):  # neighbouring elements of the first r of a head, pair i by pos * theta^(-2i/r); angles in 32-bit
        inv = 1.0 / cfg.theta ** (torch.arange(0, r, 2, dtype=torch.float32) / r)
        ang = pos.float()[:, None] * inv[None, :]
        cos, sin = ang.cos().double()[:, None, :], ang.sin().double()[:, None, :]
        out = t.clone()
        a, b = t[..., 0:r:2], t[..., 1:r:2]
        out[..., 0:r:2], out[..., 1:r:2] = a * cos - b * sin, b * cos + a * sin
        return out

    # layer 0: parallel, grouped rows (2 groups of 2 heads) with a bias, part of each head rotated in interleaved pairs
    a = ln(x, "t.h.0.norm")
    f = (a @ w["t.h.0.attn.query_key_value.weight"].T + w["t.h.0.attn.query_key_value.bias"]).view(T, 2, 4, d)
    q, k, v = f[:, :, :2].reshape(T, nh, d), f[:, :, 2], f[:, :, 3]
    o = P.attention_scores_softmax(rotate(q), rotate(k), v)
    x = x + (ffn(a, "t.h.0.mlp") + (o @ w["t.h.0.attn.dense.weight"].T + w["t.h.0.attn.dense.bias"]))
    # layer 1: sequential, one KV head at the tail, scores biased by -slope_h * (query position - key position)
    a = ln(x, "t.h.1.n1")
    f = (a @ w["t.h.1.attn.query_key_value.weight"].T).view(T, nh + 2, d)
    slopes = (cfg.slope_base ** torch.arange(1, nh + 1, dtype=torch.float32)).double()
    o = torch.empty(T, nh, d, dtype=x.dtype)
    causal = pos[None, :] <= pos[:, None]
    for h in range(nh):
        s = f[:, h] @ f[:, nh].T / math.sqrt(d) + slopes[h] * (pos[None, :] - pos[:, None]).double()
        o[:, h] = torch.softmax(s.masked_fill(~causal, float("-inf")), dim=-1) @ f[:, nh + 1]
    rsd = x + o.reshape(T, H) @ w["t.h.1.attn.dense.weight"].T
    x = rsd + ffn(ln(rsd, "t.h.1.n2"), "t.h.1.mlp")
    return ln(x, "t.final") @ w["t.embed.weight"].T


@pytest.mark.parametrize("dtype,rel", [("float32", 5e-5), ("bfloat16", helpers.REL_BF16)])
def test_toy_architecture_with_positions_of_its_own(tmp_path, dtype, rel):
    """A rotation of half of every head in interleaved pairs and a score bias by the distance between query and key,
    both defined in this file as position parts that hand the kernels their data (``Rotation``, ``ScoreBias``):
    registered, built and stepped through every schedule with no change to the framework's files; in bfloat16 also
    as decode batches of 5 and of 20 sequences, whose fused rows are rotated in the matrix launches' own tails."""
    from safetensors.torch import load_file

    from pytorch_transformers_amd import AutoModelForCausalLM
    from pytorch_transformers_amd.config import register, unregister
    from pytorch_transformers_amd.engine.replay import Replayer
    from pytorch_transformers_amd.parts import registered_parts
    from pytorch_transformers_amd.weights import write_random_model

    PositionsConfig, build = _define_positions_toy()
    assert {"partial-interleaved", "distance-bias"} <= set(registered_parts("positions"))
    register("toy-positions", PositionsConfig, build, exist_ok=True)
    try:
        cfg = PositionsConfig()
        folder = write_random_model(str(tmp_path / "positions"), cfg, seed=12, std=0.1, noise=0.1)
        w = {k: v.double() for k, v in load_file(f"{folder}/model.safetensors").items()}
        model = AutoModelForCausalLM.from_pretrained(folder, dtype=dtype)
        reqs = helpers.make_requests(cfg.vocab_size, [11, 40, 70, 5, 131], seed=4)
        want = {rid: _plain_positions_toy(cfg, w, toks).float() for rid, toks in reqs.items()}
        # the positions decide: the same tokens in another order give other logits at the last place
        swapped = list(reqs["r1"])
        swapped[3], swapped[17] = swapped[17], swapped[3]
        assert float((_plain_positions_toy(cfg, w, swapped)[-1] - want["r1"][-1].double()).abs().max()) > 1e-3
        rp = Replayer(model, 4096, max_slots=24)
        for name, records in (("whole", helpers.schedule_whole(reqs)), ("tail", helpers.schedule_tail(reqs, 16)),
                              ("batches", helpers.schedule_batches(reqs, 3)), ("one batch", helpers.schedule_batches(reqs, 5))):
            got = helpers.run_schedule(rp, records)
            for rid in reqs:
                helpers.assert_close(got[rid], want[rid], rel, f"positions toy {dtype} {name} {rid}")
        # twenty sequences at once: decode steps of 17 rows and more
        many = helpers.make_requests(cfg.vocab_size, [20 + (7 * i) % 30 for i in range(20)], seed=5)
        want = {rid: _plain_positions_toy(cfg, w, toks).float() for rid, toks in many.items()}
        got = helpers.run_schedule(rp, helpers.schedule_batches(many, 20, decode=(6, 8, 7, 9)))
        for rid in many:
            helpers.assert_close(got[rid], want[rid], rel, f"positions toy {dtype} twenty at once {rid}")
    finally:
        unregister("toy-positions")


def test_a_position_part_that_asks_for_what_no_kernel_has_is_refused_by_name():
    """A rotation or a score bias that the fields cannot say is refused when the model is put together, by the part
    that has it, with what is built."""
    from pytorch_transformers_amd.parts import AttentionMixer, NoPositions, Rotation, ScoreBias

    class Thirds(NoPositions):
        def rotation(self):
            return Rotation(torch.ones(8), 1.0, rotary_dim=16, pairing="thirds")

    class QueryBias(NoPositions):
        def score_bias(self):
            return ScoreBias(torch.ones(4), of="query")

    class TooWide(NoPositions):
        def rotation(self):
            return Rotation(torch.ones(40), 1.0, rotary_dim=80)

    for positions, match in ((Thirds(), "pairing 'thirds' is not built"), (QueryBias(), "score bias of 'query' is not built"),
                             (TooWide(), "rotary_dim must be even, from 2 up to the head size 64")):
        with pytest.raises(ValueError, match=match):
            AttentionMixer("m", 256, 4, 2, 64, "grouped", False, positions).check_sizes()


# --- a fifth toy: a norm of its own (no mean, no bias), in every place a norm stands ---
def _define_norm_toy():
    from pytorch_transformers_amd.config.base import ModelConfig
    from pytorch_transformers_amd.engine.spec import CACHE_FULL, INIT_ONE_NOISE, VECTOR, CacheGroupSpec, LayerCall, ModelSpec, TensorSpec
    from pytorch_transformers_amd.parts import (AttentionMixer, DenseFeedForward, Embedding, OutputHead, ParallelBlock, Part,
                                                RotaryPositions, SequentialBlock, register_part)

    @dataclasses.dataclass
    class NormConfig(ModelConfig):
        model_type = "toy-norm"
        vocab_size: int = 149
        width: int = 96
        heads: int = 3
        eps: float = 1e-4

    class RootMeanSquareNorm(Part):
        """``x / sqrt(mean(x^2) + eps) * w``: no mean taken off, no bias; statistics in 32-bit.  It offers the plain
        interface of a norm and none of the optional ones (no pair in one pass, no sum formed while it reads)."""

        def __init__(self, name, width, eps):
            self.name, self.width, self.eps = name, width, eps

        def tensor_specs(self):
            return [TensorSpec(self.name + ".weight", (self.width,), VECTOR, INIT_ONE_NOISE)]

        def load(self, tensors):
            self.weight = tensors[self.name + ".weight"]

        def forward(self, x, rows=None):
            if rows is not None:
                x = x.index_select(0, rows.long())
            h = x.float()
            return (h * torch.rsqrt(h.pow(2).mean(-1, keepdim=True) + self.eps) * self.weight).to(x.dtype)

    register_part("norm", "rms", RootMeanSquareNorm, exist_ok=True)

    def build(cfg):
        d, W = cfg.width // cfg.heads, cfg.width
        rms = lambda name: RootMeanSquareNorm(name, W, cfg.eps)
        pos = RotaryPositions(d, 10000.0)
        blocks = [
            ParallelBlock(AttentionMixer("t.h.0.attn", W, cfg.heads, 1, d, "tail", False, pos),
                          DenseFeedForward("t.h.0.mlp", W, 2 * W, bias=True), rms("t.h.0.n_attn"), rms("t.h.0.n_mlp")),
            SequentialBlock(AttentionMixer("t.h.1.attn", W, cfg.heads, cfg.heads, d, "interleaved", False, pos),
                            DenseFeedForward("t.h.1.mlp", W, 2 * W, bias=False), rms("t.h.1.n1"), rms("t.h.1.n2")),
            ParallelBlock(AttentionMixer("t.h.2.attn", W, cfg.heads, 1, d, "tail", False, pos),
                          DenseFeedForward("t.h.2.mlp", W, 2 * W, bias=False), rms("t.h.2.n")),
        ]
        return ModelSpec(config=cfg, embedding=Embedding("t.embed", cfg.vocab_size, W), blocks=blocks,
                         order=[LayerCall(0, "one", 0), LayerCall(1, "all", 0), LayerCall(2, "one", 1)],
                         final_norm=rms("t.final"), head=OutputHead("t.head", cfg.vocab_size, W, "t.embed.weight"),
                         cache_groups=[CacheGroupSpec("one", CACHE_FULL, 2, 1, d), CacheGroupSpec("all", CACHE_FULL, 1, cfg.heads, d)])

    return NormConfig, build


def _plain_norm_toy(cfg, w, ids):
    T, W, nh = len(ids), cfg.width, cfg.heads
    d = W // nh
    x = w["t.embed.weight"][torch.as_tensor(ids)]
    rms = lambda h, n: h / torch.sqrt((h * h).mean(-1, keepdim=True) + cfg.eps) * w[n + ".weight"]
    cos, sin = P.rope_cos_sin(torch.arange(T), P.rope_inv_freq(d, 10000.0))

    def attn(h, p, layout):
        f = h @ w[p + ".query_key_value.weight"].T
        if layout == "tail":
            f = f.view(T, nh + 2, d)
            q, k, v = f[:, :nh], f[:, nh:nh + 1], f[:, nh + 1:]
        else:
            f = f.view(T, nh, 3, d)
            q, k, v = f[:, :, 0], f[:, :, 1], f[:, :, 2]
        return P.attention_scores_softmax(P.apply_rope(q, cos, sin), P.apply_rope(k, cos, sin), v) @ w[p + ".dense.weight"].T

    def ffn(h, p, bias):
        u = h @ w[p + ".dense_h_to_4h.weight"].T + (w[p + ".dense_h_to_4h.bias"] if bias else 0)
        return P.gelu(u) @ w[p + ".dense_4h_to_h.weight"].T + (w[p + ".dense_4h_to_h.bias"] if bias else 0)

    x = x + (ffn(rms(x, "t.h.0.n_mlp"), "t.h.0.mlp", True) + attn(rms(x, "t.h.0.n_attn"), "t.h.0.attn", "tail"))
    r = x + attn(rms(x, "t.h.1.n1"), "t.h.1.attn", "interleaved")
    x = r + ffn(rms(r, "t.h.1.n2"), "t.h.1.mlp", False)
    a = rms(x, "t.h.2.n")
    x = x + (ffn(a, "t.h.2.mlp", False) + attn(a, "t.h.2.attn", "tail"))
    return rms(x, "t.final") @ w["t.embed.weight"].T


@pytest.mark.parametrize("dtype,rel", [("float32", 5e-5), ("bfloat16", helpers.REL_BF16)])
def test_toy_architecture_with_a_norm_of_its_own(tmp_path, dtype, rel):
    """A norm without mean and bias, defined in this file with the plain interface alone, in every place a norm
    stands: the two norms of a parallel block, the one norm of another, both norms of a sequential block (whose
    input may arrive as a sum that is not formed yet) and the final norm on the wanted rows."""
    from safetensors.torch import load_file

    from pytorch_transformers_amd import AutoModelForCausalLM
    from pytorch_transformers_amd.config import register, unregister
    from pytorch_transformers_amd.engine.replay import Replayer
    from pytorch_transformers_amd.weights import write_random_model

    NormConfig, build = _define_norm_toy()
    register("toy-norm", NormConfig, build, exist_ok=True)
    try:
        cfg = NormConfig()
        folder = write_random_model(str(tmp_path / "norm"), cfg, seed=14, std=0.15, noise=0.1)
        w = {k: v.double() for k, v in load_file(f"{folder}/model.safetensors").items()}
        assert "t.h.0.n_attn.weight" in w and "t.h.0.n_attn.bias" not in w
        model = AutoModelForCausalLM.from_pretrained(folder, dtype=dtype)
        reqs = helpers.make_requests(cfg.vocab_size, [11, 40, 70, 5], seed=4)
        want = {rid: _plain_norm_toy(cfg, w, toks).float() for rid, toks in reqs.items()}
        rp = Replayer(model, 1024, max_slots=4)
        for name, records in (("whole", helpers.schedule_whole(reqs)), ("tail", helpers.schedule_tail(reqs, 16)),
                              ("batches", helpers.schedule_batches(reqs, 3))):
            got = helpers.run_schedule(rp, records)
            for rid in reqs:
                helpers.assert_close(got[rid], want[rid], rel, f"norm toy {dtype} {name} {rid}")
    finally:
        unregister("toy-norm")


# --- a sixth toy: its weight files hold query, key and value projections apart ---
def _define_split_toy():
    from pytorch_transformers_amd.config.base import ModelConfig
    from pytorch_transformers_amd.engine.spec import CACHE_FULL, CacheGroupSpec, LayerCall, ModelSpec
    from pytorch_transformers_amd.parts import (AttentionMixer, DenseFeedForward, Embedding, LayerNorm, OutputHead,
                                                RotaryPositions, SequentialBlock)

    @dataclasses.dataclass
    class SplitConfig(ModelConfig):
        model_type = "toy-split"
        vocab_size: int = 131
        width: int = 96
        heads: int = 6
        kv_heads: tuple = (2, 6, 1)  # per layer: grouped, one per head, one for all
        eps: float = 1e-5

    LAYOUTS = {2: "grouped", 6: "interleaved", 1: "tail"}

    def build(cfg):
        W, nh = cfg.width, cfg.heads
        d = W // nh
        pos = RotaryPositions(d, 10000.0)
        norm = lambda n: LayerNorm(n, W, cfg.eps)
        blocks = [SequentialBlock(AttentionMixer(f"s.h.{i}.attn", W, nh, nkv, d, LAYOUTS[nkv], True, pos, out_name="o_proj",
                                                 qkv_pieces=("q_proj", "k_proj", "v_proj")),
                                  DenseFeedForward(f"s.h.{i}.mlp", W, 2 * W, bias=False), norm(f"s.h.{i}.n1"), norm(f"s.h.{i}.n2"))
                  for i, nkv in enumerate(cfg.kv_heads)]
        return ModelSpec(config=cfg, embedding=Embedding("s.embed", cfg.vocab_size, W), blocks=blocks,
                         order=[LayerCall(i, f"g{i}", 0) for i in range(len(blocks))], final_norm=norm("s.final"),
                         head=OutputHead("s.head", cfg.vocab_size, W, "s.embed.weight"),
                         cache_groups=[CacheGroupSpec(f"g{i}", CACHE_FULL, 1, nkv, d) for i, nkv in enumerate(cfg.kv_heads)])

    return SplitConfig, build


def _plain_split_toy(cfg, w, ids):
    """Separate projections, heads in order; query head h reads KV head h // (heads / kv heads)."""
    T, W, nh = len(ids), cfg.width, cfg.heads
    d = W // nh
    x = w["s.embed.weight"][torch.as_tensor(ids)]
    ln = lambda h, n: P.layer_norm(h, w[n + ".weight"], w[n + ".bias"], cfg.eps)
    cos, sin = P.rope_cos_sin(torch.arange(T), P.rope_inv_freq(d, 10000.0))
    for i, nkv in enumerate(cfg.kv_heads):
        a = ln(x, f"s.h.{i}.n1")
        proj = lambda n, heads: (a @ w[f"s.h.{i}.attn.{n}.weight"].T + w[f"s.h.{i}.attn.{n}.bias"]).view(T, heads, d)
        q, k, v = proj("q_proj", nh), proj("k_proj", nkv), proj("v_proj", nkv)
        k, v = (t.repeat_interleave(nh // nkv, dim=1) for t in (k, v))
        o = P.attention_scores_softmax(P.apply_rope(q, cos, sin), P.apply_rope(k, cos, sin), v)
        x = x + o @ w[f"s.h.{i}.attn.o_proj.weight"].T + w[f"s.h.{i}.attn.o_proj.bias"]
        m = ln(x, f"s.h.{i}.n2")
        x = x + P.gelu(m @ w[f"s.h.{i}.mlp.dense_h_to_4h.weight"].T) @ w[f"s.h.{i}.mlp.dense_4h_to_h.weight"].T
    return ln(x, "s.final") @ w["s.embed.weight"].T


@pytest.mark.parametrize("dtype,rel", [("float32", 5e-5), ("bfloat16", helpers.REL_BF16)])
def test_toy_architecture_whose_files_hold_query_key_and_value_apart(tmp_path, dtype, rel):
    """The attention part runs one fused projection; this toy's weight files hold ``q_proj``, ``k_proj`` and
    ``v_proj`` apart, with grouped heads, one KV head per head, and one for all, and the loader lays their rows out
    as each layer's fused launch wants them.  The file is written by this test from matrices of its own; the plain
    implementation multiplies by the separate matrices."""
    from safetensors.torch import load_file, save_file

    from pytorch_transformers_amd import AutoModelForCausalLM
    from pytorch_transformers_amd.config import register, unregister
    from pytorch_transformers_amd.engine.replay import Replayer
    from pytorch_transformers_amd.weights import write_random_model

    SplitConfig, build = _define_split_toy()
    register("toy-split", SplitConfig, build, exist_ok=True)
    try:
        cfg = SplitConfig()
        folder = write_random_model(str(tmp_path / "split"), cfg, seed=21, std=0.15, noise=0.1)
        path = f"{folder}/model.safetensors"
        tensors = load_file(path)
        d = cfg.width // cfg.heads
        g = torch.Generator().manual_seed(3)
        for i, nkv in enumerate(cfg.kv_heads):  # the fused tensors go, separate ones of this test's making come
            for kind in ("weight", "bias"):
                fused = tensors.pop(f"s.h.{i}.attn.query_key_value.{kind}")
                for n, heads in (("q_proj", cfg.heads), ("k_proj", nkv), ("v_proj", nkv)):
                    shape = (heads * d, cfg.width) if kind == "weight" else (heads * d,)
                    tensors[f"s.h.{i}.attn.{n}.{kind}"] = (torch.randn(shape, generator=g) * 0.15).to(fused.dtype)
        save_file(tensors, path, metadata={"format": "pt"})
        w = {k: v.double() for k, v in tensors.items()}
        model = AutoModelForCausalLM.from_pretrained(folder, dtype=dtype)
        reqs = helpers.make_requests(cfg.vocab_size, [9, 37, 66], seed=8)
        want = {rid: _plain_split_toy(cfg, w, toks).float() for rid, toks in reqs.items()}
        rp = Replayer(model, 1024, max_slots=3)
        for name, records in (("whole", helpers.schedule_whole(reqs)), ("tail", helpers.schedule_tail(reqs, 16)),
                              ("batches", helpers.schedule_batches(reqs, 2))):
            got = helpers.run_schedule(rp, records)
            for rid in reqs:
                helpers.assert_close(got[rid], want[rid], rel, f"split toy {dtype} {name} {rid}")
    finally:
        unregister("toy-split")
