"""Decode and prefill throughput at Falcon-7B layer sizes with random weights, on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one decode step of the batch (model step from the cache plus the greedy choice of the
next token, fed back).  The default run: batch 8, prompts of 1,024 synthetic token ids, the timed steps
right behind the prompt.  One JSON line is printed: decode tokens a second as ``value`` (all timed steps
over their time; ``ms_per_step_median`` is the median step by events between the steps), the
prefill of 2,048 tokens under ``prefill``, the decode step's HBM roofline under ``roofline``, and under
``points`` (flat):

* ``decode_b1`` / ``decode_b8`` / ``decode_b64``: tokens a second over the range of contexts that the
  configuration names, every decode step from 1,024 tokens to 2,048 in one run; ``decode_b64_ctx1568`` and so on
  are short runs around three contexts of that range; each with ``..._frac``, the fraction of the HBM roofline;
* ``decode_b8_ctx4128`` ... ``decode_b32_ctx16416``: short runs at batch 8 and 32 around contexts of 4,128, 8,224 and
  16,416 tokens, where the live sequences' keys and values weigh as much as the weights;
* ``decode_b8_untuned``: the same step with the built-in choices between kernels, before ``model.tune()`` has
  timed any (what a process runs that neither tunes nor loads a tuning table);
* ``falcon11b_...`` / ``falcon40b_...``: decode at batch 8 and 64 and one batch of whole requests of unequal
  lengths through ``generate()`` at the layer sizes of Falcon2-11B and Falcon-40B, each measured by a child
  process with a time limit, so that a failure there costs those figures and nothing else.

Under ``kernels``: the launches of a decode step at batch 8 and 64 and of the prefill, each with its time (events
around every launch of a step that is launched directly), the bytes it has to read or its arithmetic, and the
fraction of the published peak.
"""
import argparse
import json
import os
import statistics
import subprocess
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X, published
PEAK_TFLOPS = {"bf16": 2500.0, "fp32": 157.3}  # dense MFMA, published


def falcon7b_config(layers):
    from pytorch_transformers_amd import FalconConfig

    # the layer sizes of the published Falcon-7B configuration
    return FalconConfig(vocab_size=65024, hidden_size=4544, num_hidden_layers=layers, num_attention_heads=71,
                        multi_query=True, new_decoder_architecture=False, parallel_attn=True, bias=False, alibi=False,
                        ffn_hidden_size=18176, rope_theta=10000.0, layer_norm_epsilon=1e-5,
                        max_position_embeddings=2048, tie_word_embeddings=True)


def falcon_config(sizes, layers):
    """Layer sizes of the published models; "7b" is the default run, the others are for comparison."""
    from pytorch_transformers_amd import FalconConfig

    if sizes == "7b":
        return falcon7b_config(layers or 32), 32
    if sizes == "11b":  # Falcon2-11B: 32 heads in 8 groups of head size 128, one norm
        return FalconConfig(vocab_size=65024, hidden_size=4096, num_hidden_layers=layers or 60, num_attention_heads=32,
                            num_kv_heads=8, new_decoder_architecture=True, num_ln_in_parallel_attn=1,
                            parallel_attn=True, bias=False, alibi=False, ffn_hidden_size=16384, rope_theta=500042.0,
                            layer_norm_epsilon=1e-5, max_position_embeddings=8192, tie_word_embeddings=False), 60
    if sizes == "40b":  # Falcon-40B: 128 heads in 8 groups of head size 64, two norms
        return FalconConfig(vocab_size=65024, hidden_size=8192, num_hidden_layers=layers or 60, num_attention_heads=128,
                            num_kv_heads=8, new_decoder_architecture=True, num_ln_in_parallel_attn=2,
                            parallel_attn=True, bias=False, alibi=False, ffn_hidden_size=32768, rope_theta=10000.0,
                            layer_norm_epsilon=1e-5, max_position_embeddings=2048, tie_word_embeddings=False), 60
    raise ValueError(sizes)


def weight_bytes(cfg, elem):
    H, F, Q = cfg.hidden_size, cfg.ffn_hidden_size, cfg.qkv_out_dim
    per_layer = (Q * H + H * H + 2 * F * H) * elem
    return cfg.num_hidden_layers * per_layer + cfg.vocab_size * H * elem


def kv_bytes_per_token(cfg, elem):
    return cfg.num_hidden_layers * 2 * cfg.kv_heads * cfg.head_dim * elem


def prefill_flops(cfg, T):
    H, F, Q = cfg.hidden_size, cfg.ffn_hidden_size, cfg.qkv_out_dim
    linear = 2.0 * T * (Q * H + H * H + 2 * F * H) * cfg.num_hidden_layers
    attn = 2.0 * cfg.head_dim * cfg.num_attention_heads * T * (T + 1) * cfg.num_hidden_layers
    head = 2.0 * cfg.vocab_size * H
    return linear + attn + head


def run_decode(model, sampler_cls, gen_cfg, batch, prompt_len, steps, warmup, seed=0, start_ctx=None, per_step=False):
    """Prefill ``batch`` prompts of ``prompt_len`` tokens, then time ``steps`` decode steps; returns (seconds, mean
    context of the timed steps, median milliseconds of a step or None).  With ``start_ctx`` nothing is prefilled:
    the sequences are set to that length (pages reserved, lengths committed; the keys and values there are
    zeros) and decoding goes on from there, which puts the timed steps at any context at no cost.  ``per_step``:
    an event is recorded behind every step, for the median."""
    import torch

    g = torch.Generator().manual_seed(seed)
    page = model.page_size
    first = prompt_len if start_ctx is None else start_ctx
    total = first + warmup + steps + 1
    cache = model.new_cache(batch * ((total + page - 1) // page * page), max_slots=batch)
    sampler = sampler_cls(gen_cfg, model.vocab_size, model.device)
    slots = [cache.alloc() for _ in range(batch)]
    if start_ctx is None:
        prompts = torch.randint(0, model.vocab_size, (batch, prompt_len), generator=g).tolist()
        logits = model.step(cache, slots, prompts, "last")
    else:
        cache.reserve(slots, [start_ctx - 1] * batch)
        cache.commit(slots, [start_ctx - 1] * batch)
        logits = model.step(cache, slots, torch.randint(0, model.vocab_size, (batch, 1), generator=g).tolist(), "last")
    rng = list(range(batch))
    pending, _ = sampler.sample(logits, rng_seq=rng, rng_step=[0] * batch, need_scores=False, ahead=True)

    def one(k):  # as generate() runs a step: launched from the tokens on the device, which the host reads meanwhile
        nonlocal pending
        lg = model.step(cache, slots, pending, "last", own_logits=False)
        chosen, _ = sampler.sample(lg, rng_seq=rng, rng_step=[k] * batch, need_scores=False, ahead=True)
        pending.tolist()
        pending = chosen

    for k in range(warmup):
        one(k)
    marks = []
    if per_step:
        marks = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    if per_step:
        marks[0].record()
    for k in range(steps):
        one(warmup + k)
        if per_step:
            marks[k + 1].record()
    pending.tolist()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    median = statistics.median(marks[k].elapsed_time(marks[k + 1]) for k in range(steps)) if per_step else None
    mean_ctx = first + warmup + (steps + 1) / 2.0
    for s in slots:
        cache.free(s)
    del cache
    return dt, mean_ctx, median


# Near the start, the middle and the end of decoding from 1,024 towards 2,048 tokens, each clear of the lengths at
# which a captured decode step is exchanged for the next one (multiples of 512): a run of a few steps across such
# a length would time the capture, which decoding meets twice in a thousand steps.
RANGE_CONTEXTS = (1056, 1568, 2016)


# Contexts past the metric's range (the configuration's own limit is 2,048 positions; rotation has no limit of its
# own): where the keys and values of the live sequences weigh as much as the weights.  Clear of the captured steps'
# exchanges, as above.
LONG_CONTEXTS = (4128, 8224, 16416)
LONG_BATCHES = (8, 32)


def decode_over_range(model, sampler_cls, gen_cfg, cfg, elem, batch, steps=16, warmup=4, contexts=RANGE_CONTEXTS,
                      mean=True):
    """Decode steps of ``batch`` sequences timed around each of ``contexts``; returns flat figures: tokens a second
    and fraction of the HBM roofline at each context, and (``mean``) over the range (the mean of the step times)."""
    out, ms_all, frac_all = {}, [], []
    for c in contexts:
        dt, mean_ctx, _ = run_decode(model, sampler_cls, gen_cfg, batch, 0, steps, warmup, seed=c,
                                     start_ctx=max(1, c - warmup - steps // 2))
        ms = dt / steps * 1e3
        gbs = (weight_bytes(cfg, elem) + batch * mean_ctx * kv_bytes_per_token(cfg, elem)) / (ms * 1e-3) / 1e9
        out[f"decode_b{batch}_ctx{c}"] = round(batch / ms * 1e3, 2)
        out[f"decode_b{batch}_ctx{c}_frac"] = round(gbs / HBM_PEAK_GBS, 4)
        ms_all.append(ms)
        frac_all.append(gbs / HBM_PEAK_GBS)
    if not mean:
        return out
    mean_ms = sum(ms_all) / len(ms_all)
    out[f"decode_b{batch}"] = round(batch / mean_ms * 1e3, 2)
    out[f"decode_b{batch}_frac"] = round(sum(f * m for f, m in zip(frac_all, ms_all)) / sum(ms_all), 4)
    return out


def decode_whole_range(model, sampler_cls, gen_cfg, cfg, elem, batch, first=1024, last=2048):
    """Every decode step from a context of ``first`` tokens to one of ``last``, as one run (the captured steps that
    are exchanged on the way included): tokens a second and the fraction of the HBM roofline over the run."""
    steps = last - first - 1
    dt, mean_ctx, _ = run_decode(model, sampler_cls, gen_cfg, batch, 0, steps, 1, start_ctx=first)
    ms = dt / steps * 1e3
    gbs = (weight_bytes(cfg, elem) + batch * mean_ctx * kv_bytes_per_token(cfg, elem)) / (ms * 1e-3) / 1e9
    return {f"decode_b{batch}": round(batch / ms * 1e3, 2), f"decode_b{batch}_frac": round(gbs / HBM_PEAK_GBS, 4),
            f"decode_b{batch}_steps": steps}


def run_prefill(model, T, reps=3, seed=1):
    import torch

    g = torch.Generator().manual_seed(seed)
    prompt = torch.randint(0, model.vocab_size, (T,), generator=g).tolist()
    page = model.page_size
    cache = model.new_cache((T + page - 1) // page * page, max_slots=1)
    best = None
    for r in range(reps + 1):
        slot = cache.alloc()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        model.step(cache, [slot], [prompt], "last")
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        cache.free(slot)
        if r > 0:  # the first run warms the library's kernel selection
            best = dt if best is None else min(best, dt)
    return best


KERNEL_LABELS = {
    "pta_gemm_skinny_pair_qkv_bf16": "qkv+up (few rows; rotation and cache write in its epilogue)",
    "pta_gemm_skinny_pair_bf16": "qkv+up (few rows)",
    "pta_gemm_splitk_pair_reduced_qkv_bf16": "qkv+up (decode batch; reduction rotates and writes the cache)",
    "pta_gemm_splitk_pair_reduced_bf16": "qkv+up (decode batch)",
    "pta_gemm_splitk_pair_bf16": "dense+down (partial sums)",
    "pta_gemm_splitk_bf16": "product, K split",
    "pta_gemm_skinny_bf16": "lm_head / product of few rows",
    "pta_layernorm_sum": "residual sum + LayerNorm",
    "pta_attn_mfma": "attention over the cache (+ merge of key ranges)",
    "library_mm": "vendor library products",
    "pta_epilogue": "bias / activation / additions pass",
    "pta_qkv_rope_cache": "split, rotation, cache write",
}


def kernel_figures(model, ops, dtype, step, attn_bytes=0.0, attn_flops=0.0):
    """Per entry point of the kernel library: time of one step launched directly with events around every launch
    (a captured step cannot hold events), the bytes it has to read or the arithmetic it does, and the achieved
    rate as a fraction of the published peak.  ``step`` runs one step."""
    import torch

    graphs, model.use_graphs = model.use_graphs, False
    try:
        step()  # the shapes' first launch outside the timing
        torch.cuda.synchronize()
        ops.timing_hint.update(attn_bytes=attn_bytes, attn_flops=attn_flops)
        ops.start_timing()
        step()
        raw = ops.stop_timing()
    finally:
        model.use_graphs = graphs
    out = {}
    for name, r in sorted(raw.items(), key=lambda kv: -kv[1]["us"]):
        rec = {"what": KERNEL_LABELS.get(name, name), "calls": r["calls"], "us": round(r["us"], 1)}
        if r["flops"] and r["flops"] / max(r["bytes"], 1.0) > 300:  # bound by arithmetic
            tf = r["flops"] / r["us"] / 1e6
            rec.update({"TFLOP/s": round(tf, 1), "frac": round(tf / PEAK_TFLOPS[dtype], 3)})
        elif r["bytes"]:
            gbs = r["bytes"] / r["us"] / 1e3
            rec.update({"GB/s": round(gbs, 1), "frac": round(gbs / HBM_PEAK_GBS, 3)})
        out[name.replace("pta_", "")] = rec
    return out


def decode_kernels(model, ops, sampler_cls, gen_cfg, cfg, dtype, elem, batch, prompt_len):
    """The kernels of one decode step of ``batch`` sequences at a context of ``prompt_len``."""
    import torch

    g = torch.Generator().manual_seed(3)
    prompts = torch.randint(0, model.vocab_size, (batch, prompt_len), generator=g).tolist()
    page = model.page_size
    cache = model.new_cache(batch * ((prompt_len + 8 + page - 1) // page * page), max_slots=batch)
    slots = [cache.alloc() for _ in range(batch)]
    model.step(cache, slots, prompts, "last")
    per_layer_kv = batch * (prompt_len + 1) * 2 * cfg.kv_heads * cfg.head_dim * elem
    figures = kernel_figures(model, ops, dtype, lambda: model.step(cache, slots, [[1]] * batch, "last"),
                             attn_bytes=per_layer_kv)
    for s_ in slots:
        cache.free(s_)
    return figures


def prefill_kernels(model, ops, cfg, dtype, T):
    import torch

    g = torch.Generator().manual_seed(4)
    prompt = torch.randint(0, model.vocab_size, (T,), generator=g).tolist()
    page = model.page_size
    cache = model.new_cache((T + page - 1) // page * page * 2, max_slots=2)

    def step():
        slot = cache.alloc()
        model.step(cache, [slot], [prompt], "last")
        cache.free(slot)

    return kernel_figures(model, ops, dtype, step,
                          attn_flops=2.0 * cfg.head_dim * cfg.num_attention_heads * T * (T + 1))


MIXED = {"7b": (8, 1024, 1024, 128), "11b": (16, 128, 4096, 256), "40b": (32, 64, 1536, 512)}


def run_mixed(model, batch, lo, hi, new, seed=2):
    """One batch of prompts with seeded uniform lengths in [lo, hi] through ``generate`` (greedy, no stop
    token): the whole request, prefill included.  Returns (seconds, prompt tokens)."""
    import torch

    g = torch.Generator().manual_seed(seed)
    lens = torch.randint(lo, hi + 1, (batch,), generator=g).tolist()
    prompts = [torch.randint(0, model.vocab_size, (n,), generator=g).tolist() for n in lens]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    out = model.generate(prompts, max_new_tokens=new, do_sample=False, eos_token_id=None)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    assert all(len(o) == len(p) + new for o, p in zip(out, prompts))
    run_mixed.lens = lens
    return dt, sum(lens)


def mixed_record(model, ops, cfg, sizes, dtype, elem):
    """One batch of whole requests of unequal lengths through ``generate()`` (prefill included), with the floor of
    its arithmetic and bytes; the choices that are timed are timed first, for the shapes of this run."""
    batch, lo, hi, new = MIXED[sizes]
    with ops.live_tuning():  # the choices that are timed, for the shapes of this run; nothing of it is timed below
        run_mixed(model, batch, lo, hi, 2)
    ops.release_flush()
    # ... and the decode attention's cut at the (longest, mean) contexts that the run passes through
    lens = run_mixed.lens
    model.tune(prompt_lens=(), batches=(batch,),
               contexts=sorted({(max(lens) + k, sum(lens) // len(lens) + k) for k in range(1, new + 1, 64)}))
    dt, prompt_tokens = run_mixed(model, batch, lo, hi, new)
    # what the request has to do at the least: the prompts' arithmetic, and for every decode step all weights once
    # and the live sequences' keys and values (a sequence of n prompt tokens is n + k long at step k)
    flops = sum(prefill_flops(cfg, n) for n in run_mixed.lens)
    kv = kv_bytes_per_token(cfg, elem)
    decode_bytes = new * weight_bytes(cfg, elem) + sum(kv * (n * new + new * (new + 1) / 2) for n in run_mixed.lens)
    floor = flops / (PEAK_TFLOPS[dtype] * 1e12) + decode_bytes / (HBM_PEAK_GBS * 1e9)
    return {"metric": f"falcon{sizes}_mixed_generated_tokens_per_second",
            "value": round(batch * new / dt, 1), "unit": "tokens/s", "seconds": round(dt, 3),
            "batch": batch, "prompt_tokens": prompt_tokens, "new_tokens_each": new,
            "prompt_lengths": f"U[{lo},{hi}]", "layers": cfg.num_hidden_layers, "dtype": dtype,
            "roofline": {"bound": "prefill arithmetic + decode hbm", "prefill_tflop": round(flops / 1e12, 1),
                         "decode_gb": round(decode_bytes / 1e9, 1), "floor_s": round(floor, 3),
                         "frac": round(floor / dt, 4)},
            "note": "whole requests, prefill included; greedy, no stop token"}


EXTRA_SIZES = (("11b", 170), ("40b", 270))  # other layer sizes measured by a child process, and its time limit in seconds


def extra_points(sizes, limit, dtype):
    """Flat figures of ``--extra-record`` at ``sizes`` from a child process (the 7B model of this process keeps its
    memory; both fit).  A child that fails or overruns its limit leaves an ``..._error`` entry and nothing else."""
    tag = f"falcon{sizes}"
    cmd = [sys.executable, os.path.abspath(__file__), "--sizes", sizes, "--dtype", dtype, "--extra-record"]
    try:
        done = subprocess.run(cmd, capture_output=True, text=True, timeout=limit, cwd=ROOT)
    except subprocess.TimeoutExpired:
        return {f"{tag}_error": f"not done within {limit} s"}
    lines = [ln for ln in done.stdout.splitlines() if ln.startswith("{")]
    if done.returncode != 0 or not lines:
        return {f"{tag}_error": f"exit code {done.returncode}: {done.stderr.strip()[-200:]}"}
    return {f"{tag}_{k}": v for k, v in json.loads(lines[-1]).items()}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--prompt-len", type=int, default=1024)
    ap.add_argument("--layers", type=int, default=0, help="fewer than the model has only where memory or time needs it")
    ap.add_argument("--sizes", default="7b", choices=["7b", "11b", "40b"],
                    help="layer sizes: Falcon-7B (the default run), Falcon2-11B or Falcon-40B")
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "fp32"])
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 / batch 64 / prefill measurements")
    ap.add_argument("--no-extra", action="store_true", help="skip the figures at Falcon2-11B and Falcon-40B layer sizes")
    ap.add_argument("--mixed", action="store_true",
                    help="one batch of unequal prompts through generate(): 11b 16 x U[128,4096] + 256 new, "
                         "40b 32 x U[64,1536] + 512 new; prints its own record")
    ap.add_argument("--extra-record", action="store_true",
                    help="decode at batch 8 and 64 over the range of contexts and the --mixed request, as one flat record "
                         "(what the default run asks a child process for at the other layer sizes)")
    ap.add_argument("--only-prefill", action="store_true",
                    help="run the prefill alone and print its record (for profiling)")
    ap.add_argument("--prefill-tokens", type=int, default=2048,
                    help="with --only-prefill: the prompt's length (the default run's prefill is of 2,048 tokens)")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        return 2

    import torch

    from pytorch_transformers_amd import AutoModelForCausalLM, GenerationConfig, ops
    from pytorch_transformers_amd.sampling import Sampler

    ops.load_library()
    cfg, full_layers = falcon_config(args.sizes, args.layers)
    args.layers = cfg.num_hidden_layers
    dtype = "bfloat16" if args.dtype == "bf16" else "float32"
    elem = 2 if args.dtype == "bf16" else 4
    model = AutoModelForCausalLM.from_config(cfg, seed=0, dtype=dtype, device="cuda:0")
    gen_cfg = GenerationConfig(do_sample=False, eos_token_id=None)
    if args.mixed:
        print(json.dumps(mixed_record(model, ops, cfg, args.sizes, args.dtype, elem)))
        return 0
    if args.extra_record:
        model.tune(prompt_lens=(), batches=(8, 64), contexts=RANGE_CONTEXTS)
        rec = {}
        for b in (8, 64):
            rec.update(decode_over_range(model, Sampler, gen_cfg, cfg, elem, b, steps=12, warmup=3))
        mixed = mixed_record(model, ops, cfg, args.sizes, args.dtype, elem)
        rec.update({"mixed": mixed["value"], "mixed_seconds": mixed["seconds"], "mixed_frac": mixed["roofline"]["frac"],
                    "mixed_batch": mixed["batch"], "mixed_new_tokens_each": mixed["new_tokens_each"],
                    "mixed_prompt_lengths": mixed["prompt_lengths"], "layers": args.layers})
        print(json.dumps(rec))
        return 0
    # the choices between kernels that are timed rather than ruled, once, for the shapes measured below; the timed
    # steps themselves time nothing
    if args.only_prefill:
        T = args.prefill_tokens
        model.tune(prompt_lens=(T,), batches=())
        pt = run_prefill(model, T)
        print(json.dumps({"prefill": {"value": round(T / pt, 1), "tokens": T, "ms": round(pt * 1e3, 3),
                                      "frac": round(prefill_flops(cfg, T) / pt / (PEAK_TFLOPS[args.dtype] * 1e12), 4)},
                          "layers": args.layers, "dtype": args.dtype}))
        return 0
    points = {}
    if not args.no_points:  # before anything is timed: the step as a process runs it that neither tunes nor loads a table
        d, _, _ = run_decode(model, Sampler, gen_cfg, args.batch, args.prompt_len, 16, 4)
        points[f"decode_b{args.batch}_untuned"] = round(args.batch * 16 / d, 2)
    model.tune(prompt_lens=(2048,), batches=sorted({args.batch, 1, 64}),
               contexts=sorted({args.prompt_len + 1, args.prompt_len + args.warmup + args.steps, *RANGE_CONTEXTS}))

    dt, mean_ctx, median_ms = run_decode(model, Sampler, gen_cfg, args.batch, args.prompt_len, args.steps, args.warmup,
                                         per_step=True)
    ms = dt / args.steps * 1e3
    value = args.batch * args.steps / dt
    step_bytes = weight_bytes(cfg, elem) + args.batch * mean_ctx * kv_bytes_per_token(cfg, elem)
    achieved = step_bytes / (ms * 1e-3) / 1e9

    out = {
        "metric": f"falcon{args.sizes}_decode_tokens_per_second", "value": round(value, 2), "unit": "tokens/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 4), "ms_per_step_median": round(median_ms, 4),
        "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": args.dtype,
        "data": "synthetic token ids, random weights N(0, 0.02)",
        "config": {"model": f"falcon-{args.sizes} layer sizes", "layers": args.layers, "layers_of_config": full_layers,
                   "hidden": cfg.hidden_size, "heads": cfg.num_attention_heads, "kv_heads": cfg.kv_heads,
                   "head_dim": cfg.head_dim, "ffn": cfg.ffn_hidden_size, "vocab": cfg.vocab_size,
                   "global_batch": args.batch, "prompt_len": args.prompt_len, "seq_len": 2048,
                   "timed_ctx_from": args.prompt_len + args.warmup + 1,
                   "timed_ctx_to": args.prompt_len + args.warmup + args.steps,
                   "decode": "greedy", "parallelism": "single"},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4)},
    }
    if not args.no_points:
        T = 2048
        pt = run_prefill(model, T)
        flops = prefill_flops(cfg, T)
        out["prefill"] = {"value": round(T / pt, 1), "tokens": T, "ms": round(pt * 1e3, 3),
                          "frac": round(flops / pt / (PEAK_TFLOPS[args.dtype] * 1e12), 4)}
        for b in sorted({1, args.batch, 64}):
            points.update(decode_over_range(model, Sampler, gen_cfg, cfg, elem, b))
            # ... and what the metric names: every step from prompts of 1,024 tokens to 2,048, in place of the mean of three
            points.update(decode_whole_range(model, Sampler, gen_cfg, cfg, elem, b, 1024, 2048))
        if args.sizes == "7b" and args.layers == full_layers:  # long contexts: decode_b8_ctx4128 ... decode_b32_ctx16416
            model.tune(prompt_lens=(), batches=LONG_BATCHES, contexts=LONG_CONTEXTS)
            for b in LONG_BATCHES:
                points.update(decode_over_range(model, Sampler, gen_cfg, cfg, elem, b, steps=12, warmup=3,
                                                contexts=LONG_CONTEXTS, mean=False))
        out["points"] = points
        if args.dtype == "bf16":
            out["kernels"] = {
                f"decode_b{args.batch}": decode_kernels(model, ops, Sampler, gen_cfg, cfg, args.dtype, elem, args.batch, args.prompt_len),
                "decode_b64": decode_kernels(model, ops, Sampler, gen_cfg, cfg, args.dtype, elem, 64, args.prompt_len),
                "prefill_2048": prefill_kernels(model, ops, cfg, args.dtype, 2048),
            }
        if args.sizes == "7b" and not args.no_extra:
            for sizes, limit in EXTRA_SIZES:
                points.update(extra_points(sizes, limit, args.dtype))
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
