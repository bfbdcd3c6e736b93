"""A plain, slow Falcon: whole sequences, no cache, one function per part.

Written from the reference's formulas (each function cites the reference's
file:line); it imports nothing from the engine, reads ``config.json`` as
a dict and the weights with safetensors' own loader.  Arithmetic is float64 by
default, so what the 32-bit engine is compared with is closer to exact than the
engine itself; the places where the reference rounds on purpose (ALiBi's
bfloat16 slopes) are reproduced.

A sequence is a list of token ids; every function works on one sequence.
"""
from __future__ import annotations

import json
import math
import os
from typing import Dict, List, Optional, Sequence

import torch

DT = torch.float64


# --- files -----------------------------------------------------------------
def read_model(folder: str, dtype=DT, device=None):
    """config.json as a dict, tensors by name (src/transformers/modeling_utils.py:3680-3695, :493-560).
    ``device``: where the tensors are put (default: the CPU); every function below computes where its inputs lie."""
    from safetensors.torch import load_file

    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    single = os.path.join(folder, "model.safetensors")
    if os.path.isfile(single):
        tensors = load_file(single)
    else:
        with open(os.path.join(folder, "model.safetensors.index.json")) as f:
            wm = json.load(f)["weight_map"]
        tensors = {}
        for shard in sorted(set(wm.values())):
            tensors.update(load_file(os.path.join(folder, shard)))
    return cfg, {k: v.to(device=device, dtype=dtype) for k, v in tensors.items()}


def cfg_defaults(cfg: dict) -> dict:
    """Defaults of FalconConfig (src/transformers/models/falcon/configuration_falcon.py:144-200)."""
    c = dict(vocab_size=65024, hidden_size=4544, num_hidden_layers=32, num_attention_heads=71,
             num_ln_in_parallel_attn=None, layer_norm_epsilon=1e-5, num_kv_heads=None, alibi=False,
             new_decoder_architecture=False, multi_query=True, parallel_attn=True, bias=False,
             rope_theta=10000.0, rope_scaling=None, ffn_hidden_size=None, tie_word_embeddings=True)
    c.update(cfg)
    if c["num_kv_heads"] is None:  # :184
        c["num_kv_heads"] = c["num_attention_heads"]
    if c["ffn_hidden_size"] is None:  # :195-198
        c["ffn_hidden_size"] = 4 * c["hidden_size"]
    if c["num_ln_in_parallel_attn"] is None and c["new_decoder_architecture"]:  # modeling_falcon.py:599-600
        c["num_ln_in_parallel_attn"] = 2
    return c


# --- parts -------------------------------------------------------------------
def layer_norm(x, w, b, eps):
    """torch.nn.LayerNorm over the last axis, biased variance
    (constructed at src/transformers/models/falcon/modeling_falcon.py:603-612, :843)."""
    mean = x.mean(-1, keepdim=True)
    var = ((x - mean) ** 2).mean(-1, keepdim=True)
    return (x - mean) / torch.sqrt(var + eps) * w + b


def gelu(x):
    """Exact GELU (src/transformers/activations.py:59-78, the non-approximate branch)."""
    return 0.5 * x * (1.0 + torch.erf(x / math.sqrt(2.0)))


def linear(x, w, b=None):
    """FalconLinear: x @ W.T, then + b (src/transformers/models/falcon/modeling_falcon.py:67-72)."""
    y = x @ w.T
    return y if b is None else y + b


def rope_inv_freq(head_dim: int, theta: float, factor: float = 1.0):
    """inv_freq = 1 / theta^(2i/d) in 32-bit (src/transformers/modeling_rope_utils.py:67);
    linear scaling divides by the factor (:108)."""
    inv = 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=torch.int64).float() / head_dim))
    return inv / factor if factor != 1.0 else inv


def rope_dynamic_inv_freq(head_dim: int, theta: float, factor: float, max_pos: int, seq_len: int):
    """Dynamic NTK (src/transformers/modeling_rope_utils.py:149-158): up to the trained context the trained
    frequencies, beyond it those of a stretched base; 32-bit arithmetic as there (the length arrives as an integer
    tensor, src/transformers/models/falcon/modeling_falcon.py:142)."""
    seq_len = seq_len if seq_len > max_pos else max_pos  # :152
    n = torch.tensor(seq_len, dtype=torch.int64)
    base = theta * ((factor * n / max_pos) - (factor - 1)) ** (head_dim / (head_dim - 2))  # :155
    return 1.0 / (base ** (torch.arange(0, head_dim, 2, dtype=torch.int64).float() / head_dim))  # :156


def rope_parameters(c, seq_len: Optional[int] = None):
    """(inv_freq, factor on cos and sin) for a configuration's ``rope_scaling``
    (src/transformers/modeling_rope_utils.py: default :58-68, linear :108, dynamic :112-160, yarn :163-239,
    longrope :242-302, llama3 :310-341).  ``seq_len`` matters to ``dynamic`` alone: Falcon's rotary module hands
    the length to the types whose name holds "dynamic" and to no other
    (src/transformers/models/falcon/modeling_falcon.py:155-157), so ``longrope`` always takes its short factors."""
    d = c["hidden_size"] // c["num_attention_heads"]
    theta = float(c["rope_theta"])
    rs = c.get("rope_scaling") or {}
    kind = rs.get("rope_type", rs.get("type", "default"))
    base = rope_inv_freq(d, theta)
    if kind == "dynamic":
        return rope_dynamic_inv_freq(d, theta, float(rs["factor"]), c["max_position_embeddings"], seq_len or 0), 1.0
    if kind == "longrope":  # :276-300 with seq_len None
        factor, scale = rs.get("factor"), rs.get("attention_factor")
        trained = c["max_position_embeddings"]
        if c.get("original_max_position_embeddings"):  # :283-287
            trained = c["original_max_position_embeddings"]
            factor = c["max_position_embeddings"] / trained
        if scale is None:  # :290-294
            scale = 1.0 if factor <= 1.0 else math.sqrt(1 + math.log(factor) / math.log(trained))
        ext = torch.tensor(rs["short_factor"], dtype=torch.float32)
        shape = torch.arange(0, d, 2, dtype=torch.int64).float() / d
        return 1.0 / (ext * theta ** shape), float(scale)
    if kind == "linear":
        return base / float(rs["factor"]), 1.0
    if kind == "yarn":
        factor, ctx = float(rs["factor"]), c["max_position_embeddings"]
        scale = rs.get("attention_factor")
        if scale is None:
            scale = 0.1 * math.log(factor) + 1.0
        # pair index at which a frequency makes `rot` rotations over the trained context
        where = lambda rot: (d * math.log(ctx / (rot * 2 * math.pi))) / (2 * math.log(theta))
        lo = max(math.floor(where(rs.get("beta_fast") or 32)), 0)
        hi = min(math.ceil(where(rs.get("beta_slow") or 1)), d - 1)
        if lo == hi:
            hi += 0.001
        out = torch.empty(d // 2)
        for i in range(d // 2):
            ramp = min(max((i - lo) / (hi - lo), 0.0), 1.0)  # 0: as trained, 1: interpolated
            out[i] = float(base[i]) / factor * ramp + float(base[i]) * (1 - ramp)
        return out, float(scale)
    if kind == "llama3":
        factor, lo_f, hi_f = float(rs["factor"]), float(rs["low_freq_factor"]), float(rs["high_freq_factor"])
        old = rs["original_max_position_embeddings"]
        out = base.clone()
        for i in range(d // 2):
            wavelen = 2 * math.pi / float(base[i])
            if wavelen > old / lo_f:
                out[i] = base[i] / factor
            elif not wavelen < old / hi_f:
                smooth = (old / wavelen - lo_f) / (hi_f - lo_f)
                out[i] = (1 - smooth) * base[i] / factor + smooth * base[i]
        return out, 1.0
    return base, 1.0


def rope_cos_sin(positions, inv_freq, dtype=DT, scale=1.0):
    """angles = position * inv_freq in 32-bit, doubled along the last axis
    (src/transformers/models/falcon/modeling_falcon.py:155-164)."""
    freqs = positions.float()[:, None] * inv_freq.float().to(positions.device)[None, :]
    emb = torch.cat((freqs, freqs), dim=-1)
    return (emb.cos() * scale).to(dtype), (emb.sin() * scale).to(dtype)


def rotate_half(x):
    """(-x2, x1) of the two halves of the last axis (src/transformers/models/falcon/modeling_falcon.py:76-80)."""
    h = x.shape[-1] // 2
    return torch.cat((-x[..., h:], x[..., :h]), dim=-1)


def apply_rope(x, cos, sin):
    """x*cos + rotate_half(x)*sin; x is [T, heads, d], cos/sin [T, d]
    (src/transformers/models/falcon/modeling_falcon.py:104-108)."""
    return x * cos[:, None, :] + rotate_half(x) * sin[:, None, :]


def alibi_slopes(nh: int):
    """src/transformers/models/falcon/modeling_falcon.py:175-188, in 32-bit."""
    n2 = 2 ** math.floor(math.log2(nh))
    base = torch.tensor(2 ** (-(2 ** -(math.log2(n2) - 3))), dtype=torch.float32)
    slopes = torch.pow(base, torch.arange(1, 1 + n2, dtype=torch.int32))
    if n2 != nh:
        extra_base = torch.tensor(2 ** (-(2 ** -(math.log2(2 * n2) - 3))), dtype=torch.float32)
        rem = min(n2, nh - n2)
        slopes = torch.cat([slopes, torch.pow(extra_base, torch.arange(1, 1 + 2 * rem, 2, dtype=torch.int32))])
    return slopes


def alibi_bias(nh: int, n_keys: int, head_dim: int, dtype=DT, bf16_compat: bool = True):
    """[heads, keys]: bf16(slope) * position formed in bfloat16 (:196-198), then / sqrt(d) in the
    model's type (:1078-1085).  ``bf16_compat=False`` (not the reference): the exact product."""
    pos = torch.arange(n_keys, dtype=torch.int64)
    if not bf16_compat:
        return (alibi_slopes(nh)[:, None].to(dtype) * pos[None, :].to(dtype)) / math.sqrt(head_dim)
    alibi = alibi_slopes(nh)[:, None].bfloat16() * pos[None, :]  # bfloat16 result, as in the reference
    return alibi.to(dtype) / math.sqrt(head_dim)


def split_heads(fused, c):
    """[T, Qout] -> q [T, nh, d], k and v [T, nkv, d]
    (src/transformers/models/falcon/modeling_falcon.py:269-298; the reference then broadcasts k, v
    to every query head, :286-289, which `attention` does by indexing)."""
    T = fused.shape[0]
    nh = c["num_attention_heads"]
    d = c["hidden_size"] // nh
    if c["new_decoder_architecture"]:
        nkv = c["num_kv_heads"]
        qkv = fused.view(T, nkv, nh // nkv + 2, d)
        return qkv[:, :, :-2].reshape(T, nh, d), qkv[:, :, -2], qkv[:, :, -1]
    if not c["multi_query"]:
        qkv = fused.view(T, nh, 3, d)
        return qkv[:, :, 0], qkv[:, :, 1], qkv[:, :, 2]
    qkv = fused.view(T, nh + 2, d)
    return qkv[:, :-2], qkv[:, [-2]], qkv[:, [-1]]


def attention_scores_softmax(q, k, v, bias=None):
    """Causal softmax(q k^T / sqrt(d) + bias) v for one sequence; q [T, nh, d], k, v [T, nkv, d]
    (src/transformers/models/falcon/modeling_falcon.py:371-386 / :407-422 with the mask of :1138-1153:
    key j is visible to query t iff j <= t)."""
    T, nh, d = q.shape
    nkv = k.shape[1]
    g = nh // nkv
    out = torch.empty_like(q)
    mask = torch.full((T, T), float("-inf"), dtype=q.dtype, device=q.device).triu(1)
    for h in range(nh):
        s = q[:, h] @ k[:, h // g].T / math.sqrt(d)
        if bias is not None:
            s = s + bias[h][None, :]
        p = torch.softmax(s + mask, dim=-1)
        out[:, h] = p @ v[:, h // g]
    return out.reshape(T, nh * d)


def self_attention(x, w, prefix, c, positions, seq_lens=None):
    """FalconAttention.forward (src/transformers/models/falcon/modeling_falcon.py:326-458).  ``seq_lens``: for
    every token the length its sequence had after the forward pass that brought the token (default: the whole
    sequence at once); only frequencies that follow the length (``dynamic``) look at it, and what they rotated
    stays as it was rotated then, like a key in the reference's cache."""
    nh = c["num_attention_heads"]
    d = c["hidden_size"] // nh
    fused = linear(x, w[prefix + "query_key_value.weight"], w.get(prefix + "query_key_value.bias"))
    q, k, v = split_heads(fused, c)
    bias = None
    if c["alibi"]:
        bias = alibi_bias(nh, x.shape[0], d, x.dtype, bool(c.get("alibi_bf16_compat", True))).to(x.device)
    elif seq_lens is None or (c.get("rope_scaling") or {}).get("rope_type", (c.get("rope_scaling") or {}).get("type")) != "dynamic":
        inv_freq, scale = rope_parameters(c, x.shape[0])
        cos, sin = rope_cos_sin(positions, inv_freq, x.dtype, scale)
        q, k = apply_rope(q, cos, sin), apply_rope(k, cos, sin)
    else:
        q, k = q.clone(), k.clone()
        for n in sorted(set(int(v) for v in seq_lens)):  # the tokens of one forward pass share its table
            rows = torch.tensor([t for t, v in enumerate(seq_lens) if int(v) == n], device=x.device)
            inv_freq, scale = rope_parameters(c, n)
            cos, sin = rope_cos_sin(positions[rows], inv_freq, x.dtype, scale)
            q[rows], k[rows] = apply_rope(q[rows], cos, sin), apply_rope(k[rows], cos, sin)
    o = attention_scores_softmax(q, k, v, bias)
    return linear(o, w[prefix + "dense.weight"], w.get(prefix + "dense.bias"))


def activation(x, name):
    """An activation by the reference's name (src/transformers/activations.py:25-195, table :200-220)."""
    F = torch.nn.functional
    if name in ("gelu", "gelu_python"):
        return gelu(x)
    if name in ("gelu_new", "gelu_accurate", "gelu_pytorch_tanh"):  # :56, :127, :46
        return 0.5 * x * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (x + 0.044715 * torch.pow(x, 3.0))))
    if name == "gelu_fast":  # :83
        return 0.5 * x * (1.0 + torch.tanh(x * 0.7978845608 * (1.0 + 0.044715 * x * x)))
    if name == "quick_gelu":  # :90
        return x * torch.sigmoid(1.702 * x)
    if name == "gelu_10":  # :113
        return torch.clip(gelu(x), -10, 10)
    if name == "laplace":  # :176-178
        return 0.5 * (1.0 + torch.erf((x - 0.707107) / (0.282095 * math.sqrt(2.0))))
    table = {"relu": F.relu, "relu6": F.relu6, "silu": F.silu, "swish": F.silu, "sigmoid": torch.sigmoid,
             "tanh": torch.tanh, "leaky_relu": F.leaky_relu, "mish": F.mish, "linear": lambda t: t,
             "relu2": lambda t: torch.square(F.relu(t))}  # :172
    return table[name](x)


def mlp(x, w, prefix, act="gelu"):
    """FalconMLP (src/transformers/models/falcon/modeling_falcon.py:575-578); ``act`` is the configuration's
    ``activation`` (:568, ``get_activation``)."""
    u = linear(x, w[prefix + "dense_h_to_4h.weight"], w.get(prefix + "dense_h_to_4h.bias"))
    return linear(activation(u, act), w[prefix + "dense_4h_to_h.weight"], w.get(prefix + "dense_4h_to_h.bias"))


def decoder_layer(x, w, i, c, positions, seq_lens=None):
    """FalconDecoderLayer.forward (src/transformers/models/falcon/modeling_falcon.py:614-683)."""
    p = f"transformer.h.{i}."
    eps = c["layer_norm_epsilon"]
    residual = x
    if c["new_decoder_architecture"] and c["num_ln_in_parallel_attn"] == 2:  # :630-632
        attn_in = layer_norm(x, w[p + "ln_attn.weight"], w[p + "ln_attn.bias"], eps)
        mlp_in = layer_norm(x, w[p + "ln_mlp.weight"], w[p + "ln_mlp.bias"], eps)
    else:  # :634
        attn_in = layer_norm(x, w[p + "input_layernorm.weight"], w[p + "input_layernorm.bias"], eps)
        mlp_in = None
    attn = self_attention(attn_in, w, p + "self_attention.", c, positions, seq_lens)
    if not c["new_decoder_architecture"]:
        if c["parallel_attn"]:  # :649-650
            mlp_in = attn_in
        else:  # :652-659
            residual = residual + attn
            mlp_in = layer_norm(residual, w[p + "post_attention_layernorm.weight"],
                                w[p + "post_attention_layernorm.bias"], eps)
    if c["new_decoder_architecture"] and c["parallel_attn"] and c["num_ln_in_parallel_attn"] == 1:  # :661-666
        mlp_in = attn_in
    out = mlp(mlp_in, w, p + "mlp.", c.get("activation", "gelu"))
    if c["new_decoder_architecture"] or c["parallel_attn"]:  # :673-674
        out = out + attn
    return residual + out  # :676


def forward(cfg: dict, w: Dict[str, torch.Tensor], token_ids: Sequence[int], seq_lens: Optional[Sequence[int]] = None,
            hidden: Optional[list] = None, last: int = 0):
    """Logits [T, V] of one whole sequence (FalconModel.forward :864-1011, head :1230).  ``seq_lens``: see
    ``self_attention``; it says in which pieces the sequence was fed, for configurations that ask.  ``hidden``: a
    list that receives the residual stream after every layer.  ``last``: the logits of the last ``last`` places only
    (the reference's ``num_logits_to_keep``, :1230; 0: all)."""
    c = cfg_defaults(cfg)
    table = w["transformer.word_embeddings.weight"]
    ids = torch.as_tensor(list(token_ids), dtype=torch.long, device=table.device)
    x = table[ids]  # :895-896
    positions = torch.arange(len(ids), device=table.device)
    for i in range(c["num_hidden_layers"]):
        x = decoder_layer(x, w, i, c, positions, seq_lens)
        if hidden is not None:
            hidden.append(x)
    x = layer_norm(x, w["transformer.ln_f.weight"], w["transformer.ln_f.bias"], c["layer_norm_epsilon"])  # :992
    head = w["lm_head.weight"] if "lm_head.weight" in w else w["transformer.word_embeddings.weight"]  # tied :1163
    return x[-last:] @ head.T  # x[-0:] is all of x


# --- generation ---------------------------------------------------------------
def repetition_penalty(scores, seen_ids, penalty):
    """src/transformers/generation/logits_process.py:337-343."""
    out = scores.clone()
    idx = torch.as_tensor(sorted(set(int(t) for t in seen_ids)), dtype=torch.long)
    s = scores[idx]
    out[idx] = torch.where(s < 0, s * penalty, s / penalty)
    return out


def suppress(scores, ids):
    """EOS scores to -inf while the minimum length is not reached (logits_process.py:144-151, :214-223)."""
    out = scores.clone()
    out[torch.as_tensor(list(ids), dtype=torch.long)] = float("-inf")
    return out


def temperature(scores, t):
    """logits_process.py:286-289."""
    return scores / t


def top_k(scores, k, min_tokens_to_keep=1):
    """logits_process.py:505-518."""
    k = min(max(k, min_tokens_to_keep), scores.shape[-1])
    kth = torch.topk(scores, k)[0][-1]
    return scores.masked_fill(scores < kth, float("-inf"))


def top_p(scores, p, min_tokens_to_keep=1):
    """logits_process.py:452-465."""
    sorted_logits, sorted_idx = torch.sort(scores, descending=False, stable=True)
    cum = sorted_logits.softmax(-1).cumsum(-1)
    remove = cum <= (1 - p)
    remove[-min_tokens_to_keep:] = False
    mask = torch.zeros_like(remove)
    mask[sorted_idx] = remove
    return scores.masked_fill(mask, float("-inf"))


def min_p(scores, mp, min_tokens_to_keep=1):
    """logits_process.py:578-595."""
    probs = torch.softmax(scores, -1)
    remove = probs < mp * probs.max()
    order = torch.argsort(scores, descending=True)
    r = remove[order]
    r[:min_tokens_to_keep] = False
    mask = torch.zeros_like(remove)
    mask[order] = r
    return scores.masked_fill(mask, float("-inf"))


def typical_p(scores, mass, min_tokens_to_keep=1):
    """logits_process.py:663-683: tokens in the order of |(-log p) - entropy|, the nearest first; as many stay as
    it takes for their mass to reach ``mass``, and every token as near as the last of them."""
    logp = torch.log_softmax(scores, -1)
    p = logp.exp()
    entropy = -torch.nansum(logp * p)  # -inf * 0 is skipped
    distance = ((-logp) - entropy).abs()
    nearest_first = torch.argsort(distance, stable=True)
    cum = scores[nearest_first].softmax(-1).cumsum(-1)
    last = min(int((cum < mass).sum()), scores.shape[-1] - 1)
    remove = distance > distance[nearest_first[last]]
    remove[nearest_first[:min_tokens_to_keep]] = False
    return scores.masked_fill(remove, float("-inf"))


def _below_but_not_best(scores, probs, bound, min_tokens_to_keep=1):
    best = torch.topk(scores, min(min_tokens_to_keep, scores.shape[-1]))[0][-1]
    return scores.masked_fill((probs < bound) & (scores < best), float("-inf"))


def epsilon_cutoff(scores, epsilon):
    """logits_process.py:742-752: probabilities below ``epsilon`` go, the most probable token stays."""
    return _below_but_not_best(scores, scores.softmax(-1), epsilon)


def eta_cutoff(scores, epsilon):
    """logits_process.py:825-837: the bound is min(epsilon, sqrt(epsilon) * exp(-entropy)); the entropy is that
    of the normalised scores, a token that is already gone adding nothing."""
    logp = torch.log_softmax(scores, -1)
    probs = scores.softmax(-1)
    entropy = -(logp.clamp(min=torch.finfo(scores.dtype).min) * probs).sum()
    eta = min(epsilon, math.sqrt(epsilon) * math.exp(-float(entropy)))
    return _below_but_not_best(scores, probs, eta)


def no_repeat_ngram(scores, history, n):
    """logits_process.py:840-903, :954-962: every n-gram of the ids so far, filed under its first n - 1 tokens;
    what is filed under the last n - 1 ids may not come next."""
    ids = list(history)
    if len(ids) + 1 < n:
        return scores
    filed = {}
    for j in range(len(ids) - n + 1):
        gram = tuple(ids[j:j + n])
        filed.setdefault(gram[:-1], []).append(gram[-1])
    return suppress(scores, filed.get(tuple(ids[len(ids) + 1 - n:]), []))


def no_bad_words(scores, history, bad_words, eos_ids=()):
    """logits_process.py:1110-1140, :1270-1286: -inf for the last token of an entry whose other tokens end the ids
    so far (one-token entries always; an entry longer than the ids so far never applies, :1122); an entry that is an
    EOS token alone does not count."""
    ids = list(history)
    gone = []
    for word in bad_words:
        if len(word) == 1 and word[0] in eos_ids:
            continue
        if len(word) == 1 or (len(word) <= len(ids) and ids[len(ids) - (len(word) - 1):] == list(word[:-1])):
            gone.append(word[-1])
    return suppress(scores, gone)


def sequence_bias(scores, history, entries):
    """logits_process.py:1112-1140: ``entries`` is {tuple of ids: bias}; an entry of one token adds its bias to that
    token always, a longer one to its last token while the ids so far end in the tokens before it (an entry longer
    than the ids so far never applies, :1122)."""
    ids = list(history)
    out = scores.clone()
    for seq, bias in entries.items():
        seq = tuple(seq)
        if len(seq) == 1:
            out[seq[0]] += bias
        elif len(seq) <= len(ids) and tuple(ids[len(ids) - (len(seq) - 1):]) == seq[:-1]:
            out[seq[-1]] += bias
    return out


def forced_eos(scores, cur_len, max_length, forced_ids):
    """logits_process.py:1590-1596: with one token left before ``max_length`` every score becomes -inf and the
    forced ids' become 0."""
    if cur_len != max_length - 1:
        return scores
    out = torch.full_like(scores, float("-inf"))
    out[torch.as_tensor(list(forced_ids), dtype=torch.long)] = 0
    return out


def exponential_decay(scores, cur_len, prompt_len, start_index, factor, eos_ids):
    """logits_process.py:1699-1727: past ``start_index + prompt_len`` ids, the EOS scores gain
    ``|score| * (factor ** (ids past that) - 1)``."""
    start = start_index + prompt_len
    if cur_len <= start:
        return scores
    out = scores.clone()
    idx = torch.as_tensor(list(eos_ids), dtype=torch.long)
    out[idx] = scores[idx] + torch.abs(scores[idx]) * (pow(factor, cur_len - start) - 1)
    return out


def process(scores, history, *, do_sample, temperature_=1.0, top_k_=0, top_p_=1.0, min_p_=None, typical_p_=None,
            epsilon_cutoff_=None, eta_cutoff_=None, repetition_penalty_=1.0, suppress_ids=(), no_repeat_ngram_size_=0,
            bad_words_ids_=None, eos_ids_=(), sequence_bias_=None, forced_eos_=None, exponential_decay_=None,
            custom_=()):
    """Processors in the order the reference builds them (src/transformers/generation/utils.py:898-1097):
    sequence bias, repetition penalty, no-repeat n-grams, bad words, minimum length, forced last token
    (``forced_eos_``: (max_length, ids)), the growing bonus on EOS (``exponential_decay_``: (prompt length, start index,
    factor)), the caller's own processors (``custom_``: functions of (history, scores), :1038-1039), then (sampling
    only) temperature, top-k, top-p, min-p, typical-p, epsilon and eta cut-offs."""
    s = scores
    if sequence_bias_:
        s = sequence_bias(s, history, sequence_bias_)
    if repetition_penalty_ is not None and repetition_penalty_ != 1.0:
        s = repetition_penalty(s, history, repetition_penalty_)
    if no_repeat_ngram_size_:
        s = no_repeat_ngram(s, history, no_repeat_ngram_size_)
    if bad_words_ids_:
        s = no_bad_words(s, history, bad_words_ids_, eos_ids_)
    if suppress_ids:
        s = suppress(s, suppress_ids)
    if forced_eos_ is not None:
        s = forced_eos(s, len(history), forced_eos_[0], forced_eos_[1])
    if exponential_decay_ is not None:
        s = exponential_decay(s, len(history), exponential_decay_[0], exponential_decay_[1], exponential_decay_[2], eos_ids_)
    for fn in custom_:
        s = fn(list(history), s)
    if do_sample:
        if temperature_ is not None and temperature_ != 1.0:
            s = temperature(s, temperature_)
        if top_k_:
            s = top_k(s, top_k_)
        if top_p_ is not None and top_p_ < 1.0:
            s = top_p(s, top_p_)
        if min_p_ is not None:
            s = min_p(s, min_p_)
        if typical_p_ is not None and typical_p_ < 1.0:
            s = typical_p(s, typical_p_)
        if epsilon_cutoff_ is not None and 0.0 < epsilon_cutoff_ < 1.0:
            s = epsilon_cutoff(s, epsilon_cutoff_)
        if eta_cutoff_ is not None and 0.0 < eta_cutoff_ < 1.0:
            s = eta_cutoff(s, eta_cutoff_)
    return s


def pick(scores, u: Optional[float]):
    """argmax, or the token whose interval of the cumulative distribution holds ``u``
    (the reference draws with torch.multinomial, src/transformers/generation/utils.py:3274-3279;
    a given uniform number makes the draw repeatable)."""
    if u is None:
        return int(torch.argmax(scores))
    cdf = torch.softmax(scores.double(), -1).cumsum(-1)
    return int(min(torch.searchsorted(cdf, torch.tensor(u, dtype=torch.float64), right=True), scores.shape[-1] - 1))


def generate(cfg, w, prompt: Sequence[int], max_new_tokens: int, *, eos_ids=(), min_new_tokens=0,
             uniforms: Optional[Sequence[float]] = None, forced_eos_ids=None, exponential_decay_length_penalty=None,
             stop_when=(), **proc) -> List[int]:
    """One sequence, recomputed whole at every step (no cache); returns the new tokens, EOS included
    (loop of src/transformers/generation/utils.py:3220-3296, stop test stopping_criteria.py:446-467)."""
    seq = list(prompt)
    new = []
    if forced_eos_ids is not None:  # max_length = prompt + new tokens (src/transformers/generation/utils.py:1461)
        proc["forced_eos_"] = (len(prompt) + max_new_tokens, list(forced_eos_ids))
    if exponential_decay_length_penalty is not None:
        proc["exponential_decay_"] = (len(prompt), *exponential_decay_length_penalty)
        proc.setdefault("eos_ids_", tuple(eos_ids))
    for step in range(max_new_tokens):
        logits = forward(cfg, w, seq)[-1].float()
        s = process(logits, seq, do_sample=uniforms is not None,
                    suppress_ids=tuple(eos_ids) if len(new) < min_new_tokens else (), **proc)
        tok = pick(s, None if uniforms is None else uniforms[step])
        seq.append(tok)
        new.append(tok)
        if tok in eos_ids or any(fn(list(seq)) for fn in stop_when):  # the caller's criteria see the new token too
            break
    return new
