// What becomes of the rows of a fused query_key_value projection in a decode step when the launch that makes them
// also takes them to their end: split into heads, bias, rotation, queries out, keys and values into the cache
// pages (what qkv_rope_cache does as a kernel of its own; the row orders and page layouts are described there).
#pragma once

#include "common.h"

struct QkvTail {
    bf16_t* q_out;  // [M, heads, d]
    const float* inv_freq;  // [d/2], or null: no rotation
    int inv_freq_ld;        // 0: one table for all tokens; else a table per sequence of the step, this many apart
    float cs_scale;
    const int* token_pos;
    const int* token_seq;
    const int* block_table;
    int bt_stride;
    bf16_t* k_pool;
    bf16_t* v_pool;
    int nh, nkv, d, layout, write_cache;
};

// the frequency table of token m
__device__ __forceinline__ const float* qkv_tail_freq(const QkvTail& t, int m) {
    return t.inv_freq + (t.inv_freq_ld ? (long)t.token_seq[m] * t.inv_freq_ld : 0L);
}

// segment `seg` of d features of the fused row: kind 0 query, 1 key, 2 value, and which head
__device__ __forceinline__ void qkv_tail_segment(const QkvTail& t, int seg, int& kind, int& head) {
    const int gq = t.nh / t.nkv;
    if (t.layout == PTA_QKV_GROUPED) {
        const int grp = seg / (gq + 2), w = seg % (gq + 2);
        kind = w < gq ? 0 : w - gq + 1;
        head = w < gq ? grp * gq + w : grp;
    } else if (t.layout == PTA_QKV_TAIL) {
        kind = seg < t.nh ? 0 : seg - t.nh + 1;
        head = seg < t.nh ? seg : 0;
    } else {
        kind = seg % 3;
        head = seg / 3;
    }
}

// One pair of a token's segment: a is feature i of its lower half, b feature i + d/2, both as the product's own
// epilogue would have stored them (rounded to bfloat16, bias not yet added).
__device__ __forceinline__ void qkv_tail_pair(const QkvTail& t, const float* __restrict__ bias, int m, int seg, int i,
                                              float a, float b) {
    int kind, head;
    qkv_tail_segment(t, seg, kind, head);
    if (kind != 0 && !t.write_cache) return;
    const int d = t.d, half = d >> 1, pos = t.token_pos[m];
    if (bias) {
        a = round_to_bf16(a + bias[seg * d + i]);
        b = round_to_bf16(b + bias[seg * d + half + i]);
    }
    if (t.inv_freq && kind != 2) {
        const float ang = (float)pos * qkv_tail_freq(t, m)[i];
        const float c = cosf(ang) * t.cs_scale, sn = sinf(ang) * t.cs_scale;
        const float x0 = a, x1 = b;
        a = x0 * c - x1 * sn;
        b = x1 * c + x0 * sn;
    }
    if (kind == 0) {
        bf16_t* dst = t.q_out + ((long)m * t.nh + head) * d + i;
        dst[0] = f32_to_bf16_bits(a);
        dst[half] = f32_to_bf16_bits(b);
        return;
    }
    const long page = t.block_table[(long)t.token_seq[m] * t.bt_stride + pos / PTA_PAGE];
    const int in_page = pos % PTA_PAGE;
    if (kind == 1) {
        bf16_t* dst = t.k_pool + ((page * t.nkv + head) * PTA_PAGE + in_page) * (long)d + i;
        dst[0] = f32_to_bf16_bits(a);
        dst[half] = f32_to_bf16_bits(b);
    } else {
        bf16_t* dst = t.v_pool + ((page * t.nkv + head) * (long)d + i) * PTA_PAGE + in_page;
        dst[0] = f32_to_bf16_bits(a);
        dst[(long)half * PTA_PAGE] = f32_to_bf16_bits(b);
    }
}
