// What becomes of the rows of a fused query_key_value projection in a decode step when the launch that makes them
// also takes them to their end: split into heads, bias, rotation, queries out, keys and values into the cache
// pages (what qkv_rope_cache does as a kernel of its own; the row orders and page layouts are described there).
#pragma once

#include "common.h"
#include "pta_kernels.h"

struct QkvTail {
    bf16_t* q_out;  // [M, heads, d]
    PtaRotation rot;  // rot.inv_freq null: no rotation
    const int* token_pos;
    const int* token_seq;
    const int* block_table;
    int bt_stride;
    bf16_t* k_pool;
    bf16_t* v_pool;
    int nh, nkv, d, layout, write_cache;
};

// a rotation as the launches take it: null stands for none
__host__ __device__ __forceinline__ PtaRotation pta_rotation_of(const PtaRotation* r) {
    return r && r->inv_freq ? *r : PtaRotation{nullptr, 0, 1.0f, 0, PTA_PAIR_HALF};
}

// What every launch that rotates asks of a rotation (0: fine).  The frequency tables' rows hold rotary_dim / 2 values.
static inline int pta_check_rotation(const char* what, const PtaRotation& r, int d, const int* token_seq) {
    if (!r.inv_freq) return 0;
    PTA_REQUIRE(r.rotary_dim >= 2 && r.rotary_dim % 2 == 0 && r.rotary_dim <= d && d <= 256,
                "%s: rotation of the first %d elements of heads of %d: an even number from 2 up to the head size, heads up to 256",
                what, r.rotary_dim, d);
    PTA_REQUIRE(r.pairing == PTA_PAIR_HALF || r.pairing == PTA_PAIR_INTERLEAVED,
                "%s: pairing %d is not built; built are half-split pairs (i, i + rotary_dim / 2) and interleaved pairs (2i, 2i + 1)",
                what, r.pairing);
    PTA_REQUIRE(r.inv_freq_ld == 0 || (token_seq && r.inv_freq_ld >= r.rotary_dim / 2),
                "%s: a frequency table per sequence needs the tokens' sequences and rows of %d", what, r.rotary_dim / 2);
    return 0;
}

// the frequency table of token m
__device__ __forceinline__ const float* qkv_tail_freq(const QkvTail& t, int m) {
    return t.rot.inv_freq + (t.rot.inv_freq_ld ? (long)t.token_seq[m] * t.rot.inv_freq_ld : 0L);
}

// whether the rotation takes whole heads in half-split pairs (or there is none): pair p is then elements p and
// p + d/2, and runs of consecutive pairs are runs of consecutive elements
__host__ __device__ __forceinline__ bool qkv_tail_plain_pairs(const PtaRotation& r, int d) {
    return !r.inv_freq || (r.rotary_dim == d && r.pairing == PTA_PAIR_HALF);
}

// The d elements of a segment are taken as d/2 pairs.  Pair p below rotary_dim / 2 is rotated: elements
// (p, p + rotary_dim / 2) or (2p, 2p + 1) by the pairing, by the angle of frequency p; the pairs from there on are
// the elements past rotary_dim two by two, which pass.  Without a rotation the pairs are (p, p + d/2) and pass.
__host__ __device__ __forceinline__ void qkv_tail_pair_elements(const PtaRotation& r, int d, int p, int& ea, int& eb,
                                                                bool& rotated) {
    if (!r.inv_freq) { ea = p; eb = p + (d >> 1); rotated = false; return; }
    const int hr = r.rotary_dim >> 1;
    rotated = p < hr;
    if (!rotated) { ea = r.rotary_dim + 2 * (p - hr); eb = ea + 1; }
    else if (r.pairing == PTA_PAIR_INTERLEAVED) { ea = 2 * p; eb = ea + 1; }
    else { ea = p; eb = p + hr; }
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

// where element e of a token's query, key or value goes
__device__ __forceinline__ bf16_t* qkv_tail_place(const QkvTail& t, int m, int kind, int head, int pos, int e) {
    if (kind == 0) return t.q_out + ((long)m * t.nh + head) * t.d + e;
    const long page = t.block_table[(long)t.token_seq[m] * t.bt_stride + pos / PTA_PAGE];
    const int in_page = pos % PTA_PAGE;
    if (kind == 1) return t.k_pool + ((page * t.nkv + head) * PTA_PAGE + in_page) * (long)t.d + e;
    return t.v_pool + ((page * t.nkv + head) * (long)t.d + e) * PTA_PAGE + in_page;
}

// One pair of a token's segment (``qkv_tail_pair_elements``): a and b are its two elements as the product's own
// epilogue would have stored them (rounded to bfloat16, bias not yet added).
__device__ __forceinline__ void qkv_tail_pair(const QkvTail& t, const float* __restrict__ bias, int m, int seg, int p,
                                              float a, float b) {
    int kind, head, ea, eb;
    bool rotated;
    qkv_tail_segment(t, seg, kind, head);
    if (kind != 0 && !t.write_cache) return;
    qkv_tail_pair_elements(t.rot, t.d, p, ea, eb, rotated);
    const int pos = t.token_pos[m];
    if (bias) {
        a = round_to_bf16(a + bias[seg * t.d + ea]);
        b = round_to_bf16(b + bias[seg * t.d + eb]);
    }
    if (rotated && kind != 2) {
        const float ang = (float)pos * qkv_tail_freq(t, m)[p];
        const float c = cosf(ang) * t.rot.cs_scale, sn = sinf(ang) * t.rot.cs_scale;
        const float x0 = a, x1 = b;
        a = x0 * c - x1 * sn;
        b = x1 * c + x0 * sn;
    }
    *qkv_tail_place(t, m, kind, head, pos, ea) = f32_to_bf16_bits(a);
    *qkv_tail_place(t, m, kind, head, pos, eb) = f32_to_bf16_bits(b);
}
