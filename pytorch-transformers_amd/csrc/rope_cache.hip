// Split the fused query_key_value rows into heads, add the bias, rotate queries
// and keys, write queries to [M, heads, d] and append keys and values to the
// sequence's cache pages -- one pass over the fused activations.
//
// Row orders of the fused projection (src/transformers/models/falcon/modeling_falcon.py:269-298):
//   grouped      per KV group j: q_{j,0} .. q_{j,g-1}, k_j, v_j     (g = heads / kv_heads)
//   tail         q_0 .. q_{heads-1}, k, v
//   interleaved  per head h: q_h, k_h, v_h
// Rotation is data (PtaRotation, pta_kernels.h): the first rotary_dim elements of a head, in pairs (i, i + rotary_dim/2)
// (rotate_half, :76-80; apply :104-108: what the reference's Falcon does, over the whole head) or (2i, 2i + 1); the
// angle is position * inv_freq[i], taken in 32-bit (:155-164).  Keys are stored rotated (:350-358).
// Key pages are [kv_head][64 positions][d]; value pages are transposed, [kv_head][d][64 positions].
//
// One workgroup per token: the cosines and sines of the token's position are computed once into
// LDS and used by every head; then the threads walk (head, element) items of the whole fused row.
#include "common.h"
#include "pta_kernels.h"
#include "qkv_tail.h"

#define RC_THREADS 256

template <typename T>
__global__ __launch_bounds__(RC_THREADS) void qkv_rope_cache_kernel(
    T* __restrict__ q_out, const T* __restrict__ fused, long fused_ld, const float* __restrict__ bias,
    PtaRotation rot, const int* __restrict__ token_pos,
    const int* __restrict__ token_seq, const int* __restrict__ block_table, int bt_stride, T* __restrict__ k_pool,
    T* __restrict__ v_pool, int nh, int nkv, int d, int layout, int write_cache) {
    __shared__ float cos_s[128], sin_s[128];
    const int m = blockIdx.x, tid = threadIdx.x;
    const int g = nh / nkv;
    const int R = rot.inv_freq ? rot.rotary_dim : 0, half = R >> 1;  // rotated elements of a head, and their pairs
    const int pos = token_pos[m];
    const T* row = fused + (long)m * fused_ld;  // rows of the fused projection may lie apart
    const int n_slots = write_cache ? nh + 2 * nkv : nh;  // queries, then keys, then values
    // rotated items: (slot < nh + nkv, pair i < half); plain items: every other element of every slot
    const int rot_slots = R ? min(n_slots, nh + nkv) : 0;
    // gridDim.y workgroups share a token's items (a decode step has few tokens and many heads)
    const int stride = RC_THREADS * gridDim.y, first = tid + blockIdx.y * RC_THREADS;
    // bfloat16, half-split pairs whose halves are multiples of eight: eight pairs per item, sixteen bytes per access
    const bool wide = sizeof(T) == 2 && rot.pairing == PTA_PAIR_HALF && half > 0 && (half & 7) == 0 && (d & 7) == 0;
    const int h8 = half >> 3;
    auto source_head = [&](int kind, int head) {
        if (layout == PTA_QKV_GROUPED) return kind == 0 ? (head / g) * (g + 2) + (head % g) : head * (g + 2) + g + (kind ? kind - 1 : 0);
        if (layout == PTA_QKV_TAIL) return kind == 0 ? head : nh + kind - 1;
        return head * 3 + kind;
    };
    // A thread's first two items are asked for before anything else, so that the table of angles is made and the
    // page looked up while they are on their way: a token's row is read in one round trip to memory, not three.
    constexpr int AHEAD = 2;
    uint4 ra[AHEAD], rb[AHEAD];
    if (wide) {
#pragma unroll
        for (int u = 0; u < AHEAD; ++u) {
            const int item = first + u * stride;
            if (item < rot_slots * h8) {
                const int slot = item / h8, i = (item - slot * h8) * 8;
                const bf16_t* src = (const bf16_t*)row + (long)source_head(slot < nh ? 0 : 1, slot < nh ? slot : slot - nh) * d;
                ra[u] = *reinterpret_cast<const uint4*>(src + i);
                rb[u] = *reinterpret_cast<const uint4*>(src + i + half);
            }
        }
    }
    if (R) {
        // one table for all tokens, or one per sequence of the step (frequencies that follow a sequence's length)
        const float* freq = rot.inv_freq + (rot.inv_freq_ld ? (long)token_seq[m] * rot.inv_freq_ld : 0L);
        for (int i = tid; i < half; i += RC_THREADS) {
            const float ang = (float)pos * freq[i];
            cos_s[i] = cosf(ang) * rot.cs_scale;
            sin_s[i] = sinf(ang) * rot.cs_scale;
        }
        __syncthreads();
    }
    long page = 0;
    if (write_cache) page = block_table[(long)token_seq[m] * bt_stride + pos / PTA_PAGE];
    const int in_page = pos % PTA_PAGE;

    if (wide) {
        auto rotate_item = [&](int item, const uint4& va, const uint4& vb) {
            const int slot = item / h8, i = (item - slot * h8) * 8;
            const int kind = slot < nh ? 0 : 1, head = slot < nh ? slot : slot - nh;
            const int src_head = source_head(kind, head);
            float a[8], b[8], lo[8], hi[8];
            unpack8(va, a);
            unpack8(vb, b);
            if (bias) {
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    a[e] = round_to_bf16(a[e] + bias[(long)src_head * d + i + e]);
                    b[e] = round_to_bf16(b[e] + bias[(long)src_head * d + i + half + e]);
                }
            }
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float c = cos_s[i + e], s = sin_s[i + e];
                lo[e] = a[e] * c - b[e] * s;
                hi[e] = b[e] * c + a[e] * s;
            }
            bf16_t* dst = kind == 0 ? (bf16_t*)q_out + ((long)m * nh + head) * d
                                    : (bf16_t*)k_pool + ((page * nkv + head) * PTA_PAGE + in_page) * (long)d;
            *reinterpret_cast<uint4*>(dst + i) = pack8(lo);
            *reinterpret_cast<uint4*>(dst + i + half) = pack8(hi);
        };
#pragma unroll
        for (int u = 0; u < AHEAD; ++u)
            if (first + u * stride < rot_slots * h8) rotate_item(first + u * stride, ra[u], rb[u]);
        for (int item = first + AHEAD * stride; item < rot_slots * h8; item += stride) {
            const int slot = item / h8, i = (item - slot * h8) * 8;
            const bf16_t* src = (const bf16_t*)row + (long)source_head(slot < nh ? 0 : 1, slot < nh ? slot : slot - nh) * d;
            rotate_item(item, *reinterpret_cast<const uint4*>(src + i), *reinterpret_cast<const uint4*>(src + i + half));
        }
    } else {
        for (int item = first; item < rot_slots * half; item += stride) {
            const int slot = item / half, i = item - slot * half;
            const int kind = slot < nh ? 0 : 1, head = slot < nh ? slot : slot - nh;
            const int src_head = source_head(kind, head);
            const int ea = rot.pairing == PTA_PAIR_INTERLEAVED ? 2 * i : i, eb = rot.pairing == PTA_PAIR_INTERLEAVED ? ea + 1 : i + half;
            const T* src = row + (long)src_head * d;
            float a = Io<T>::ld(src + ea), b = Io<T>::ld(src + eb);
            if (bias) {
                a = Io<T>::round(a + bias[(long)src_head * d + ea]);
                b = Io<T>::round(b + bias[(long)src_head * d + eb]);
            }
            const float c = cos_s[i], s = sin_s[i];
            T* dst = kind == 0 ? q_out + ((long)m * nh + head) * d
                               : k_pool + ((page * nkv + head) * PTA_PAGE + in_page) * (long)d;
            Io<T>::st(dst + ea, a * c - b * s);
            Io<T>::st(dst + eb, b * c + a * s);
        }
    }
    // what is not rotated: the elements past rotary_dim of the rotated slots, then every element of the other slots
    const int rest = d - R, n_rest = rot_slots * rest;
    for (int item = first; item < n_rest + (n_slots - rot_slots) * d; item += stride) {
        int slot, i;
        if (item < n_rest) { slot = item / rest; i = R + (item - slot * rest); }
        else { slot = rot_slots + (item - n_rest) / d; i = (item - n_rest) % d; }
        int kind, head;
        if (slot < nh) { kind = 0; head = slot; }
        else if (slot < nh + nkv) { kind = 1; head = slot - nh; }
        else { kind = 2; head = slot - nh - nkv; }
        const int src_head = source_head(kind, head);
        float a = Io<T>::ld(row + (long)src_head * d + i);
        if (bias) a = Io<T>::round(a + bias[(long)src_head * d + i]);
        if (kind == 0) Io<T>::st(q_out + ((long)m * nh + head) * d + i, a);
        else if (kind == 1) Io<T>::st(k_pool + ((page * nkv + head) * PTA_PAGE + in_page) * (long)d + i, a);
        else Io<T>::st(v_pool + ((page * nkv + head) * (long)d + i) * PTA_PAGE + in_page, a);
    }
}

extern "C" int pta_qkv_rope_cache(void* q_out, const void* fused, int fused_ld, const float* bias, const PtaRotation* rotation,
                                  const int* token_pos, const int* token_seq,
                                  const int* block_table, int bt_stride, void* k_pool, void* v_pool, int M, int nh,
                                  int nkv, int d, int layout, int write_cache, int dtype, void* stream) {
    PTA_REQUIRE(M > 0 && nh > 0 && nkv > 0 && d > 0, "qkv_rope_cache: sizes must be positive (M=%d nh=%d nkv=%d d=%d)", M, nh, nkv, d);
    PTA_REQUIRE(nh % nkv == 0, "qkv_rope_cache: heads (%d) must be a multiple of kv heads (%d)", nh, nkv);
    PTA_REQUIRE(layout >= 0 && layout <= 2, "qkv_rope_cache: unknown layout %d", layout);
    PTA_REQUIRE(layout != PTA_QKV_TAIL || nkv == 1, "qkv_rope_cache: the tail layout has one kv head, got %d", nkv);
    PTA_REQUIRE(layout != PTA_QKV_INTERLEAVED || nkv == nh, "qkv_rope_cache: the interleaved layout needs kv heads == heads");
    const PtaRotation rot = pta_rotation_of(rotation);
    if (pta_check_rotation("qkv_rope_cache", rot, d, token_seq)) return 1;
    PTA_REQUIRE(!write_cache || (k_pool && v_pool && block_table && token_seq), "qkv_rope_cache: null cache pointer");
    PTA_REQUIRE(fused_ld >= (long)(nh + 2 * nkv) * d, "qkv_rope_cache: fused rows of %ld elements cannot lie %d apart",
                (long)(nh + 2 * nkv) * d, fused_ld);
    const bool wide = dtype == PTA_BF16 && rot.inv_freq && rot.pairing == PTA_PAIR_HALF && (rot.rotary_dim / 2) % 8 == 0 && d % 8 == 0;
    PTA_REQUIRE(!wide || ((((uintptr_t)fused | (uintptr_t)q_out | (uintptr_t)k_pool) % 16) == 0 && fused_ld % 8 == 0),
                "qkv_rope_cache: bfloat16 rows are moved sixteen bytes at a time and must be aligned so");
    hipStream_t s = (hipStream_t)stream;
    int slices = 1;  // enough workgroups to occupy the chip when the step has few tokens
    while (slices < 16 && M * slices < 512 && slices * RC_THREADS < (nh + 2 * nkv) * d) slices *= 2;
    if (dtype == PTA_F32)
        hipLaunchKernelGGL(qkv_rope_cache_kernel<float>, dim3(M, slices), dim3(RC_THREADS), 0, s, (float*)q_out,
                           (const float*)fused, fused_ld, bias, rot, token_pos, token_seq, block_table, bt_stride,
                           (float*)k_pool, (float*)v_pool, nh, nkv, d, layout, write_cache);
    else if (dtype == PTA_BF16)
        hipLaunchKernelGGL(qkv_rope_cache_kernel<bf16_t>, dim3(M, slices), dim3(RC_THREADS), 0, s, (bf16_t*)q_out,
                           (const bf16_t*)fused, fused_ld, bias, rot, token_pos, token_seq, block_table,
                           bt_stride, (bf16_t*)k_pool, (bf16_t*)v_pool, nh, nkv, d, layout, write_cache);
    else
        return pta_fail("qkv_rope_cache: unknown dtype %d", dtype);
    return pta_check_launch("qkv_rope_cache");
}

// Frequencies that follow each sequence's length (dynamic NTK scaling, src/transformers/modeling_rope_utils.py:112-160):
// out[s, i] = 1 / base_s^(2i/d), base_s = theta * (factor * len_s / max_pos - (factor - 1))^(d / (d - 2)) once the
// sequence's length after this step, len_s = seq_start[s] + its tokens of the step, exceeds max_pos, else theta.
// Evaluated in double precision and rounded once.
__global__ void rope_dynamic_table_kernel(float* __restrict__ out, const int* __restrict__ seq_start,
                                          const int* __restrict__ cu_tokens, int n_seqs, int half, double theta,
                                          double factor, int max_pos) {
    const int s = blockIdx.x;
    const int len = seq_start[s] + cu_tokens[s + 1] - cu_tokens[s];
    const int d = 2 * half;
    double base = theta;
    if (len > max_pos) base = theta * pow(factor * (double)len / (double)max_pos - (factor - 1.0), (double)d / (double)(d - 2));
    for (int i = threadIdx.x; i < half; i += blockDim.x) out[(long)s * half + i] = (float)(1.0 / pow(base, (double)(2 * i) / (double)d));
}

extern "C" int pta_rope_dynamic_table(float* out, const int* seq_start, const int* cu_tokens, int n_seqs, int d,
                                      float theta, float factor, int max_pos, void* stream) {
    PTA_REQUIRE(out && seq_start && cu_tokens, "rope_dynamic_table: null pointer");
    PTA_REQUIRE(n_seqs > 0 && d > 2 && d % 2 == 0, "rope_dynamic_table: %d sequences, head size %d (even, more than 2)", n_seqs, d);
    PTA_REQUIRE(theta > 0.f && factor >= 1.f && max_pos > 0, "rope_dynamic_table: theta %g, factor %g, positions %d", theta,
                factor, max_pos);
    hipLaunchKernelGGL(rope_dynamic_table_kernel, dim3(n_seqs), dim3(64), 0, (hipStream_t)stream, out, seq_start, cu_tokens,
                       n_seqs, d / 2, (double)theta, (double)factor, max_pos);
    return pta_check_launch("rope_dynamic_table");
}
