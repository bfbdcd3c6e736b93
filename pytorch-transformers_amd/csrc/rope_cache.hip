// Split the fused query_key_value rows into heads, add the bias, rotate queries
// and keys, write queries to [M, heads, d] and append keys and values to the
// sequence's cache pages -- one pass over the fused activations.
//
// Row orders of the fused projection (src/transformers/models/falcon/modeling_falcon.py:269-298):
//   grouped      per KV group j: q_{j,0} .. q_{j,g-1}, k_j, v_j     (g = heads / kv_heads)
//   tail         q_0 .. q_{heads-1}, k, v
//   interleaved  per head h: q_h, k_h, v_h
// Rotation pairs element i with i + d/2 (rotate_half, :76-80; apply :104-108); the angle is
// position * inv_freq[i], taken in 32-bit (:155-164).  Keys are stored rotated (:350-358).
// Key pages are [kv_head][64 positions][d]; value pages are transposed, [kv_head][d][64 positions].
#include "common.h"
#include "pta_kernels.h"

template <typename T>
__global__ void qkv_rope_cache_kernel(T* __restrict__ q_out, const T* __restrict__ fused,
                                      const float* __restrict__ bias, const float* __restrict__ inv_freq,
                                      float cs_scale, const int* __restrict__ token_pos,
                                      const int* __restrict__ token_seq, const int* __restrict__ block_table,
                                      int bt_stride, T* __restrict__ k_pool, T* __restrict__ v_pool, int nh, int nkv,
                                      int d, int layout, int write_cache) {
    const int m = blockIdx.x;
    const int slot = blockIdx.y;  // 0..nh-1 queries, then nkv keys, then nkv values
    const int g = nh / nkv;
    int kind, head;  // kind 0 q, 1 k, 2 v
    if (slot < nh) { kind = 0; head = slot; }
    else if (slot < nh + nkv) { kind = 1; head = slot - nh; }
    else { kind = 2; head = slot - nh - nkv; }
    if (kind != 0 && !write_cache) return;

    int src_head;  // index of the d-wide row block inside the fused row
    if (layout == PTA_QKV_GROUPED) {
        src_head = kind == 0 ? (head / g) * (g + 2) + (head % g) : head * (g + 2) + g + (kind - 1);
    } else if (layout == PTA_QKV_TAIL) {
        src_head = kind == 0 ? head : nh + (kind - 1);
    } else {
        src_head = head * 3 + kind;
    }
    const long qout = (long)(nh + 2 * nkv) * d;
    const T* src = fused + (long)m * qout + (long)src_head * d;
    const float* bsrc = bias ? bias + (long)src_head * d : nullptr;

    const int pos = token_pos[m];
    T* dst;
    long dst_stride = 1;  // values are stored transposed, [d][64], so that eight keys of one feature are contiguous
    if (kind == 0) {
        dst = q_out + ((long)m * nh + head) * d;
    } else {
        const int seq = token_seq[m];
        const long page = block_table[(long)seq * bt_stride + pos / PTA_PAGE];
        if (kind == 1) {
            dst = k_pool + ((page * nkv + head) * PTA_PAGE + (pos % PTA_PAGE)) * (long)d;
        } else {
            dst = v_pool + (page * nkv + head) * (long)PTA_PAGE * d + (pos % PTA_PAGE);
            dst_stride = PTA_PAGE;
        }
    }

    if (kind != 2 && inv_freq) {
        const int half = d >> 1;
        for (int i = threadIdx.x; i < half; i += blockDim.x) {
            float a = Io<T>::ld(src + i), b = Io<T>::ld(src + i + half);
            if (bsrc) { a = Io<T>::round(a + bsrc[i]); b = Io<T>::round(b + bsrc[i + half]); }
            const float ang = (float)pos * inv_freq[i];
            const float c = cosf(ang) * cs_scale, s = sinf(ang) * cs_scale;
            Io<T>::st(dst + i, a * c - b * s);
            Io<T>::st(dst + i + half, b * c + a * s);
        }
    } else {
        for (int i = threadIdx.x; i < d; i += blockDim.x) {
            float a = Io<T>::ld(src + i);
            if (bsrc) a = Io<T>::round(a + bsrc[i]);
            Io<T>::st(dst + i * dst_stride, a);
        }
    }
}

extern "C" int pta_qkv_rope_cache(void* q_out, const void* fused, const float* bias, const float* inv_freq,
                                  float cs_scale, const int* token_pos, const int* token_seq,
                                  const int* block_table, int bt_stride, void* k_pool, void* v_pool, int M, int nh,
                                  int nkv, int d, int layout, int write_cache, int dtype, void* stream) {
    PTA_REQUIRE(M > 0 && nh > 0 && nkv > 0 && d > 0, "qkv_rope_cache: sizes must be positive (M=%d nh=%d nkv=%d d=%d)", M, nh, nkv, d);
    PTA_REQUIRE(nh % nkv == 0, "qkv_rope_cache: heads (%d) must be a multiple of kv heads (%d)", nh, nkv);
    PTA_REQUIRE(layout >= 0 && layout <= 2, "qkv_rope_cache: unknown layout %d", layout);
    PTA_REQUIRE(layout != PTA_QKV_TAIL || nkv == 1, "qkv_rope_cache: the tail layout has one kv head, got %d", nkv);
    PTA_REQUIRE(layout != PTA_QKV_INTERLEAVED || nkv == nh, "qkv_rope_cache: the interleaved layout needs kv heads == heads");
    PTA_REQUIRE(!inv_freq || d % 2 == 0, "qkv_rope_cache: rotation needs an even head size, got %d", d);
    PTA_REQUIRE(!write_cache || (k_pool && v_pool && block_table && token_seq), "qkv_rope_cache: null cache pointer");
    PTA_REQUIRE(nh + 2 * nkv <= 65535, "qkv_rope_cache: too many heads for one launch");
    hipStream_t s = (hipStream_t)stream;
    dim3 grid(M, nh + 2 * nkv);
    if (dtype == PTA_F32)
        hipLaunchKernelGGL(qkv_rope_cache_kernel<float>, grid, dim3(64), 0, s, (float*)q_out, (const float*)fused,
                           bias, inv_freq, cs_scale, token_pos, token_seq, block_table, bt_stride, (float*)k_pool,
                           (float*)v_pool, nh, nkv, d, layout, write_cache);
    else if (dtype == PTA_BF16)
        hipLaunchKernelGGL(qkv_rope_cache_kernel<bf16_t>, grid, dim3(64), 0, s, (bf16_t*)q_out,
                           (const bf16_t*)fused, bias, inv_freq, cs_scale, token_pos, token_seq, block_table,
                           bt_stride, (bf16_t*)k_pool, (bf16_t*)v_pool, nh, nkv, d, layout, write_cache);
    else
        return pta_fail("qkv_rope_cache: unknown dtype %d", dtype);
    return pta_check_launch("qkv_rope_cache");
}
