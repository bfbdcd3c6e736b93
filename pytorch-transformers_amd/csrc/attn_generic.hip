// Causal attention over the paged cache, any number of new tokens per sequence,
// all arithmetic in 32-bit.  One wave per (token, head): keys are taken a page
// (64) at a time from position 0 in a running softmax, so what a token computes
// does not depend on how the sequence was cut into steps or on the rest of the
// batch.  This is the engine's 32-bit path and the fallback for sizes the MFMA
// kernels refuse.
//
// score[j] = q . k_j / sqrt(d) + bias_j, keys 0 .. pos (or the last `window` of them)
// (src/transformers/models/falcon/modeling_falcon.py:371-386, :407-422).
// The bias is data (PtaScoreBias, pta_kernels.h).  The reference's ALiBi is bf16(bf16(slope_h) * bf16(j)) / sqrt(d):
// it forms slope x position in bfloat16 even in a 32-bit model (:196-198) and divides by sqrt(d) when it folds the
// bias into the mask (:1078-1085); `slopes` then holds the slopes already rounded to bfloat16, and the scale 1 / sqrt(d).
#include "common.h"
#include "pta_kernels.h"
#include "score_bias.h"

template <typename T>
__global__ void attn_generic_kernel(T* __restrict__ out, const T* __restrict__ q, const T* __restrict__ k_pool,
                                    const T* __restrict__ v_pool, const int* __restrict__ block_table,
                                    int bt_stride, const int* __restrict__ token_seq,
                                    const int* __restrict__ token_pos, const float* __restrict__ slopes, int bias_mode, float bias_scale,
                                    int nh, int nkv, int d, float scale, int window) {
    __shared__ float q_s[256];
    __shared__ float p_s[PTA_PAGE];
    const int m = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const int kvh = h / (nh / nkv);
    const int seq = token_seq[m];
    const int nkeys = token_pos[m] + 1;
    const int* bt = block_table + (long)seq * bt_stride;
    const T* qr = q + ((long)m * nh + h) * d;
    for (int i = lane; i < d; i += PTA_WAVE) q_s[i] = Io<T>::ld(qr + i);
    __syncthreads();
    const float slope = slopes ? slopes[h] : 0.f;

    // with a window the token sees keys first .. pos only; pages wholly before `first` may be gone
    const int first = window > 0 ? max(0, nkeys - window) : 0;
    float m_run = -INFINITY, l_run = 0.f;
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    for (int c0 = first / PTA_PAGE * PTA_PAGE; c0 < nkeys; c0 += PTA_PAGE) {
        const long page = bt[c0 / PTA_PAGE];
        const T* kp = k_pool + (page * nkv + kvh) * (long)PTA_PAGE * d;
        const T* vp = v_pool + (page * nkv + kvh) * (long)PTA_PAGE * d;
        const int j = c0 + lane;
        const bool valid = j >= first && j < nkeys;
        float s = -INFINITY;
        if (valid) {
            const T* kr = kp + (long)lane * d;
            float dot = 0.f;
            for (int i = 0; i < d; ++i) dot += q_s[i] * Io<T>::ld(kr + i);
            s = dot * scale;
            if (slopes)  // slope x key position as the reference rounds it (0), exact (1), or x the distance from the query (2)
                s += (bias_mode == 0 ? round_to_bf16(slope * round_to_bf16((float)j))
                                     : slope * (float)(bias_mode == 2 ? j - (nkeys - 1) : j)) * bias_scale;
        }
        const float m_new = fmaxf(m_run, wave_max(s));
        const float p = valid ? expf(s - m_new) : 0.f;
        const float corr = expf(m_run - m_new);  // 0 on the first page
        l_run = l_run * corr + wave_sum(p);
        __syncthreads();
        p_s[lane] = p;
        __syncthreads();
        const int cnt = min(PTA_PAGE, nkeys - c0);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int dim = lane + r * PTA_WAVE;
            if (dim < d) {
                float a = acc[r] * corr;
                for (int jj = max(0, first - c0); jj < cnt; ++jj) a += p_s[jj] * Io<T>::ld(vp + (long)dim * PTA_PAGE + jj);
                acc[r] = a;
            }
        }
        m_run = m_new;
    }
    T* orow = out + ((long)m * nh + h) * d;
    const float inv = 1.0f / l_run;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int dim = lane + r * PTA_WAVE;
        if (dim < d) Io<T>::st(orow + dim, acc[r] * inv);
    }
}

// Whether the attention kernels and the kernel that rotates queries and keys take these sizes (0), or why not
// (pta_last_error): for a caller that wants to refuse a model before it reads a weight.  ``rotated``: queries and
// keys are rotated by position (pairs of elements: an even head size).
extern "C" int pta_attention_sizes_ok(int nh, int nkv, int d, int rotated) {
    PTA_REQUIRE(nh > 0 && nkv > 0 && nh % nkv == 0, "attention: %d heads are no multiple of %d kv heads", nh, nkv);
    PTA_REQUIRE(d > 0 && d <= 256, "attention: head size %d is outside 1..256, which is what the kernels take", d);
    PTA_REQUIRE(nh <= 65535, "attention: at most 65535 heads, got %d", nh);
    PTA_REQUIRE(!rotated || d % 2 == 0, "attention: rotation pairs elements and needs an even head size, got %d", d);
    return 0;
}

extern "C" int pta_attn_generic(void* out, const void* q, const void* k_pool, const void* v_pool,
                                const int* block_table, int bt_stride, const int* token_seq, const int* token_pos,
                                const PtaScoreBias* score_bias, int M, int nh, int nkv, int d, float scale, int window, int dtype,
                                void* stream) {
    int bias_mode = 0;
    if (pta_score_bias_mode("attn_generic", score_bias, &bias_mode)) return 1;
    const float* slopes = score_bias ? score_bias->slopes : nullptr;
    const float bias_scale = slopes ? score_bias->scale : 0.f;
    PTA_REQUIRE(M > 0 && nh > 0 && nkv > 0, "attn_generic: sizes must be positive (M=%d nh=%d nkv=%d)", M, nh, nkv);
    PTA_REQUIRE(nh % nkv == 0, "attn_generic: heads (%d) must be a multiple of kv heads (%d)", nh, nkv);
    PTA_REQUIRE(d > 0 && d <= 256, "attn_generic: head size %d is outside 1..256", d);
    PTA_REQUIRE(nh <= 65535, "attn_generic: at most 65535 heads, got %d", nh);
    PTA_REQUIRE(window >= 0, "attn_generic: window must be 0 (none) or positive, got %d", window);
    hipStream_t s = (hipStream_t)stream;
    dim3 grid(M, nh);
    if (dtype == PTA_F32)
        hipLaunchKernelGGL(attn_generic_kernel<float>, grid, dim3(PTA_WAVE), 0, s, (float*)out, (const float*)q,
                           (const float*)k_pool, (const float*)v_pool, block_table, bt_stride, token_seq, token_pos,
                           slopes, bias_mode, bias_scale, nh, nkv, d, scale, window);
    else if (dtype == PTA_BF16)
        hipLaunchKernelGGL(attn_generic_kernel<bf16_t>, grid, dim3(PTA_WAVE), 0, s, (bf16_t*)out, (const bf16_t*)q,
                           (const bf16_t*)k_pool, (const bf16_t*)v_pool, block_table, bt_stride, token_seq,
                           token_pos, slopes, bias_mode, bias_scale, nh, nkv, d, scale, window);
    else
        return pta_fail("attn_generic: unknown dtype %d", dtype);
    return pta_check_launch("attn_generic");
}
