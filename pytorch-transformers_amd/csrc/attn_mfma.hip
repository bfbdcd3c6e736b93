// The entry points of the attention on the matrix cores and the merge of a decode launch's ranges of keys; the
// attention kernel itself and its launchers are in attn_mfma_impl.h, instantiated per head size in attn_mfma_dt*.hip.
#include "attn_mfma_impl.h"

#define PTA_ATTN_HEAD(DT_) extern template int attn_launch_head<DT_>(const AttnLaunch&, bool, bool, bool, int);
PTA_ATTN_HEAD(1) PTA_ATTN_HEAD(2) PTA_ATTN_HEAD(3) PTA_ATTN_HEAD(4) PTA_ATTN_HEAD(5) PTA_ATTN_HEAD(6) PTA_ATTN_HEAD(7)
PTA_ATTN_HEAD(8) PTA_ATTN_HEAD(16)
#undef PTA_ATTN_HEAD

// out[row, :] = sum_s w_s po[row, s, :] / sum_s w_s pl[row, s], w_s = 2^(pm[row, s] - max_s pm).  A split whose
// maximum is -inf (a range past the row's keys) has weight zero and is not read.
//
// A row's splits are many short vectors, and a chain of loads one behind the other is what this kernel's time
// would be: so LPS lanes (the next power of two from D/4) take one split's vector as float4 each, the 64/LPS
// groups of a wave and the WAVES waves of the workgroup take every (64/LPS * WAVES)-th split, four of them in
// flight per group; the groups' sums are added across the wave by lane exchange and across waves through LDS in
// wave order.  The order of the additions depends on (n_splits, D, WAVES) alone.
template <int WAVES>
__global__ __launch_bounds__(64 * WAVES) void attn_combine_kernel(bf16_t* __restrict__ out, const float* __restrict__ po,
                                                                  const float* __restrict__ pm, const float* __restrict__ pl,
                                                                  int D, int n_splits, int lps) {
    __shared__ float part[WAVES][256 + 4];
    const long row = blockIdx.x;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const float* m = pm + row * n_splits;
    const float* l = pl + row * n_splits;
    float mx = -INFINITY;
    for (int s = lane; s < n_splits; s += 64) mx = fmaxf(mx, m[s]);
    mx = wave_max(mx);
    const int per_wave = 64 / lps, g = lane / lps, c = (lane % lps) * 4;
    const bool active = c < D;
    const int stride = per_wave * WAVES;
    const float* p = po + row * (long)n_splits * D + c;
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    float L = 0.f;
    for (int s0 = wave * per_wave + g; s0 < n_splits; s0 += 4 * stride) {
        float w[4], ll[4];
        float4 v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int s = s0 + u * stride;
            w[u] = 0.f; ll[u] = 0.f; v[u] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (s < n_splits) {
                const float ms = m[s];
                if (ms != -INFINITY) {
                    w[u] = __builtin_amdgcn_exp2f(ms - mx);
                    ll[u] = l[s];
                    if (active) v[u] = *reinterpret_cast<const float4*>(p + (long)s * D);
                }
            }
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            acc.x += w[u] * v[u].x; acc.y += w[u] * v[u].y; acc.z += w[u] * v[u].z; acc.w += w[u] * v[u].w;
            L += w[u] * ll[u];
        }
    }
    for (int off = lps; off < 64; off <<= 1) {
        acc.x += __shfl_xor(acc.x, off); acc.y += __shfl_xor(acc.y, off);
        acc.z += __shfl_xor(acc.z, off); acc.w += __shfl_xor(acc.w, off);
        L += __shfl_xor(L, off);
    }
    if constexpr (WAVES > 1) {
        if (g == 0 && active) *reinterpret_cast<float4*>(&part[wave][c]) = acc;
        if (lane == 0) part[wave][256] = L;
        __syncthreads();
        if (wave != 0) return;
        acc = make_float4(0.f, 0.f, 0.f, 0.f);
        L = 0.f;
        if (active) {
#pragma unroll
            for (int wv = 0; wv < WAVES; ++wv) {
                const float4 a = *reinterpret_cast<const float4*>(&part[wv][c]);
                acc.x += a.x; acc.y += a.y; acc.z += a.z; acc.w += a.w;
                L += part[wv][256];
            }
        }
    }
    if (g == 0 && active) {
        const float inv = 1.0f / L;
        bf16_t r[4] = {f32_to_bf16_bits(acc.x * inv), f32_to_bf16_bits(acc.y * inv), f32_to_bf16_bits(acc.z * inv),
                       f32_to_bf16_bits(acc.w * inv)};
        *reinterpret_cast<uint2*>(out + row * D + c) = *reinterpret_cast<const uint2*>(r);
    }
}

extern "C" int pta_attn_decode_shared_ok(int d, int heads_per_kv_head) {
    return d % 16 == 0 && heads_per_kv_head > 0 && decode_shared_built(d / 16, (heads_per_kv_head + 15) / 16);
}

extern "C" int pta_attn_mfma_supported(int d) { return d % 16 == 0 && ((d >= 16 && d <= 128) || d == 256); }

extern "C" int pta_attn_decode_max_tiles(int d) { return decode_max_tiles(d / 16); }

extern "C" int pta_attn_decode_waves_ok(int d, int tiles, int waves) {
    return pta_attn_mfma_supported(d) && tiles >= 1 && decode_waves_built(d / 16, tiles, waves);
}

extern "C" int pta_attn_mfma(void* out, const void* q, const void* k_pool, const void* v_pool, const int* block_table,
                             int bt_stride, const int* cu_tokens, const int* seq_start, const PtaScoreBias* score_bias,
                             int n_seqs, int max_new, int M, int nh, int nkv, int d, float scale, int split_size, int n_splits,
                             float* po, float* pm, float* pl, int window, int decode_tiles, int decode_waves,
                             int prompt_wide, void* stream) {
    PTA_REQUIRE(n_seqs > 0 && max_new > 0 && M > 0 && nh > 0 && nkv > 0, "attn_mfma: sizes must be positive");
    int bias_mode = 0;
    if (pta_score_bias_mode("attn_mfma", score_bias, &bias_mode)) return 1;
    const float* slopes = score_bias ? score_bias->slopes : nullptr;
    const float bias_scale = slopes ? score_bias->scale : 0.f;
    PTA_REQUIRE(nh % nkv == 0, "attn_mfma: heads (%d) must be a multiple of kv heads (%d)", nh, nkv);
    PTA_REQUIRE(pta_attn_mfma_supported(d), "attn_mfma: head size %d is not built (16..128 in steps of 16, or 256)", d);
    PTA_REQUIRE(n_splits >= 1 && n_splits <= 1024, "attn_mfma: n_splits must be 1..1024, got %d", n_splits);
    PTA_REQUIRE(window >= 0, "attn_mfma: window must be 0 (none) or positive, got %d", window);
    PTA_REQUIRE(n_splits == 1 || (split_size > 0 && split_size % 64 == 0 && po && pm && pl),
                "attn_mfma: splitting needs a split size that is a multiple of 64 and buffers for partial results");
    PTA_REQUIRE((long)n_seqs * n_splits <= 65535 && nkv <= 65535, "attn_mfma: too many sequences x splits for one launch");
    PTA_REQUIRE(((uintptr_t)q % 16) == 0 && ((uintptr_t)k_pool % 16) == 0 && ((uintptr_t)v_pool % 16) == 0 &&
                    ((uintptr_t)out % 8) == 0, "attn_mfma: pointers must be 16-byte aligned");
    hipStream_t s = (hipStream_t)stream;
    // Prompts: four waves of two column tiles share each stage of keys through LDS (head sizes up to 128;
    // beyond, one wave per workgroup).
    // One token per sequence (decode): workgroups of `decode_waves` waves, each of which holds `decode_tiles` column
    // tiles of its KV head (at most what the head size leaves registers for).  More tiles: the keys cross the memory
    // path fewer times; fewer: shorter waves, more of them (71 heads on one KV head, 2,048 keys: 64
    // sequences 39.5 us a layer with one tile, 27.5 us with five; 8 sequences 14.6 and 18.5 us).
    // `decode_waves` 0: the heads of a KV head on the waves of one workgroup, keys shared through LDS
    // (`launch_decode_shared`; `decode_tiles` does not apply).  71 heads on one KV head of 64, with the merge of
    // the ranges, after a flush of the caches: 64 sequences of 1,100 keys 12.6 us against 17.5 with the best cut
    // of one-wave workgroups, of 2,100 keys 14.8 against 26.0; 8 sequences of 16,384 keys 19.8 against 24.8; 8
    // sequences of 1,100 keys 11.4 against 9.8.
    const bool shared = max_new == 1 && decode_waves == 0;
    PTA_REQUIRE(!shared || pta_attn_decode_shared_ok(d, nh / nkv),
                "attn_mfma: a decode launch with keys shared through LDS is not built for %d heads on a KV head of "
                "size %d (49 to 128 heads, sizes 64 and 128)", nh / nkv, d);
    const bool narrow = max_new == 1 && !shared;
    // Prompts: whether workgroups take a late and an early column group each.  Paired workgroups all do the
    // same work, which ends a launch evenly if their number fills the compute units evenly; unpaired ones are
    // twice as many and of all lengths, which the longest-first order spreads well over any number of units.
    // In units of a mean workgroup's work a unit's share is max(n / units, 2) unpaired and 2 ceil(n / 2 / units)
    // paired; pairs win where the two are equal (32 heads on 8 KV heads of 128: 2,048 tokens 92 -> 77 us a layer,
    // 8,192 tokens 787 -> 657; 128 on 8 of 64: 123 -> 103 and 1,264 -> 1,214) and lose where they are not (71 on
    // 1 of 64: 68 -> 89, and 737 -> 766 where the two differ by 2 %).
    // Eight waves a workgroup where that still leaves four workgroups and more for every compute unit (71 heads on
    // 1 KV head of 64: 2,048 tokens 67 -> 72 us a layer, 4,096 the same, 8,192 712 -> 693, 16,384 2,542 -> 2,433;
    // 128 on 8 of 64: 2,048 tokens 101 -> 94, 8,192 1,213 -> 1,151).
    static const int pair_env = getenv("PTA_ATTN_PAIR") ? atoi(getenv("PTA_ATTN_PAIR")) : -1;
    int paired = 0;
    bool wide = false;
    if (!narrow && !shared) {
        const double units = pta_compute_units();
        const double wide_wgs = std::ceil((double)M * (nh / nkv) / prompt_columns(d / 16, true)) * nkv;
        wide = d <= 64 && (prompt_wide >= 0 ? prompt_wide != 0 : wide_wgs >= 4.0 * units);
        const double wgs = std::ceil((double)M * (nh / nkv) / prompt_columns(d / 16, wide)) * nkv;
        paired = pair_env >= 0 ? pair_env : 2.0 * std::ceil(wgs / 2.0 / units) <= 1.01 * std::max(wgs / units, 2.0);
    }
    const int dct_most = std::min((nh / nkv + 15) / 16, pta_attn_decode_max_tiles(d));
    PTA_REQUIRE(decode_tiles >= 0 && decode_tiles <= dct_most,
                "attn_mfma: %d column tiles per decode wave; these sizes allow 1..%d (0: as many as that)", decode_tiles,
                dct_most);
    const int dct = decode_tiles > 0 ? decode_tiles : dct_most;
    PTA_REQUIRE(!narrow || pta_attn_decode_waves_ok(d, dct, decode_waves),
                "attn_mfma: %d waves on the keys of a workgroup with %d column tiles are not built for head size %d "
                "(one wave, or four or eight with up to two tiles)", decode_waves, dct, d);
    const AttnLaunch a{(bf16_t*)out, po, pm, pl, (const bf16_t*)q, (const bf16_t*)k_pool, (const bf16_t*)v_pool,
                       block_table, bt_stride, cu_tokens, seq_start, slopes, bias_mode, bias_scale, n_seqs, max_new, nh, nkv, scale,
                       split_size, n_splits, window, paired, narrow ? decode_waves : 1, s};
#define PTA_ATTN_CASE(DT_)                                                                        \
    case DT_: {                                                                                   \
        const int none = attn_launch_head<DT_>(a, shared, narrow, wide, dct);                     \
        if (none == 1) return pta_fail("attn_mfma: no kernel with shared keys at head size %d", d); \
        if (none == 2)                                                                            \
            return pta_fail("attn_mfma: no kernel for %d waves and %d column tiles at head size %d", decode_waves, dct, d); \
        break;                                                                                    \
    }
    switch (d / 16) {
        PTA_ATTN_CASE(1)
        PTA_ATTN_CASE(2)
        PTA_ATTN_CASE(3)
        PTA_ATTN_CASE(4)
        PTA_ATTN_CASE(5)
        PTA_ATTN_CASE(6)
        PTA_ATTN_CASE(7)
        PTA_ATTN_CASE(8)
        PTA_ATTN_CASE(16)
        default:
            return pta_fail("attn_mfma: head size %d is not built", d);
    }
#undef PTA_ATTN_CASE
    int rc = pta_check_launch("attn_mfma");
    if (rc) return rc;
    if (n_splits > 1) {
        int lps = 4;  // lanes that share a split's vector of d floats, a float4 each
        while (lps * 4 < d) lps *= 2;
        const dim3 rows((unsigned)((long)M * nh));
        if (n_splits > 4 * (64 / lps))  // more splits than one wave has in flight at once
            hipLaunchKernelGGL(attn_combine_kernel<4>, rows, dim3(256), 0, s, (bf16_t*)out, po, pm, pl, d, n_splits, lps);
        else
            hipLaunchKernelGGL(attn_combine_kernel<1>, rows, dim3(64), 0, s, (bf16_t*)out, po, pm, pl, d, n_splits, lps);
        rc = pta_check_launch("attn_combine");
    }
    return rc;
}
