// Causal attention over the paged cache on the matrix cores, bfloat16 in, 32-bit softmax and
// accumulation: the prefill kernel and the decode kernel are the same code.
//
// Work is laid out in *columns*: a column is one (new token, query head) pair of one KV head of one
// sequence, ordered token-major.  Heads that share a KV head therefore sit side by side and read
// its keys and values once: with one KV head for 71 query heads, a decode step's 71 columns are five
// tiles of 16 that share every key load.  A wave owns CT column tiles and walks the keys 32 at a
// time, always with the next block's keys and values already on their way:
//
//   S^T[32 keys x 16 cols]  = K[32 x d] . Q^T[d x 16]         (A = key rows, B = query columns)
//   online softmax over keys, per column (statistics in 32-bit, four lanes hold a column)
//   O^T[d x 16 cols]       += V^T[d x 32 keys] . P^T[32 x 16]  (A = value pages, stored transposed)
//   l[16 cols]             += 1[16 x 32] . P^T[32 x 16]        (the sums of the weights, as they were rounded)
//
// The score tile's accumulator layout (lane: column = lane % 16, four consecutive rows at
// (lane / 16) * 4) is turned into the B operand of the second product without leaving registers:
// key rows are assigned to the two 16-row score tiles so that a lane ends up with the eight
// consecutive keys 8 * (lane / 16) .. + 7 of the block, which is what the B operand wants.
//
// Decoding splits a long context over several workgroups (split_size keys each); each writes an
// unnormalised partial result with its running maximum and sum, and attn_combine merges them in split
// order.  A workgroup is one wave, or four or eight that take its keys block by block in turn and merge
// through LDS in the order of the waves; with the whole context in one workgroup there is no second
// launch, but all of a sequence's keys then pass through one compute unit.  Prefill does not split.
//
// score = q . k / sqrt(d) + alibi, alibi = bf16(bf16(slope) * bf16(key position)) / sqrt(d)
// (src/transformers/models/falcon/modeling_falcon.py:371-386, :407-422, :196-198, :1078-1085).
#pragma once

#include "common.h"
#include "pta_kernels.h"
#include "score_bias.h"

#include <stdlib.h>

#include <algorithm>
#include <cmath>
#include <type_traits>

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

union AFrag {
    uint4 u;
    bf16x8_t v;
};

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));

// two 32-bit floats to two bfloat16 (round to nearest even) in one instruction
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
    union { bf16x2_t b; uint32_t u; } c;
    c.b = __builtin_convertvector(f32x2_t{lo, hi}, bf16x2_t);
    return c.u;
}

// the largest of three in one instruction; written out because the compiler, asked for fmaxf of values that
// come through a branch, first makes each of them canonical with an instruction of its own
__device__ __forceinline__ float max3(float a, float b, float c) {
    float r;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}

#ifndef PTA_ATTN_DEPTH
#define PTA_ATTN_DEPTH 2  // register buffers of a wave that walks its keys alone (measured: four gain 15 % on one
                          // long range and lose as much on ranges of 64 to 256 keys, which are the ones chosen)
#endif
#define PTA_LOG2E 1.4426950408889634f

template <int DT>
struct KvBlock {
    AFrag k[2][(DT + 1) / 2];
    AFrag v[DT];
};

// Keys and values of the 32-key block at kb, straight into matrix-operand registers.  Nothing here
// depends on the loaded data, so the loads of the next block stay in flight while this one is used.
template <int DT>
__device__ __forceinline__ void load_block(KvBlock<DT>& b, int kb, const int* __restrict__ bt,
                                           const bf16_t* __restrict__ k_pool, const bf16_t* __restrict__ v_pool,
                                           int nkv, int kvh, int c, int gq) {
    constexpr int D = DT * 16, DS = (DT + 1) / 2, CHUNKS = D / 8;
    const long page = bt[kb >> 6];
    const int in_page = kb & 63;
    const bf16_t* kpage = k_pool + (page * nkv + kvh) * (long)(PTA_PAGE * D);
    const bf16_t* vpage = v_pool + (page * nkv + kvh) * (long)(PTA_PAGE * D);
    // key rows: tile tt, row r holds key 8*(r/4) + 4*tt + r%4 of the block
#pragma unroll
    for (int tt = 0; tt < 2; ++tt) {
        const bf16_t* kp = kpage + (long)(in_page + 8 * (c >> 2) + 4 * tt + (c & 3)) * D;
#pragma unroll
        for (int ds = 0; ds < DS; ++ds)
            b.k[tt][ds].u = *reinterpret_cast<const uint4*>(kp + min(ds * 4 + gq, CHUNKS - 1) * 8);
    }
    // value rows: feature dt*16 + c, keys 8*gq .. 8*gq+7 of the block
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
        b.v[dt].u = *reinterpret_cast<const uint4*>(vpage + (long)(dt * 16 + c) * PTA_PAGE + in_page + gq * 8);
}

// W = 1: a workgroup is one wave, which loads its keys and values straight from global memory.
// W > 1 (prompts; one token per sequence with many heads on a KV head): W waves with neighbouring column groups
// walk the keys together and share every block through LDS, so that a block crosses the vector memory path once
// for 16 * W * CT columns.
// WIN: the launch has a window (a kernel of its own, so that launches without one pay nothing for it).
// KS > 1 (one token per sequence): KS waves of a workgroup hold the same columns and take every KS-th block of the
// workgroup's keys; their partial results meet in LDS, so that a context walked by KS waves needs no second launch.
// AL: whether there is ALiBi, known when the kernel is compiled (0: none, 1: there is) or looked up (2).
// OCC: waves that a SIMD is to hold at least (the registers a wave may use follow from it; 1: as many as it likes).
template <int DT, int CT, int W, bool WIN, int KS = 1, int AL = 2, int OCC = 1>
__global__ __launch_bounds__(64 * W * KS, OCC) void attn_mfma_kernel(
    bf16_t* __restrict__ out, float* __restrict__ po, float* __restrict__ pm, float* __restrict__ pl,
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_pool, const bf16_t* __restrict__ v_pool,
    const int* __restrict__ block_table, int bt_stride, const int* __restrict__ cu_tokens,
    const int* __restrict__ seq_start, const float* __restrict__ slopes, int bias_mode, int nh, int nkv, float scale,
    float alibi_mul,
    int split_size, int n_splits, int window_arg, int paired) {
    constexpr int D = DT * 16;
    const int window = WIN ? window_arg : 0;
    constexpr int DS = (DT + 1) / 2;   // 32-wide steps over the head dimension
    constexpr int CHUNKS = D / 8;      // 16-byte chunks in a row of d elements
    static_assert(KS == 1 || W == 1, "waves either share key blocks or divide them");
    const int lane = threadIdx.x & 63, c = lane & 15, gq = lane >> 4;
    const int wave = KS > 1 ? 0 : __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);   // which columns of the workgroup
    const int kw = KS > 1 ? threadIdx.x >> 6 : 0;     // which blocks of the keys
    // Ranges of keys are handed out range-major: the first ranges of every sequence, which all of them have whole,
    // start first, and the last ones, which are short or empty for most sequences, fill the launch's end.  (Sequence-
    // major, 32 sequences of 16,405 keys in ranges of 1,024 left two whole ranges to start when the first ones ended:
    // 45.8 us against 30.3 us at 16,384 keys.)
    const int n_seqs_z = gridDim.z / n_splits;
    const int seq = blockIdx.z % n_seqs_z, split = blockIdx.z / n_seqs_z;
    const int kvh = blockIdx.y, g = nh / nkv;
    const int t0 = cu_tokens[seq], n_new = cu_tokens[seq + 1] - t0, start = seq_start[seq];
    const int ncols = n_new * g, n_groups = (ncols + 16 * CT * W - 1) / (16 * CT * W);
    // Column groups are handed out last first: late tokens see the most keys, and the longest work should
    // start first so that the launch ends evenly.  A paired launch has half the workgroups, and each takes a
    // late group and then the early group that mirrors it: under the causal mask the two together see as
    // many keys as any other pair, so a launch whose workgroups are all resident at once ends evenly too.
    for (int pass = 0; pass <= paired; ++pass) {
    int group = (int)(gridDim.x - 1 - blockIdx.x);
    if (paired) {
        const int late = n_groups - 1 - (int)blockIdx.x, early = (int)blockIdx.x;
        if (late < early || (pass == 1 && late == early)) return;
        group = pass == 0 ? late : early;
    }
    const int wg_col0 = group * (16 * CT * W);
    if (wg_col0 >= ncols) return;
    const int col0 = wg_col0 + wave * (16 * CT);
    const bool active = col0 < ncols;  // W > 1: a wave past the last column still loads and waits with the others
    const int last_col = min(ncols, col0 + 16 * CT) - 1;
    const int max_qpos = start + last_col / g;
    const int kv_len = start + n_new;
    // with a window a column at position t sees keys t - window + 1 .. t; this wave starts at the block of
    // the first key its first column sees (earlier pages may be gone), and at its range's start if split
    const int lo_first = window > 0 ? max(0, start + col0 / g - window + 1) : 0;   // lowest key any column sees
    const int lo_last = window > 0 ? max(0, max_qpos - window + 1) : 0;            // lowest key the last column sees
    const int k_begin = max(n_splits > 1 ? split * split_size : 0, lo_first & ~31);
    const int k_end = !active ? 0 : n_splits > 1 ? min(max_qpos + 1, split * split_size + split_size) : max_qpos + 1;
    const int kb_last = (kv_len - 1) & ~31;  // the last block that has a page
    // below this key index no column of this wave masks anything (columns are ordered by token)
    const int min_lim = min(start + col0 / g + 1, k_end);
    const uint4 zero4 = make_uint4(0u, 0u, 0u, 0u);
    // in the last 32-wide step of an odd number of 16-wide tiles, the upper half of the lanes has no data
    const uint32_t tail_keep = (DT % 2 == 1 && (DS - 1) * 4 + gq >= CHUNKS) ? 0u : 0xffffffffu;

    int qpos[CT], tok[CT], head[CT];
    float slope[CT];
    AFrag qf[CT][DS];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
        const int col = col0 + ct * 16 + c;
        const int colc = min(col, ncols - 1);
        const int t = colc / g;
        tok[ct] = t0 + t;
        head[ct] = kvh * g + colc % g;
        qpos[ct] = col < ncols ? start + t : -1;  // -1: every key is masked for a column that does not exist
        slope[ct] = slopes ? slopes[head[ct]] : 0.f;
        const bf16_t* qp = q + ((long)tok[ct] * nh + head[ct]) * D;
#pragma unroll
        for (int ds = 0; ds < DS; ++ds) {
            const int chunk = ds * 4 + gq;
            qf[ct][ds].u = *reinterpret_cast<const uint4*>(qp + min(chunk, CHUNKS - 1) * 8);
            if (chunk >= CHUNKS) qf[ct][ds].u = zero4;
        }
    }

    // The sum of a column's weights is one more product: a tile of ones in the place of the values adds the
    // block's (rounded) weights of every column into lacc, whose sixteen rows all hold the same sums.  The
    // vector units, which bound this kernel, are spared eight additions a tile; the matrix cores take a ninth
    // instruction beside eight.
    f32x4_t oacc[DT][CT], lacc[CT];
    float m_run[CT], m_raise[CT];  // m_raise: the raw score above which the running maximum is brought up
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
        m_run[ct] = -INFINITY;
        m_raise[ct] = -INFINITY;
        lacc[ct] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) oacc[dt][ct] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    }
    AFrag ones;
    ones.u = make_uint4(0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u);

    const int* bt = block_table + (long)seq * bt_stride;

    // AL says at compile time whether there is ALiBi (0: none, 1: there is; 2: whatever the launch brings), so
    // that the kernels for prompts, which are bound by their instruction stream, branch on nothing in it.
    const bool has_alibi = AL == 2 ? slopes != nullptr : AL == 1;
    // Scores are kept in units of log 2 (the scale carries log2 e), so that the exponential is the hardware's
    // exp2.  Without ALiBi the products are left unscaled, and the scale rides in the one multiply-add in front
    // of the exponential: s_mul is what a settled score is still to be multiplied by (positive).
    const float s_mul = has_alibi ? 1.0f : scale;

    // The work on a block of 32 keys, in the four pieces that the loops below put together:
    // the products S^T = K . Q^T of the block, raw
    auto scores = [&](const AFrag (&k)[2][DS], f32x4_t (&sacc)[2][CT]) {
#pragma unroll
        for (int tt = 0; tt < 2; ++tt) {
            AFrag k_last = k[tt][DS - 1];
            if (DT % 2 == 1) {
                k_last.u.x &= tail_keep; k_last.u.y &= tail_keep; k_last.u.z &= tail_keep; k_last.u.w &= tail_keep;
            }
#pragma unroll
            for (int ct = 0; ct < CT; ++ct) {
                f32x4_t acc = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ds = 0; ds < DS; ++ds)
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ds == DS - 1 ? k_last.v : k[tt][ds].v, qf[ct][ds].v, acc, 0, 0, 0);
                sacc[tt][ct] = acc;
            }
        }
    };
    // what the products become before the exponentials: with ALiBi, scaled and biased; keys that a column does
    // not see set to -inf; and the column's running maximum looked after.  MASKED = false is for a block that
    // every column of the wave sees whole: no key of it is past the sequence's end, past a column's own position
    // or before its window, and the code that would look is not there.
    auto settle = [&](auto masked_tag, f32x4_t (&sacc)[2][CT], int kb, float (&mx)[CT]) {
        constexpr bool MASKED = decltype(masked_tag)::value;
        const bool interior = !MASKED || (kb + 32 <= min_lim && kb >= lo_last);
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            if (has_alibi) {  // one branch for the tile, not one per score
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const int key = kb + 8 * gq + j;  // j = 4*tt + e
                    // the slope times the key's position, rounded as the reference rounds it (0) or exact (1), or
                    // times the key's distance from the query (2)
                    const float bias = bias_mode == 0 ? round_to_bf16(slope[ct] * round_to_bf16((float)key))
                                                      : slope[ct] * (float)(bias_mode == 2 ? key - qpos[ct] : key);
                    sacc[j >> 2][ct][j & 3] = sacc[j >> 2][ct][j & 3] * scale + bias * alibi_mul;
                }
            }
            if (MASKED && !interior) {
                const int lim = min(qpos[ct] + 1, k_end);  // keys below this, and from `lo` on, count for the column
                const int lo = window > 0 ? qpos[ct] - window + 1 : 0;
#pragma unroll
                for (int j = 0; j < 8; ++j)
                    if (kb + 8 * gq + j >= lim || kb + 8 * gq + j < lo) sacc[j >> 2][ct][j & 3] = -INFINITY;
            }
            const f32x4_t s0 = sacc[0][ct], s1 = sacc[1][ct];
            const float mx3 = max3(s1[2], s1[3], max3(s0[0], s0[1], s0[2]));
            mx[ct] = max3(s0[3], s1[0], s1[1]);
            mx[ct] = max3(mx[ct], mx3, mx3);
        }
    };
    // The running maximum is only a reference point for the exponentials, shared by the four lanes of a column;
    // it is brought up to the true maximum (an exchange between those lanes, and a rescale of what was summed)
    // only when some score of the block lies more than 2^8 above it, which after the first blocks of a row is
    // rare.  Weights stay below 2^8 and their rounding to bfloat16 is relative, so nothing is lost by a
    // reference that lags.  mx: the largest settled score of each tile's block, per lane.
    auto raise = [&](const float (&mx)[CT]) {
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            if (!__any(mx[ct] > m_raise[ct])) continue;
            float m = mx[ct] * s_mul;
            m = fmaxf(m, __shfl_xor(m, 16, 64));
            m = fmaxf(m, __shfl_xor(m, 32, 64));
            const float m_new = fmaxf(m_run[ct], m);
            const float corr = __builtin_amdgcn_exp2f(m_run[ct] - (m_new == -INFINITY ? 0.f : m_new));
            lacc[ct][0] *= corr;  // the one row of the sums that is read at the end
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                oacc[dt][ct][0] *= corr; oacc[dt][ct][1] *= corr; oacc[dt][ct][2] *= corr; oacc[dt][ct][3] *= corr;
            }
            m_run[ct] = m_new;
            m_raise[ct] = (m_new + 8.0f) / s_mul;
        }
    };
    // the weights 2^(score - reference) of the block, rounded, as the second product's operand
    auto weights = [&](const f32x4_t (&sacc)[2][CT], AFrag (&pf)[CT]) {
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            const float m_use = m_run[ct] == -INFINITY ? 0.f : m_run[ct];
            float p[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) p[j] = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[j >> 2][ct][j & 3], s_mul, -m_use));
            pf[ct].u = make_uint4(pack_bf16(p[0], p[1]), pack_bf16(p[2], p[3]), pack_bf16(p[4], p[5]), pack_bf16(p[6], p[7]));
        }
    };
    // sums of weights and O^T += V^T . P^T
    auto values = [&](const AFrag (&v)[DT], const AFrag (&pf)[CT]) {
#pragma unroll
        for (int ct = 0; ct < CT; ++ct)
            lacc[ct] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones.v, pf[ct].v, lacc[ct], 0, 0, 0);
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int ct = 0; ct < CT; ++ct)
                oacc[dt][ct] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(v[dt].v, pf[ct].v, oacc[dt][ct], 0, 0, 0);
    };
    const std::true_type masked_block;
    const std::false_type whole_block;
    // a key whose index is not below lim is taken out of eight values of consecutive keys from kbase on
    auto keep_below = [&](uint4& v, int kbase, int lim) {
        uint32_t mk[4];
#pragma unroll
        for (int w = 0; w < 4; ++w)
            mk[w] = (kbase + 2 * w < lim ? 0x0000ffffu : 0u) | (kbase + 2 * w + 1 < lim ? 0xffff0000u : 0u);
        v.x &= mk[0]; v.y &= mk[1]; v.z &= mk[2]; v.w &= mk[3];
    };

    if constexpr (W == 1) {
        // all of a block at once (a block past k_end changes nothing)
        auto use_block = [&](KvBlock<DT>& b, int kb) {
            if (kb + 32 > kv_len || kb >= k_end) {
                // positions past the sequence's end were never written; whatever lies there must not reach the
                // sum, not even with weight zero.  A block past this wave's range was loaded from a clamped
                // address and is dropped whole.
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) keep_below(b.v[dt].u, kb + gq * 8, kb >= k_end ? 0 : kv_len);
            }
            f32x4_t sacc[2][CT];
            AFrag pf[CT];
            float mx[CT];
            scores(b.k, sacc);
            settle(masked_block, sacc, kb, mx);
            raise(mx);
            weights(sacc, pf);
            values(b.v, pf);
        };
        // NB register buffers: while one block is used, the loads of the next NB - 1 are in flight (a wave alone
        // has nothing else to hide the memory's latency behind).  Addresses past the last block are clamped to
        // it, and such a block is not used.
        constexpr int NB = DT <= 4 ? PTA_ATTN_DEPTH : 2;
        constexpr int STEP = 32 * KS;  // from one block of this wave to its next
        KvBlock<DT> b[NB];
        const int k_first = k_begin + 32 * kw;
        const int n_mine = k_first < k_end ? (k_end - k_first + STEP - 1) / STEP : 0;  // blocks of this wave
        auto blk = [&](int j) { return j < n_mine ? min(k_first + STEP * j, kb_last) : kb_last; };
        if (n_mine > 0) {
#pragma unroll
            for (int i = 0; i < NB - 1; ++i) load_block<DT>(b[i], blk(i), bt, k_pool, v_pool, nkv, kvh, c, gq);
        }
        for (int j = 0; j < n_mine; j += NB) {
#pragma unroll
            for (int i = 0; i < NB; ++i) {
                load_block<DT>(b[(i + NB - 1) % NB], blk(j + i + NB - 1), bt, k_pool, v_pool, nkv, kvh, c, gq);
                __builtin_amdgcn_sched_barrier(0);
                if (j + i < n_mine) use_block(b[i], blk(j + i));
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    } else {
        // The workgroup's waves walk the keys of its last column together, a stage of SK keys (one or two
        // blocks) between barriers.  A stage goes global memory -> registers (one stage ahead) -> one of two
        // LDS buffers -> each wave's operand registers.  Key rows are stored in the order the score tiles want
        // them (within a block: tile tt, lane column c <-> key 8*(c/4) + 4*tt + c%4), so that sixteen lanes
        // read sixteen consecutive LDS rows; the row strides (D*2 + 16 and SK*2 + 16 bytes) put those on
        // distinct banks.  Small heads take a whole page per stage: half the barriers.
        constexpr int SK = D <= 64 ? 64 : 32, NBK = SK / 32;
        constexpr int KROW = D + 8, VROW = SK + 8;                // elements
        constexpr int KPIECES = SK / 8 * D, THREADS = 64 * W;     // 16-byte pieces of a stage's keys (and values)
        constexpr int PER = (KPIECES + THREADS - 1) / THREADS;
        constexpr int VCH = SK / 8;                               // pieces in a stage's row of values
        __shared__ __attribute__((aligned(16))) bf16_t kbuf[2][SK * KROW];
        __shared__ __attribute__((aligned(16))) bf16_t vbuf[2][D * VROW];
        const int tid = threadIdx.x;
        const int wg_last_col = min(ncols, wg_col0 + 16 * CT * W) - 1;
        // (a launch that cuts the keys into ranges walks its own range only)
        const int k_end_wg = n_splits > 1 ? min(start + wg_last_col / g + 1, split * split_size + split_size)
                                          : start + wg_last_col / g + 1;
        const int k_begin_wg = max(window > 0 ? max(0, start + wg_col0 / g - window + 1) & ~(SK - 1) : 0,
                                   n_splits > 1 ? split * split_size : 0);
        const int ks_last = (kv_len - 1) & ~(SK - 1);  // the last stage that has a page
        static_assert(PER <= 2, "a thread moves at most two pieces of keys and two of values per stage");
        static_assert(PTA_PAGE % SK == 0, "a stage lies in one page");
        // the pieces in flight are plain variables, not an array: an array that lambdas index stays in
        // scratch memory at the larger head sizes, and every stage then waits for its loads at once
        uint4 gk0, gk1, gv0, gv1;
        const int p0 = min(tid, KPIECES - 1), p1 = min(tid + THREADS, KPIECES - 1);
        auto gload = [&](int ks) {  // keys and values of the stage at ks (clamped to the last one there is)
            ks = min(ks, ks_last);
            const long page = ((long)bt[ks >> 6] * nkv + kvh) * (long)(PTA_PAGE * D);
            const bf16_t* kpage = k_pool + page + (long)(ks & 63) * D;
            const bf16_t* vpage = v_pool + page + (ks & 63);
            gk0 = *reinterpret_cast<const uint4*>(kpage + (long)(p0 / CHUNKS) * D + (p0 % CHUNKS) * 8);
            gv0 = *reinterpret_cast<const uint4*>(vpage + (long)(p0 / VCH) * PTA_PAGE + (p0 % VCH) * 8);
            if constexpr (PER > 1) {
                gk1 = *reinterpret_cast<const uint4*>(kpage + (long)(p1 / CHUNKS) * D + (p1 % CHUNKS) * 8);
                gv1 = *reinterpret_cast<const uint4*>(vpage + (long)(p1 / VCH) * PTA_PAGE + (p1 % VCH) * 8);
            }
        };
        // Positions past the sequence's end were never written; whatever lies there must not reach the sums, not
        // even with weight zero: such values are cleared on their way into LDS.
        auto put = [&](int buf, int p, const uint4& k, uint4 v, int ks) {
            if (p < KPIECES) {
                const int kk = p / CHUNKS;  // key of the stage -> its row in operand order
                const int row = (kk & ~31) + ((kk & 7) >> 2) * 16 + 4 * ((kk & 31) >> 3) + (kk & 3);
                *reinterpret_cast<uint4*>(&kbuf[buf][row * KROW + (p % CHUNKS) * 8]) = k;
                if (ks + SK > kv_len) keep_below(v, ks + (p % VCH) * 8, kv_len);
                *reinterpret_cast<uint4*>(&vbuf[buf][(p / VCH) * VROW + (p % VCH) * 8]) = v;
            }
        };
        auto sstore = [&](int ks) {  // into the buffer of the stage's number, whatever was loaded for it
            const int buf = (ks / SK) & 1;
            put(buf, tid, gk0, gv0, min(ks, ks_last));
            if constexpr (PER > 1) put(buf, tid + THREADS, gk1, gv1, min(ks, ks_last));
        };
        auto lfetch_k = [&](AFrag (&k)[2][DS], int kb) {  // the keys of the block at kb, from its stage's buffer
            const bf16_t* kb_lds = &kbuf[(kb / SK) & 1][((kb & (SK - 1)) + c) * KROW];
#pragma unroll
            for (int tt = 0; tt < 2; ++tt)
#pragma unroll
                for (int ds = 0; ds < DS; ++ds)
                    k[tt][ds].u = *reinterpret_cast<const uint4*>(kb_lds + tt * 16 * KROW + min(ds * 4 + gq, CHUNKS - 1) * 8);
        };
        auto lfetch_v = [&](AFrag (&v)[DT], int kb) {
            const bf16_t* vb_lds = &vbuf[(kb / SK) & 1][c * VROW + (kb & (SK - 1)) + gq * 8];
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) v[dt].u = *reinterpret_cast<const uint4*>(vb_lds + dt * 16 * VROW);
        };
        gload(k_begin_wg);
        sstore(k_begin_wg);
        __syncthreads();
        for (int ks = k_begin_wg; ks < k_end_wg; ks += SK) {
            gload(ks + SK);
            __builtin_amdgcn_sched_barrier(0);
            // the blocks of the stage that are this wave's: a plain loop with one way through it, in which the
            // compiler leaves the sums in their registers (two copies of the block's second half, one for the
            // rare block that raises a maximum, made it move all of them in every block)
            const int b_hi = min(ks + SK, k_end);
            for (int kb = max(ks, k_begin); kb < b_hi; kb += 32) {
                f32x4_t sacc[2][CT];
                AFrag pf[CT], kf[2][DS], vf[DT];
                float mx[CT];
                lfetch_k(kf, kb);
                scores(kf, sacc);
                if (kb + 32 <= min_lim && kb >= lo_last) settle(whole_block, sacc, kb, mx);
                else settle(masked_block, sacc, kb, mx);
                raise(mx);
                weights(sacc, pf);
                lfetch_v(vf, kb);
                values(vf, pf);
            }
            __builtin_amdgcn_sched_barrier(0);
            sstore(ks + SK);
            __syncthreads();
        }
    }

    if constexpr (KS > 1) {
        // every wave's sums, running maxima and unnormalised results go to LDS; then the (column tile, feature
        // tile) pairs are dealt out to the waves, and each merges its pairs over the waves in their order
        extern __shared__ __attribute__((aligned(16))) float ks_mem[];
        float4* so = reinterpret_cast<float4*>(ks_mem);
        float* sm = ks_mem + KS * CT * DT * 256;
        float* sl = sm + KS * CT * 16;
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
            const float l = lacc[ct][0];
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
                so[((kw * CT + ct) * DT + dt) * 64 + lane] =
                    make_float4(oacc[dt][ct][0], oacc[dt][ct][1], oacc[dt][ct][2], oacc[dt][ct][3]);
            if (gq == 0) {
                sm[(kw * CT + ct) * 16 + c] = m_run[ct];
                sl[(kw * CT + ct) * 16 + c] = l;
            }
        }
        __syncthreads();
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                if ((ct * DT + dt) % KS != kw || qpos[ct] < 0) continue;
                float mx = -INFINITY;
#pragma unroll
                for (int w = 0; w < KS; ++w) mx = fmaxf(mx, sm[(w * CT + ct) * 16 + c]);
                float l = 0.f;
                float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
                for (int w = 0; w < KS; ++w) {
                    const float mw = sm[(w * CT + ct) * 16 + c];
                    const float wgt = mw == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(mw - mx);
                    const float4 o = so[((w * CT + ct) * DT + dt) * 64 + lane];
                    l += wgt * sl[(w * CT + ct) * 16 + c];
                    acc.x += wgt * o.x; acc.y += wgt * o.y; acc.z += wgt * o.z; acc.w += wgt * o.w;
                }
                const long row = (long)tok[ct] * nh + head[ct];
                if (n_splits == 1) {
                    const float inv = 1.0f / l;
                    uint2 w2;
                    w2.x = pack_bf16(acc.x * inv, acc.y * inv);
                    w2.y = pack_bf16(acc.z * inv, acc.w * inv);
                    *reinterpret_cast<uint2*>(out + row * D + dt * 16 + gq * 4) = w2;
                } else {
                    *reinterpret_cast<float4*>(po + (row * n_splits + split) * D + dt * 16 + gq * 4) = acc;
                    if (dt == 0 && gq == 0) {
                        pm[row * n_splits + split] = mx;
                        pl[row * n_splits + split] = l;
                    }
                }
            }
        }
    } else {
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
        const float l = lacc[ct][0];
        if (qpos[ct] < 0) continue;
        const long row = (long)tok[ct] * nh + head[ct];
        if (n_splits == 1) {
            const float inv = 1.0f / l;
            bf16_t* o = out + row * D;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                uint2 w;
                w.x = pack_bf16(oacc[dt][ct][0] * inv, oacc[dt][ct][1] * inv);
                w.y = pack_bf16(oacc[dt][ct][2] * inv, oacc[dt][ct][3] * inv);
                *reinterpret_cast<uint2*>(o + dt * 16 + gq * 4) = w;
            }
        } else {
            // a range past the column's keys has nothing to add: only its marker is written, and the combine
            // does not read past the last range that has one.  A range before a window is followed by ranges
            // that count, so it is read with weight zero and must hold numbers: the (zero) sums are written.
            if (k_begin < k_end || WIN) {
                float* o = po + (row * n_splits + split) * D;
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)
                    *reinterpret_cast<float4*>(o + dt * 16 + gq * 4) =
                        make_float4(oacc[dt][ct][0], oacc[dt][ct][1], oacc[dt][ct][2], oacc[dt][ct][3]);
            }
            if (gq == 0) {
                pm[row * n_splits + split] = m_run[ct];
                pl[row * n_splits + split] = l;
            }
        }
    }
    }
    }  // pass
}

struct AttnLaunch {
    bf16_t* out; float *po, *pm, *pl;
    const bf16_t *q, *k_pool, *v_pool;
    const int* block_table; int bt_stride;
    const int *cu_tokens, *seq_start; const float* slopes; int bias_mode; float bias_scale;
    int n_seqs, max_new, nh, nkv; float scale;
    int split_size, n_splits, window;
    int paired;  // workgroups take two column groups each, a late one and the early one that mirrors it
    int waves;   // one token per sequence: waves of a workgroup that divide its keys among them
    hipStream_t s;
};

// LDS in which KS waves of CT column tiles leave their partial results
constexpr size_t key_split_lds(int dt, int ct, int ks) { return ks == 1 ? 0 : (size_t)ks * ct * (dt * 1024 + 128); }

template <int DT, int CT, int W, int KS = 1, int OCC = 1>
static void launch_attn(const AttnLaunch& a) {
    const int g = a.nh / a.nkv;
    const int groups = (a.max_new * g + 16 * CT * W - 1) / (16 * CT * W);
    const int paired = a.paired && groups > 1 ? 1 : 0;
    const dim3 grid(paired ? (groups + 1) / 2 : groups, a.nkv, a.n_seqs * a.n_splits);
    // prompts: a kernel with ALiBi and one without; one token per sequence: one kernel that looks
    constexpr int AL0 = W > 1 ? 0 : 2, AL1 = W > 1 ? 1 : 2;
    auto kern = a.window > 0 ? attn_mfma_kernel<DT, CT, W, true, KS, AL0, OCC> : attn_mfma_kernel<DT, CT, W, false, KS, AL0, OCC>;
    if (W > 1 && a.slopes)
        kern = a.window > 0 ? attn_mfma_kernel<DT, CT, W, true, KS, AL1, OCC> : attn_mfma_kernel<DT, CT, W, false, KS, AL1, OCC>;
    constexpr size_t lds = key_split_lds(DT, CT, KS);
    if constexpr (lds > 64 * 1024) {  // more than a launch may ask for unless the kernel has been told, once per device
        static bool told[64] = {};
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) dev = 0;
        if (!told[dev]) {
            (void)hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            told[dev] = true;
        }
    }
    hipLaunchKernelGGL(kern, grid, dim3(64 * W * KS), lds, a.s, a.out, a.po, a.pm, a.pl, a.q, a.k_pool, a.v_pool,
                       a.block_table, a.bt_stride, a.cu_tokens, a.seq_start, a.slopes, a.bias_mode, a.nh, a.nkv,
                       a.scale * PTA_LOG2E, PTA_LOG2E * a.bias_scale, a.split_size, a.n_splits, a.window, paired);
}

// column tiles (of sixteen query heads of one KV head) that one wave of a decode launch holds at most:
// what the head size leaves registers for
constexpr int decode_max_tiles(int dt) { return dt <= 4 ? 5 : dt <= 8 ? 4 : 1; }

// waves that may divide a workgroup's keys: one, or four or eight with up to two column tiles each (more tiles
// gained nothing with more waves wherever that was measured, and every combination is a kernel to build)
constexpr bool decode_waves_built(int dt, int ct, int ks) {
    return ks == 1 || ((ks == 4 || ks == 8) && ct <= 2 && ct <= decode_max_tiles(dt) &&
                       key_split_lds(dt, ct, ks) <= 144 * 1024);
}

template <int DT, int CT, int KS = 1>
static bool launch_decode_waves(const AttnLaunch& a) {
    if constexpr (KS <= 8) {
        if (a.waves == KS) {
            if constexpr (decode_waves_built(DT, CT, KS)) { launch_attn<DT, CT, 1, KS>(a); return true; }
            return false;
        }
        return launch_decode_waves<DT, CT, KS * 2>(a);
    }
    return false;
}

// one token per sequence: workgroups of `waves` waves with `tiles` column tiles
template <int DT, int CT = 1>
static bool launch_decode(const AttnLaunch& a, int tiles) {
    if constexpr (CT <= decode_max_tiles(DT)) {
        if (tiles == CT) return launch_decode_waves<DT, CT>(a);
        return launch_decode<DT, CT + 1>(a, tiles);
    }
    return false;
}

// prompts: four waves of two column tiles share each stage of keys through LDS (head sizes up to 128;
// beyond, one wave per workgroup).  Heads up to 64 fit four waves a SIMD (measured at 8,192 tokens, 71 heads
// on one KV head of 64: as many registers as the compiler likes, three waves, 800 us a layer; four waves 760;
// a third column tile, 256 registers, two waves, 817), and with many column groups eight waves share a stage
// (`wide`: 256 columns a workgroup, half the staging for every wave).
constexpr int prompt_columns(int dt, bool wide) { return dt <= 4 && wide ? 256 : dt <= 8 ? 128 : 16; }

template <int DT>
static void launch_prompt(const AttnLaunch& a, bool wide) {
    if constexpr (DT <= 4) {
        if (wide) launch_attn<DT, 2, 8, 1, 4>(a);
        else launch_attn<DT, 2, 4, 1, 4>(a);
    } else if constexpr (DT <= 8) launch_attn<DT, 2, 4>(a);
    else launch_attn<DT, 1, 1>(a);
}

// One token per sequence, the heads of a KV head on the waves of one workgroup, which share its keys through LDS
// as a prompt's column groups do: a wave per tile of sixteen heads for four or five tiles (49 to 80 heads on a KV
// head), four waves of two tiles for six to eight.  Built for head sizes 64 and 128.  Fewer heads on a KV head fit
// the tiles of one wave (`launch_decode`), which reads the keys once as well.
constexpr bool decode_shared_built(int dt, int tiles) { return (dt == 4 || dt == 8) && tiles >= 4 && tiles <= 8; }

template <int DT>
static bool launch_decode_shared(const AttnLaunch& a) {
    if constexpr (DT == 4 || DT == 8) {
        constexpr int OCC = DT <= 4 ? 4 : 1;
        const int tiles = (a.nh / a.nkv + 15) / 16;
        if (tiles == 4) launch_attn<DT, 1, 4, 1, OCC>(a);
        else if (tiles == 5) launch_attn<DT, 1, 5, 1, OCC>(a);
        else if (tiles >= 6 && tiles <= 8) launch_attn<DT, 2, 4, 1, OCC>(a);
        else return false;
        return true;
    }
    return false;
}

// What pta_attn_mfma launches for heads of DT x 16 elements.  Every head size is a translation unit of its own
// (attn_mfma_dt*.hip, one explicit instantiation each), so that the sizes compile side by side.
// 0: launched; 1: no kernel with shared keys at this size; 2: no kernel for these waves and column tiles.
template <int DT>
int attn_launch_head(const AttnLaunch& a, bool shared, bool narrow, bool wide, int tiles) {
    if (shared) return launch_decode_shared<DT>(a) ? 0 : 1;
    if (!narrow) {
        launch_prompt<DT>(a, wide);
        return 0;
    }
    return launch_decode<DT>(a, tiles) ? 0 : 2;
}
