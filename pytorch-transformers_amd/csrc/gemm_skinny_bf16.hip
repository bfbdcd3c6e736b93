// y[M,N] = act(x[M,K] . W[N,K]^T + bias) + add1 + add2 for few rows (M <= 64), bfloat16 in,
// 32-bit accumulation on the matrix cores.  This is the decode step's linear layer: the work is
// reading W once from HBM, so the kernel is laid out for that, not for the arithmetic.
//
// A workgroup of S waves owns 16*RT rows of W and all of K.  Its waves take the 64-element K-steps
// round robin (wave w: steps w, w + S, ...), so neighbouring waves read neighbouring 128-byte lines
// of the same rows.  A wave works in stages of U steps and always has the next stage's loads in
// flight while the matrix cores consume the current one (two register buffers), so every wave
// keeps 2*U*RT KB of W on its way from HBM for as long as it runs.  W rows are the A operand of
// v_mfma_f32_16x16x32_bf16 (lane: row = lane % 16, eight consecutive k at (lane / 16) * 8, one
// 16-byte load straight from global memory), x rows are the B operand (same shape, buffer loads whose
// bounds are the M real rows, so the padding rows of the tile read zeros and cost no traffic).  The S partial tiles are summed through LDS in wave order, then bias,
// activation and additions are applied and the tile is stored.  S is chosen from N and K alone, so
// the order of summation never depends on M or on what else is in the batch.
#include "common.h"
#include "pta_kernels.h"
#include "qkv_tail.h"

#include <stdlib.h>

#include <algorithm>

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

typedef int i32x4_t __attribute__((ext_vector_type(4)));

union Frag {
    uint4 u;
    bf16x8_t v;
    i32x4_t i;
};

template <typename OutT> struct OutIo;
template <> struct OutIo<float> {
    static __device__ __forceinline__ float round(float v) { return v; }
    static __device__ __forceinline__ void st(float* p, float v) { *p = v; }
};
template <> struct OutIo<bf16_t> {
    static __device__ __forceinline__ float round(float v) { return round_to_bf16(v); }
    static __device__ __forceinline__ void st(bf16_t* p, float v) { *p = f32_to_bf16_bits(v); }
};

template <int MT, int RT, int U>
struct Stage {
    Frag a[U][2][RT];
    Frag b[U][2][MT];
    uint32_t keep[U][2];  // all ones if the chunk lies inside K, else zero
};

// Loads are unconditional: the address is clamped into the row, and the data of a chunk past K is
// masked to zero only when it is used.  A load under a branch, or a mask applied here, would make
// the wave wait for loads it has just issued, and the two stages would no longer overlap.
template <int MT, int RT, int U>
__device__ __forceinline__ void load_stage(Stage<MT, RT, U>& st, const bf16_t* const (&wrow)[RT],
                                           __amdgpu_buffer_rsrc_t xres, int r, int first_step, int S, int g, int K,
                                           int nsteps, int rot) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
        // the workgroup walks K from its own starting step and wraps round; steps past the last are masked
        int step = first_step + u * S;
        if (step < nsteps) { step += rot; step -= step >= nsteps ? nsteps : 0; }
        const int k0 = step * 64 + g * 8;  // K % 8 == 0: a chunk of 8 is inside K or outside it
#pragma unroll
        for (int hf = 0; hf < 2; ++hf) {
            const int k = k0 + hf * 32;
            const int kc = min(k, K - 8);
            st.keep[u][hf] = k < K ? 0xffffffffu : 0u;
#pragma unroll
            for (int t = 0; t < RT; ++t) st.a[u][hf][t].u = *reinterpret_cast<const uint4*>(wrow[t] + kc);
#pragma unroll
            for (int t = 0; t < MT; ++t)  // a row past M lies outside the buffer's bounds: it reads zeros and costs no traffic
                st.b[u][hf][t].i = __builtin_amdgcn_raw_buffer_load_b128(xres, ((t * 16 + r) * K + kc) * 2, 0, 0);
        }
    }
}

template <int MT, int RT, int U>
__device__ __forceinline__ void compute_stage(const Stage<MT, RT, U>& st, f32x4_t (&acc)[RT][MT]) {
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
        for (int hf = 0; hf < 2; ++hf)
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) {
                Frag a = st.a[u][hf][rt];
                const uint32_t keep = st.keep[u][hf];
                a.u.x &= keep; a.u.y &= keep; a.u.z &= keep; a.u.w &= keep;
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
                    acc[rt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, st.b[u][hf][mt].v, acc[rt][mt], 0, 0, 0);
            }
}

// One product of a launch: a launch may carry two that share M and K (a block's two input projections),
// so that the second one's workgroups fill the chip while the first one's drain.
struct SkinnyProblem {
    void* y;
    const bf16_t* x;
    const bf16_t* W;
    const float* bias;
    const bf16_t* add1;
    const bf16_t* add2;
    int N;
    int act;
    int blocks;  // workgroups of this product
};

// With a QkvTail (qkv_tail.h) the first product's rows are not stored: they are split into heads, rotated and written
// as queries and into the cache pages.  The rotation works on pairs of a head's elements, so a workgroup takes the
// first elements of sixteen pairs as its first row tile and their partners as its second (TAIL 1: whole heads in
// half-split pairs, or no rotation: pair p is elements p and p + d/2, and four pairs in a row are stored as eight
// bytes; TAIL 2: any rotation that qkv_tail_pair_elements describes, stored element by element).
template <int MT, int RT, int U, typename OutT, int TAIL = 0>
__global__ __launch_bounds__(512) void gemm_skinny_kernel(SkinnyProblem pa, SkinnyProblem pb, int M, int K,
                                                          int rot_stride, QkvTail tail) {
    static_assert(!TAIL || (RT == 2 && MT == 1 && sizeof(OutT) == 2), "the query_key_value tail: two row tiles, sixteen rows of x");
    extern __shared__ f32x4_t part[];  // [S][RT][MT][64]
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, S = blockDim.x >> 6;
    const int r = lane & 15, g = lane >> 4;
    const bool second = (int)blockIdx.x >= pa.blocks;
    OutT* __restrict__ y = (OutT*)(second ? pb.y : pa.y);
    const bf16_t* __restrict__ x = second ? pb.x : pa.x;
    const bf16_t* __restrict__ W = second ? pb.W : pa.W;
    const float* __restrict__ bias = second ? pb.bias : pa.bias;
    const bf16_t* __restrict__ add1 = second ? pb.add1 : pa.add1;
    const bf16_t* __restrict__ add2 = second ? pb.add2 : pa.add2;
    const int N = second ? pb.N : pa.N, act = second ? pb.act : pa.act;
    // the workgroups of a product share its rows evenly: this one has rows n0 .. n1 - 1, at most 16 * RT
    const int blocks = second ? pb.blocks : pa.blocks, j = (int)blockIdx.x - (second ? pa.blocks : 0);
    const int n0 = (int)((long)j * N / blocks), n1 = (int)((long)(j + 1) * N / blocks);
    const bf16_t* wrow[RT];
    const bool tailed = TAIL && !second;
    // with the tail: workgroup j has pairs s16*16 .. +15 of segment seg (a head's q, k or v)
    const int per_seg = TAIL ? tail.d / 32 : 1, seg = j / per_seg, s16 = j % per_seg;
    int pair_e[2] = {0, 0};  // the two elements of this lane's pair
    if (TAIL == 1) {
        pair_e[0] = s16 * 16 + r;
        pair_e[1] = pair_e[0] + (tail.d >> 1);
    } else if (TAIL == 2) {
        bool rotated;
        qkv_tail_pair_elements(tail.rot, tail.d, s16 * 16 + r, pair_e[0], pair_e[1], rotated);
    }
#pragma unroll
    for (int t = 0; t < RT; ++t) {
        const int row = tailed ? seg * tail.d + pair_e[t & 1] : min(n0 + t * 16 + r, n1 - 1);
        wrow[t] = W + (long)row * K;
    }
    // x through a buffer descriptor whose bounds are the M real rows (0x00020000: 32-bit raw data format)
    __amdgpu_buffer_rsrc_t xres = __builtin_amdgcn_make_buffer_rsrc((void*)x, 0, M * K * 2, 0x00020000);

    f32x4_t acc[RT][MT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[rt][mt] = f32x4_t{0.f, 0.f, 0.f, 0.f};

    const int nsteps = (K + 63) >> 6;
    // Where a row of W is a power of two long, every workgroup walking K from its start would ask the same few
    // memory channels at the same time (K = 4,096: 13 % slower than K = 4,160).  So each starts `rot_stride`
    // steps after its neighbour.  A feature's order of summation follows from N, K and the launch alone.
    const int rot = rot_stride > 0 ? (int)(((long)blockIdx.x * rot_stride) % nsteps) : 0;
    Stage<MT, RT, U> s0, s1;
    load_stage<MT, RT, U>(s0, wrow, xres, r, wave, S, g, K, nsteps, rot);
    // the scheduling barriers keep the compiler from sinking a stage's loads down to their first
    // use, which would shrink what is in flight to a load or two
    for (int step = wave; step < nsteps; step += 2 * U * S) {
        load_stage<MT, RT, U>(s1, wrow, xres, r, step + U * S, S, g, K, nsteps, rot);
        __builtin_amdgcn_sched_barrier(0);
        compute_stage<MT, RT, U>(s0, acc);
        __builtin_amdgcn_sched_barrier(0);
        load_stage<MT, RT, U>(s0, wrow, xres, r, step + 2 * U * S, S, g, K, nsteps, rot);
        __builtin_amdgcn_sched_barrier(0);
        compute_stage<MT, RT, U>(s1, acc);
        __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) part[((wave * RT + rt) * MT + mt) * 64 + lane] = acc[rt][mt];
    __syncthreads();

    if constexpr (TAIL) {
        if (tailed) {
            // thread ln: token m = ln % 16, features i0 .. i0+3 of the segment's lower half and their partners
            for (int ln = threadIdx.x; ln < 64; ln += blockDim.x) {
                f32x4_t lo = part[ln], hi = part[64 + ln];
                for (int w = 1; w < S; ++w) {
                    const f32x4_t p = part[(w * 2) * 64 + ln], q = part[(w * 2 + 1) * 64 + ln];
                    lo[0] += p[0]; lo[1] += p[1]; lo[2] += p[2]; lo[3] += p[3];
                    hi[0] += q[0]; hi[1] += q[1]; hi[2] += q[2]; hi[3] += q[3];
                }
                const int m = ln & 15;
                if (m >= M) continue;
                const int d = tail.d, half = d >> 1, i0 = s16 * 16 + (ln >> 4) * 4;
                if constexpr (TAIL == 2) {  // pairs i0 .. i0+3, wherever their elements lie
#pragma unroll
                    for (int e = 0; e < 4; ++e) qkv_tail_pair(tail, bias, m, seg, i0 + e, round_to_bf16(lo[e]), round_to_bf16(hi[e]));
                    continue;
                }
                int kind, head;  // 0 query, 1 key, 2 value
                qkv_tail_segment(tail, seg, kind, head);
                if (kind != 0 && !tail.write_cache) continue;
                const int pos = tail.token_pos[m];
                float a[4], b[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    a[e] = round_to_bf16(lo[e]);
                    b[e] = round_to_bf16(hi[e]);
                    if (bias) {
                        a[e] = round_to_bf16(a[e] + bias[seg * d + i0 + e]);
                        b[e] = round_to_bf16(b[e] + bias[seg * d + half + i0 + e]);
                    }
                }
                if (tail.rot.inv_freq && kind != 2) {
                    const float* freq = qkv_tail_freq(tail, m);
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const float ang = (float)pos * freq[i0 + e];
                        const float c = cosf(ang) * tail.rot.cs_scale, sn = sinf(ang) * tail.rot.cs_scale;
                        const float x0 = a[e], x1 = b[e];
                        a[e] = x0 * c - x1 * sn;
                        b[e] = x1 * c + x0 * sn;
                    }
                }
                uint2 pa4, pb4;
                pa4.x = (uint32_t)f32_to_bf16_bits(a[0]) | ((uint32_t)f32_to_bf16_bits(a[1]) << 16);
                pa4.y = (uint32_t)f32_to_bf16_bits(a[2]) | ((uint32_t)f32_to_bf16_bits(a[3]) << 16);
                pb4.x = (uint32_t)f32_to_bf16_bits(b[0]) | ((uint32_t)f32_to_bf16_bits(b[1]) << 16);
                pb4.y = (uint32_t)f32_to_bf16_bits(b[2]) | ((uint32_t)f32_to_bf16_bits(b[3]) << 16);
                if (kind == 0) {
                    bf16_t* dst = tail.q_out + ((long)m * tail.nh + head) * d + i0;
                    *reinterpret_cast<uint2*>(dst) = pa4;
                    *reinterpret_cast<uint2*>(dst + half) = pb4;
                    continue;
                }
                const long page = tail.block_table[(long)tail.token_seq[m] * tail.bt_stride + pos / PTA_PAGE];
                const int in_page = pos % PTA_PAGE;
                if (kind == 1) {
                    bf16_t* dst = tail.k_pool + ((page * tail.nkv + head) * PTA_PAGE + in_page) * (long)d + i0;
                    *reinterpret_cast<uint2*>(dst) = pa4;
                    *reinterpret_cast<uint2*>(dst + half) = pb4;
                } else {
                    bf16_t* dst = tail.v_pool + ((page * tail.nkv + head) * (long)d + i0) * PTA_PAGE + in_page;
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        dst[(long)e * PTA_PAGE] = f32_to_bf16_bits(a[e]);
                        dst[(long)(half + e) * PTA_PAGE] = f32_to_bf16_bits(b[e]);
                    }
                }
            }
            return;
        }
    }
    // item (rt, mt, ln): outputs of row m = mt*16 + ln%16, columns n0 + rt*16 + (ln/16)*4 + 0..3
    for (int item = threadIdx.x; item < RT * MT * 64; item += blockDim.x) {
        const int ln = item & 63, mt = (item >> 6) % MT, rt = (item >> 6) / MT;
        f32x4_t sum = part[(rt * MT + mt) * 64 + ln];
        for (int w = 1; w < S; ++w) {
            const f32x4_t p = part[((w * RT + rt) * MT + mt) * 64 + ln];
            sum[0] += p[0]; sum[1] += p[1]; sum[2] += p[2]; sum[3] += p[3];
        }
        const int m = mt * 16 + (ln & 15);
        if (m >= M) continue;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int n = n0 + rt * 16 + (ln >> 4) * 4 + i;
            if (n < n1) {
                float v = OutIo<OutT>::round(sum[i]);
                if (bias) v = OutIo<OutT>::round(v + bias[n]);
                if (act == PTA_ACT_GELU) v = gelu_erf(v);  // other activations run as a pass of their own
                const long o = (long)m * N + n;
                if (add1) v += bf16_bits_to_f32(add1[o]);
                if (add2) v += bf16_bits_to_f32(add2[o]);
                OutIo<OutT>::st(y + o, v);
            }
        }
    }
}

// Waves per workgroup, i.e. how many ways K is split.  Measured on MI355X: long streams per wave beat
// many short ones, so K is split only when N alone gives too few waves.  It depends on N only, never
// on M or on the tile variant, so the order of summation is the same for every batch.
static int pick_split(int N) {
    const int groups = (N + 31) / 32;
    if (groups >= 512) return 1;
    if (groups >= 128) return 2;
    if (groups >= 32) return 4;
    return 8;
}

template <int MT, int RT, int U, typename OutT>
static void launch_cfg(SkinnyProblem a, SkinnyProblem b, int M, int K, int S, hipStream_t s) {
    const int rows = 16 * RT;
    if (S <= 0) S = pick_split(a.N + b.N);
    a.blocks = (a.N + rows - 1) / rows;
    b.blocks = (b.N + rows - 1) / rows;
    // A launch takes as long as the compute unit with the most workgroups: 714 workgroups on 256 units take
    // the time of 768 (measured: 44.7 us for 22,848 rows, 45.5 us for 24,576).  So a launch with more
    // workgroups than units gets a whole number of workgroups per unit, each with a little fewer rows.
    const int units = pta_compute_units(), natural = a.blocks + b.blocks;
    if (natural > units && natural % units != 0) {
        const int total = (natural + units - 1) / units * units;
        if (b.blocks == 0) {
            a.blocks = total;
        } else {
            const int first = (int)((long)total * a.N / (a.N + b.N));
            a.blocks = std::max(a.blocks, std::min(first, total - b.blocks));
            b.blocks = total - a.blocks;
        }
    }
    const dim3 grid(a.blocks + b.blocks), block(S * 64);
    const size_t lds = (size_t)S * RT * MT * 64 * sizeof(f32x4_t);
    static const int rot_env = getenv("PTA_SKINNY_ROT") ? atoi(getenv("PTA_SKINNY_ROT")) : -1;
    const int rot_stride = rot_env >= 0 ? rot_env : (K % 2048 == 0 ? 5 : 0);  // rows a multiple of 4 KB long
    hipLaunchKernelGGL((gemm_skinny_kernel<MT, RT, U, OutT>), grid, block, lds, s, a, b, M, K, rot_stride, QkvTail{});
}

template <typename OutT>
static int launch_skinny(SkinnyProblem a, SkinnyProblem b, int M, int K, int variant, int S, hipStream_t s) {
    // variant: row tiles per wave and steps per stage; 0: chosen here
    if (M <= 16) {
        if (variant == 0) variant = 2;
        if (variant == 1) launch_cfg<1, 1, 4, OutT>(a, b, M, K, S, s);
        else if (variant == 2) launch_cfg<1, 2, 2, OutT>(a, b, M, K, S, s);
        else if (variant == 3) launch_cfg<1, 4, 1, OutT>(a, b, M, K, S, s);
        else if (variant == 4) launch_cfg<1, 4, 2, OutT>(a, b, M, K, S, s);
        else launch_cfg<1, 2, 4, OutT>(a, b, M, K, S, s);
    } else if (M <= 32) {
        if (variant == 3 || variant == 4) launch_cfg<2, 4, 1, OutT>(a, b, M, K, S, s);
        else launch_cfg<2, 2, 1, OutT>(a, b, M, K, S, s);
    } else if (M <= 48) {
        launch_cfg<3, 2, 1, OutT>(a, b, M, K, S, s);
    } else {
        if (variant == 3 || variant == 4) launch_cfg<4, 4, 1, OutT>(a, b, M, K, S, s);
        else launch_cfg<4, 2, 1, OutT>(a, b, M, K, S, s);
    }
    return pta_check_launch("gemm_skinny_bf16");
}

static bool in_kernel(int act) { return act == PTA_ACT_NONE || act == PTA_ACT_GELU; }

static int check_skinny(const char* what, const void* y, const void* x, const void* W, int M, int N, int K, int act) {
    PTA_REQUIRE(M > 0 && N > 0 && K > 0, "%s: sizes must be positive (M=%d N=%d K=%d)", what, M, N, K);
    PTA_REQUIRE(M <= 64, "%s: at most 64 rows, got %d (use the library product)", what, M);
    PTA_REQUIRE(K % 8 == 0, "%s: K=%d must be a multiple of 8 (16-byte loads)", what, K);
    PTA_REQUIRE(y && x && W, "%s: null pointer", what);
    PTA_REQUIRE((long)M * K * 2 < (1L << 31), "%s: x is too large for 32-bit buffer offsets", what);
    PTA_REQUIRE(((uintptr_t)x % 16) == 0 && ((uintptr_t)W % 16) == 0, "%s: x and W must be 16-byte aligned", what);
    PTA_REQUIRE(pta_act_known(act), "%s: unknown activation %d", what, act);
    return 0;
}

extern "C" int pta_gemm_skinny_bf16(void* y, const void* x, const void* W, const float* bias, const void* add1,
                                    const void* add2, int M, int N, int K, int act, int out_f32, int variant,
                                    int waves, void* stream) {
    if (check_skinny("gemm_skinny_bf16", y, x, W, M, N, K, act)) return 1;
    PTA_REQUIRE(variant >= 0 && variant <= 5, "gemm_skinny_bf16: unknown variant %d", variant);
    PTA_REQUIRE(waves == 0 || (waves >= 1 && waves <= 8 && (waves & (waves - 1)) == 0),
                "gemm_skinny_bf16: waves per workgroup must be 0 (choose) or a power of two up to 8, got %d", waves);
    hipStream_t s = (hipStream_t)stream;
    const SkinnyProblem none{nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, 0, 0, 0};
    if (!in_kernel(act)) {
        // the kernel's epilogue knows the exact GELU only (every activation there would cost it its unrolled
        // loops): the product with its bias first, then activation and additions as a pass over y
        PTA_REQUIRE(!out_f32, "gemm_skinny_bf16: activation %d needs a bfloat16 result", act);
        const SkinnyProblem plain{y, (const bf16_t*)x, (const bf16_t*)W, bias, nullptr, nullptr, N, PTA_ACT_NONE, 0};
        if (launch_skinny<bf16_t>(plain, none, M, K, variant, waves, s)) return 1;
        return pta_epilogue(y, N, nullptr, add1, add2, M, N, act, PTA_BF16, stream);
    }
    const SkinnyProblem a{y, (const bf16_t*)x, (const bf16_t*)W, bias, (const bf16_t*)add1, (const bf16_t*)add2, N, act, 0};
    if (out_f32) return launch_skinny<float>(a, none, M, K, variant, waves, s);
    return launch_skinny<bf16_t>(a, none, M, K, variant, waves, s);
}

// The pair launch of a decode step whose first product is a fused query_key_value projection: its rows never
// reach memory as such; queries come out rotated in q_out [M, heads, d], keys (rotated) and values go to the
// cache pages of their sequences, as pta_qkv_rope_cache would have left them.  Up to 16 rows, head sizes that are
// multiples of 32.  The second product is y2 = act2(x2 . W2^T + bias2) as in the plain pair.
extern "C" int pta_gemm_skinny_pair_qkv_bf16(void* q_out, const void* x1, const void* W1, const float* bias1,
                                             const PtaRotation* rotation, const int* token_pos,
                                             const int* token_seq, const int* block_table, int bt_stride, void* k_pool,
                                             void* v_pool, int nh, int nkv, int d, int layout, int write_cache, void* y2,
                                             const void* x2, const void* W2, const float* bias2, int N2, int act2, int M,
                                             int K, void* stream) {
    PTA_REQUIRE(nh > 0 && nkv > 0 && d > 0 && nh % nkv == 0, "gemm_skinny_pair_qkv_bf16: heads %d, kv heads %d, head size %d", nh, nkv, d);
    const int N1 = (nh + 2 * nkv) * d;
    if (check_skinny("gemm_skinny_pair_qkv_bf16", q_out, x1, W1, M, N1, K, PTA_ACT_NONE)) return 1;
    if (check_skinny("gemm_skinny_pair_qkv_bf16", y2, x2, W2, M, N2, K, act2)) return 1;
    PTA_REQUIRE(M <= 16, "gemm_skinny_pair_qkv_bf16: at most 16 rows, got %d", M);
    PTA_REQUIRE(d % 32 == 0 && d <= 256, "gemm_skinny_pair_qkv_bf16: head size %d must be a multiple of 32 up to 256", d);
    PTA_REQUIRE(layout >= 0 && layout <= 2, "gemm_skinny_pair_qkv_bf16: unknown layout %d", layout);
    PTA_REQUIRE(layout != PTA_QKV_TAIL || nkv == 1, "gemm_skinny_pair_qkv_bf16: the tail layout has one kv head, got %d", nkv);
    PTA_REQUIRE(layout != PTA_QKV_INTERLEAVED || nkv == nh, "gemm_skinny_pair_qkv_bf16: the interleaved layout needs kv heads == heads");
    PTA_REQUIRE(token_pos, "gemm_skinny_pair_qkv_bf16: null token positions");
    const PtaRotation rot = pta_rotation_of(rotation);
    if (pta_check_rotation("gemm_skinny_pair_qkv_bf16", rot, d, token_seq)) return 1;
    PTA_REQUIRE(!write_cache || (k_pool && v_pool && block_table && token_seq), "gemm_skinny_pair_qkv_bf16: null cache pointer");
    PTA_REQUIRE((((uintptr_t)q_out | (uintptr_t)k_pool) % 8) == 0, "gemm_skinny_pair_qkv_bf16: outputs must be 8-byte aligned");
    SkinnyProblem a{nullptr, (const bf16_t*)x1, (const bf16_t*)W1, bias1, nullptr, nullptr, N1, PTA_ACT_NONE, 0};
    SkinnyProblem b{y2, (const bf16_t*)x2, (const bf16_t*)W2, bias2, nullptr, nullptr, N2, in_kernel(act2) ? act2 : 0, 0};
    const QkvTail tail{(bf16_t*)q_out, rot, token_pos, token_seq, block_table, bt_stride, (bf16_t*)k_pool,
                       (bf16_t*)v_pool, nh, nkv, d, layout, write_cache};
    // the first product's workgroups are bound to heads; the second one's fill the launch up to a whole number per unit
    a.blocks = (nh + 2 * nkv) * (d / 32);
    b.blocks = (N2 + 31) / 32;
    const int units = pta_compute_units(), natural = a.blocks + b.blocks;
    if (natural > units && natural % units != 0) b.blocks = (natural + units - 1) / units * units - a.blocks;
    const int S = pick_split(N1 + N2);
    static const int rot_env = getenv("PTA_SKINNY_ROT") ? atoi(getenv("PTA_SKINNY_ROT")) : -1;
    const int rot_stride = rot_env >= 0 ? rot_env : (K % 2048 == 0 ? 5 : 0);
    if (qkv_tail_plain_pairs(rot, d))
        hipLaunchKernelGGL((gemm_skinny_kernel<1, 2, 2, bf16_t, 1>), dim3(a.blocks + b.blocks), dim3(S * 64),
                           (size_t)S * 2 * 64 * sizeof(f32x4_t), (hipStream_t)stream, a, b, M, K, rot_stride, tail);
    else
        hipLaunchKernelGGL((gemm_skinny_kernel<1, 2, 2, bf16_t, 2>), dim3(a.blocks + b.blocks), dim3(S * 64),
                           (size_t)S * 2 * 64 * sizeof(f32x4_t), (hipStream_t)stream, a, b, M, K, rot_stride, tail);
    if (pta_check_launch("gemm_skinny_pair_qkv_bf16")) return 1;
    if (!in_kernel(act2)) return pta_epilogue(y2, N2, nullptr, nullptr, nullptr, M, N2, act2, PTA_BF16, stream);
    return 0;
}

// Two products of one launch: y1 = act1(x1 . W1^T + bias1), y2 = act2(x2 . W2^T + bias2), both [M, *] in
// bfloat16 with one K.  The waves per workgroup follow N1 + N2, so a product's bits differ from those of
// its own launch, but not with M or with what else is in the batch.
extern "C" int pta_gemm_skinny_pair_bf16(void* y1, const void* x1, const void* W1, const float* bias1, int N1, int act1,
                                         void* y2, const void* x2, const void* W2, const float* bias2, int N2, int act2,
                                         int M, int K, void* stream) {
    if (check_skinny("gemm_skinny_pair_bf16", y1, x1, W1, M, N1, K, act1)) return 1;
    if (check_skinny("gemm_skinny_pair_bf16", y2, x2, W2, M, N2, K, act2)) return 1;
    const SkinnyProblem a{y1, (const bf16_t*)x1, (const bf16_t*)W1, bias1, nullptr, nullptr, N1, in_kernel(act1) ? act1 : 0, 0};
    const SkinnyProblem b{y2, (const bf16_t*)x2, (const bf16_t*)W2, bias2, nullptr, nullptr, N2, in_kernel(act2) ? act2 : 0, 0};
    if (launch_skinny<bf16_t>(a, b, M, K, 0, 0, (hipStream_t)stream)) return 1;
    if (!in_kernel(act1) && pta_epilogue(y1, N1, nullptr, nullptr, nullptr, M, N1, act1, PTA_BF16, stream)) return 1;
    if (!in_kernel(act2) && pta_epilogue(y2, N2, nullptr, nullptr, nullptr, M, N2, act2, PTA_BF16, stream)) return 1;
    return 0;
}
