// y[M,N] = act(x[M,K] . W[N,K]^T + bias) + add1 + add2 for a decode batch of up to 128 rows,
// bfloat16 in, 32-bit accumulation on the matrix cores.
//
// With more than 16 rows the activations are no longer negligible beside the weights: a wave that
// fetched its own x fragments would pull as many bytes of x out of L2 as of W out of HBM.  Here a
// workgroup of four waves owns 64*RT rows of W (16*RT each) and a range of K, and shares x: the four
// waves copy the stage's [M, KS] slice of x into LDS together (through registers, one stage ahead,
// two LDS buffers), and every wave reads its B fragments from there.  W rows go straight from global
// memory into the A operand registers, one stage ahead of the matrix cores, as in the kernel for
// few rows.  K is split over gridDim.y workgroups when N alone gives too few of them to occupy the
// chip; each writes its 32-bit partial tile to `part`, and a second small kernel adds the partials
// in the order of the ranges and applies bias, activation and additions; with reduce = 0 the partials
// are the result, and the kernel that reads them next adds them in the same order.  The split is chosen from N
// and K alone, so the order of summation does not depend on the batch.
//
// Chunks of x past the workgroup's K range, or rows past M, are read through a buffer descriptor at
// an offset outside its bounds and arrive as zeros; W addresses are clamped into the range instead, so
// a stage past the end multiplies weights that are already in cache by zeros.
#include "common.h"
#include "pta_kernels.h"
#include "qkv_tail.h"

#include <stdlib.h>

#include <array>
#include <map>
#include <mutex>
#include <utility>

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef int i32x4_t __attribute__((ext_vector_type(4)));

union Frag8 {
    uint4 u;
    bf16x8_t v;
    i32x4_t i;
};

#define SK_THREADS 256
#define SK_CHUNK_ROWS 128  // eight tiles of sixteen rows of x: what a workgroup holds
#define SK_MAX_ROWS 256

// One product of a launch.  A launch may carry two that share M (a block's two output projections, left
// as partial sums): the workgroups of the second follow those of the first in a one-dimensional grid.
struct SplitkProblem {
    void* y;
    float* part;
    const bf16_t* x;
    const bf16_t* W;
    const float* bias;
    const bf16_t* add1;
    const bf16_t* add2;
    int N, K, act, out_f32;
    int blocks_per_part;  // 64-element blocks of K per range
    int tiles;            // workgroups along N
    int parts;            // ranges of K
    int direct;           // one range and the epilogue in this kernel
};

template <int MT, int RT, int U, int D, bool ROT>
__global__ __launch_bounds__(SK_THREADS) void gemm_splitk_kernel(SplitkProblem pa, SplitkProblem pb, int M, int chunks,
                                                                 int chunk_rows, int rot_stride) {
    constexpr int KS = U * 64;                       // elements of K per stage
    constexpr int MP = MT * 16;                      // rows of x, padded to whole tiles
    constexpr int LDW = KS + 8;                      // LDS row stride: 16 bytes of padding keep 16-byte reads off each other's banks
    constexpr int PIECES = MP * (KS / 8) / SK_THREADS;  // 16-byte pieces of the x slice per thread
    constexpr int STEPS = U * 2;                     // 32-element matrix-core steps per stage
    static_assert(MP * (KS / 8) % SK_THREADS == 0, "the x slice must divide over the threads");
    static_assert(D % 2 == 0, "stages alternate between two LDS buffers");
    extern __shared__ __attribute__((aligned(16))) bf16_t xs[];  // [2][MP][LDW]

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r = lane & 15, g = lane >> 4;
    // More rows than a workgroup holds are cut into `chunks` chunks of `chunk_rows`; the workgroups that take the
    // same rows of W for the chunks sit a multiple of eight apart in the grid, so that they start together on one
    // die and all but the first find W in its cache.
    const int first_blocks = pa.tiles * pa.parts;
    int block = (int)blockIdx.x, chunk = 0;
    if (chunks > 1) {
        const int per_chunk = (int)gridDim.x / chunks, whole = per_chunk / 8 * 8, rest = per_chunk - whole;
        if (block < whole * chunks) {
            chunk = (block >> 3) % chunks;
            block = block / (8 * chunks) * 8 + (block & 7);
        } else {
            const int t = block - whole * chunks;
            chunk = t / rest;
            block = whole + t % rest;
        }
    }
    const int m0 = chunk * chunk_rows, m_end = min(M, m0 + chunk_rows);
    const bool second = block >= first_blocks;
    void* __restrict__ y = second ? pb.y : pa.y;
    float* __restrict__ part = second ? pb.part : pa.part;
    const bf16_t* __restrict__ x = second ? pb.x : pa.x;
    const bf16_t* __restrict__ W = second ? pb.W : pa.W;
    const float* __restrict__ bias = second ? pb.bias : pa.bias;
    const bf16_t* __restrict__ add1 = second ? pb.add1 : pa.add1;
    const bf16_t* __restrict__ add2 = second ? pb.add2 : pa.add2;
    const int N = second ? pb.N : pa.N, K = second ? pb.K : pa.K, act = second ? pb.act : pa.act;
    const int out_f32 = second ? pb.out_f32 : pa.out_f32, direct = second ? pb.direct : pa.direct;
    const int blocks_per_part = second ? pb.blocks_per_part : pa.blocks_per_part;
    const int tiles = second ? pb.tiles : pa.tiles;
    const int idx = block - (second ? first_blocks : 0);
    const int tile = idx % tiles, range = idx / tiles;  // neighbours share a range of K: its x slice stays in L2
    const int n_base = tile * (64 * RT) + wave * (16 * RT);
    const int nkb = (K + 63) >> 6;
    const int kb0 = range * blocks_per_part, kb1 = min(kb0 + blocks_per_part, nkb);
    const int k_begin = kb0 * 64, k_end = min(kb1 * 64, K);
    const int nstages = (kb1 - kb0 + U - 1) / U;

    const bf16_t* wrow[RT];
#pragma unroll
    for (int t = 0; t < RT; ++t) wrow[t] = W + (long)min(n_base + t * 16 + r, N - 1) * K;
    __amdgpu_buffer_rsrc_t xres = __builtin_amdgcn_make_buffer_rsrc((void*)x, 0, M * K * 2, 0x00020000);

    f32x4_t acc[RT][MT];
#pragma unroll
    for (int t = 0; t < RT; ++t)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[t][mt] = f32x4_t{0.f, 0.f, 0.f, 0.f};

    // Where a row of W is a power of two long, workgroups that walk the same range of K in step ask the same few
    // memory channels at the same time (N = 4,096, K = 16,384: a third slower than K = 16,448).  So each walks its
    // range from a starting stage of its own and wraps round; stages past the last read nothing.  A feature's
    // order of summation follows from N, K and the launch alone.
    // (ROT is a compile-time choice: the wrap costs the other shapes 5 % of this kernel at 17 to 32 rows.)
    const int rot = ROT && nstages > 0 ? (int)(((long)tile * rot_stride) % nstages) : 0;
    auto stage_k = [&](int stage) {
        if (!ROT) return k_begin + stage * KS;
        if (stage >= nstages) return k_end;
        int at = stage + rot;
        at -= at >= nstages ? nstages : 0;
        return k_begin + at * KS;
    };
    auto load_x = [&](int stage, i32x4_t(&xr)[PIECES]) {
        const int k_stage = stage_k(stage);
#pragma unroll
        for (int j = 0; j < PIECES; ++j) {
            const int q = tid + j * SK_THREADS, row = m0 + q / (KS / 8), k = k_stage + (q % (KS / 8)) * 8;
            const int off = (k < k_end && row < m_end) ? (row * K + k) * 2 : 0x7ffffff0;
            xr[j] = __builtin_amdgcn_raw_buffer_load_b128(xres, off, 0, 0);
        }
    };
    auto store_x = [&](int buf, const i32x4_t(&xr)[PIECES]) {
#pragma unroll
        for (int j = 0; j < PIECES; ++j) {
            const int q = tid + j * SK_THREADS, row = q / (KS / 8), c8 = q % (KS / 8);
            *reinterpret_cast<i32x4_t*>(&xs[(buf * MP + row) * LDW + c8 * 8]) = xr[j];
        }
    };
    auto load_w = [&](int stage, Frag8(&wr)[STEPS][RT]) {
        const int k_stage = stage_k(stage) + g * 8;
#pragma unroll
        for (int j = 0; j < STEPS; ++j) {
            const int kc = min(k_stage + j * 32, k_end - 8);
#pragma unroll
            for (int t = 0; t < RT; ++t) wr[j][t].u = *reinterpret_cast<const uint4*>(wrow[t] + kc);
        }
    };
    auto compute = [&](int buf, const Frag8(&wr)[STEPS][RT]) {
#pragma unroll
        for (int j = 0; j < STEPS; ++j) {
            bf16x8_t b[MT];
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
                b[mt] = *reinterpret_cast<const bf16x8_t*>(&xs[(buf * MP + mt * 16 + r) * LDW + j * 32 + g * 8]);
#pragma unroll
            for (int t = 0; t < RT; ++t)
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
                    acc[t][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wr[j][t].v, b[mt], acc[t][mt], 0, 0, 0);
        }
    };

    // D stages of loads are in flight per wave: stage s lives in register set s % D.  x loads are issued
    // before the W loads of their stage, so that waiting for the next stage's x leaves younger loads in
    // flight; the scheduling barriers keep the compiler from sinking loads down to their use.
    i32x4_t xr[D][PIECES];
    Frag8 w[D][STEPS][RT];
#pragma unroll
    for (int d = 0; d < D; ++d) {
        load_x(d, xr[d]);
        load_w(d, w[d]);
    }
    __builtin_amdgcn_sched_barrier(0);
    store_x(0, xr[0]);
    __syncthreads();
    for (int s = 0; s < nstages; s += D) {
#pragma unroll
        for (int d = 0; d < D; ++d) {  // stage s + d: LDS buffer d % 2 (D is even)
            compute(d % 2, w[d]);
            __builtin_amdgcn_sched_barrier(0);
            load_x(s + d + D, xr[d]);
            load_w(s + d + D, w[d]);
            __builtin_amdgcn_sched_barrier(0);
            store_x((d + 1) % 2, xr[(d + 1) % D]);
            __syncthreads();
        }
    }

    // lane: row m = mt*16 + r of x, columns n_base + t*16 + g*4 + 0..3
#pragma unroll
    for (int t = 0; t < RT; ++t)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const int m = m0 + mt * 16 + r, n = n_base + t * 16 + g * 4;
            if (m >= m_end || n >= N) continue;
            const long o = (long)m * N + n;
            if (!direct) {
                const long at = (long)range * M * N + o;
                float* dst = part + at;
                if (n + 3 < N && (at & 3) == 0) *reinterpret_cast<f32x4_t*>(dst) = acc[t][mt];
                else
                    for (int i = 0; i < 4 && n + i < N; ++i) dst[i] = acc[t][mt][i];
                continue;
            }
            for (int i = 0; i < 4 && n + i < N; ++i) {
                float v = acc[t][mt][i];
                if (!out_f32) v = round_to_bf16(v);
                if (bias) { v += bias[n + i]; if (!out_f32) v = round_to_bf16(v); }
                if (act == PTA_ACT_GELU) v = gelu_erf(v);  // other activations: see pta_gemm_splitk_bf16
                if (add1) v += bf16_bits_to_f32(add1[o + i]);
                if (add2) v += bf16_bits_to_f32(add2[o + i]);
                if (out_f32) ((float*)y)[o + i] = v;
                else ((bf16_t*)y)[o + i] = f32_to_bf16_bits(v);
            }
        }
}

// y = act(sum over the parts + bias) + add1 + add2; parts are added in the order of their K ranges
__global__ __launch_bounds__(256) void gemm_splitk_reduce_kernel(void* __restrict__ y, const float* __restrict__ part,
                                                                 const float* __restrict__ bias,
                                                                 const bf16_t* __restrict__ add1,
                                                                 const bf16_t* __restrict__ add2, long MN, int N,
                                                                 int P, int act, int out_f32) {
    const long o = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (o >= MN) return;
    float v = part[o];
    for (int p = 1; p < P; ++p) v += part[(long)p * MN + o];
    const int n = (int)(o % N);
    if (!out_f32) v = round_to_bf16(v);
    if (bias) { v += bias[n]; if (!out_f32) v = round_to_bf16(v); }
    if (act) v = apply_act(v, act);
    if (add1) v += bf16_bits_to_f32(add1[o]);
    if (add2) v += bf16_bits_to_f32(add2[o]);
    if (out_f32) ((float*)y)[o] = v;
    else ((bf16_t*)y)[o] = f32_to_bf16_bits(v);
}

// the same for the two products of a pair launch, bfloat16 out, no additions
__global__ __launch_bounds__(256) void gemm_splitk_reduce2_kernel(bf16_t* __restrict__ y1, const float* __restrict__ part1,
                                                                  const float* __restrict__ bias1, long MN1, int N1, int P1,
                                                                  int act1, bf16_t* __restrict__ y2,
                                                                  const float* __restrict__ part2,
                                                                  const float* __restrict__ bias2, long MN2, int N2, int P2,
                                                                  int act2) {
    long o = (long)blockIdx.x * blockDim.x + threadIdx.x;
    const bool second = o >= MN1;
    if (second) o -= MN1;
    const long MN = second ? MN2 : MN1;
    if (o >= MN) return;
    const float* part = second ? part2 : part1;
    const float* bias = second ? bias2 : bias1;
    const int N = second ? N2 : N1, P = second ? P2 : P1, act = second ? act2 : act1;
    float v = part[o];
    for (int p = 1; p < P; ++p) v += part[(long)p * MN + o];
    v = round_to_bf16(v);
    if (bias) v = round_to_bf16(v + bias[(int)(o % N)]);
    if (act) v = apply_act(v, act);
    (second ? y2 : y1)[o] = f32_to_bf16_bits(v);
}

// The reduction on its own, for partial sums that something else made (the vendor library's batched product
// over ranges of K): y[M, N] = act(sum over part[P, M, N] in order + bias) + add1 + add2.
extern "C" int pta_gemm_reduce_parts(void* y, const float* part, const float* bias, const void* add1, const void* add2,
                                     int M, int N, int P, int act, int out_f32, void* stream) {
    PTA_REQUIRE(M > 0 && N > 0 && P > 0, "gemm_reduce_parts: sizes must be positive (M=%d N=%d P=%d)", M, N, P);
    PTA_REQUIRE(y && part, "gemm_reduce_parts: null pointer");
    PTA_REQUIRE(pta_act_known(act), "gemm_reduce_parts: unknown activation %d", act);
    const long MN = (long)M * N;
    PTA_REQUIRE((MN + 255) / 256 < (1L << 31), "gemm_reduce_parts: too many elements for one launch");
    hipLaunchKernelGGL(gemm_splitk_reduce_kernel, dim3((unsigned)((MN + 255) / 256)), dim3(256), 0, (hipStream_t)stream, y,
                       part, bias, (const bf16_t*)add1, (const bf16_t*)add2, MN, N, P, act, out_f32);
    return pta_check_launch("gemm_reduce_parts");
}

// The reduction of a pair launch whose first product is a fused query_key_value projection: a thread adds the
// partial sums of one pair of a segment's elements (the two that are rotated together, or two that pass;
// qkv_tail_pair_elements) and takes it to its end (qkv_tail.h); the second product as in gemm_splitk_reduce2_kernel.
__global__ __launch_bounds__(256) void gemm_splitk_reduce2_qkv_kernel(QkvTail tail, const float* __restrict__ part1,
                                                                      const float* __restrict__ bias1, long MN1, int N1,
                                                                      int P1, bf16_t* __restrict__ y2,
                                                                      const float* __restrict__ part2,
                                                                      const float* __restrict__ bias2, long MN2, int N2,
                                                                      int P2, int act2) {
    long o = (long)blockIdx.x * blockDim.x + threadIdx.x;
    const long pairs = MN1 >> 1;
    if (o < pairs) {
        const int half = tail.d >> 1, per_row = N1 >> 1;
        const int m = (int)(o / per_row), p = (int)(o % per_row), seg = p / half, i = p % half;
        int ea, eb;
        bool rotated;
        qkv_tail_pair_elements(tail.rot, tail.d, i, ea, eb, rotated);
        const long lo = (long)m * N1 + (long)seg * tail.d + ea, hi = (long)m * N1 + (long)seg * tail.d + eb;
        float a = part1[lo], b = part1[hi];
        for (int q = 1; q < P1; ++q) { a += part1[(long)q * MN1 + lo]; b += part1[(long)q * MN1 + hi]; }
        qkv_tail_pair(tail, bias1, m, seg, i, round_to_bf16(a), round_to_bf16(b));
        return;
    }
    o -= pairs;
    if (o >= MN2) return;
    float v = part2[o];
    for (int q = 1; q < P2; ++q) v += part2[(long)q * MN2 + o];
    v = round_to_bf16(v);
    if (bias2) v = round_to_bf16(v + bias2[(int)(o % N2)]);
    if (act2) v = apply_act(v, act2);
    y2[o] = f32_to_bf16_bits(v);
}

static int pick_rt(int N) { return N >= 16384 ? 2 : 1; }

// ranges that are not empty when K is cut into `parts` ranges of whole 64-element blocks
static int effective_parts(int K, int parts) {
    const int nkb = (K + 63) / 64, per = (nkb + parts - 1) / parts;
    return (nkb + per - 1) / per;
}

// Ranges of K (workgroups along gridDim.y).  Measured at K = 4,096 to 32,768 and N = 4,096 to 32,768: a workgroup does best
// with a range of about 2,304 elements (some 290 KB of weights for its 64 rows), and a launch with at least
// some 512 workgroups; no range is shorter than 512 elements, and there are at most 16.
#define SK_RANGE 2304
static int splitk_target() {
    static const int target = getenv("PTA_SPLITK_WGS") ? atoi(getenv("PTA_SPLITK_WGS")) : 512;
    return target;
}
static int clamp_parts(int P, int K) { return max(1, min(min(P, 16), max(1, K / 512))); }

// with many row tiles the ranges may be longer: fewer partial sums for the same number of workgroups
static int range_for(int groups) { return SK_RANGE * max(1, groups / 64); }

// Among the counts near that rule's, the one with the least (rounds of workgroups on the chip's compute units)
// x (a workgroup's fixed cost + the length of its range).  Measured at 32 to 128 rows: a launch just over a whole
// number of rounds pays for the last one in full (N = 9,216 and K = 8,192, 144 row tiles: 4 ranges, 2.25 rounds, 81
// us; 3 ranges, 1.69 rounds, 65 us; N = 4,672 and K = 4,544, 73 row tiles: 8 ranges 31.6 us, 7 ranges 27.6 us), and the fixed
// cost of a workgroup (start, first loads, its tile of partial sums) is that of some 1,300 elements of K.
#define SK_WG_FIXED 1300
static int pick_parts(int N, int K, int rt) {
    const int groups = (N + 64 * rt - 1) / (64 * rt), range = range_for(groups);
    const int p0 = clamp_parts(max((splitk_target() + groups - 1) / groups, (K + range / 2) / range), K);
    const long units = max(1, pta_compute_units());
    auto cost = [&](int p) { return (((long)groups * p + units - 1) / units) * (SK_WG_FIXED + K / p); };
    static const bool balance = !getenv("PTA_SPLITK_BALANCE") || atoi(getenv("PTA_SPLITK_BALANCE")) != 0;
    int best = p0;
    for (int p = max(1, p0 - 2); balance && p <= p0 + 2; ++p) {
        if (clamp_parts(p, K) != p || effective_parts(K, p) != p || (long)groups * p < 384) continue;
        if (cost(p) < cost(best)) best = p;
    }
    return best;
}

extern "C" int pta_gemm_splitk_parts(int N, int K, int parts, int rt) {
    if (N <= 0 || K <= 0) return 0;
    if (rt <= 0) rt = pick_rt(N);
    return effective_parts(K, parts > 0 ? parts : pick_parts(N, K, rt));
}

static SplitkProblem make_problem(void* y, float* part, const void* x, const void* W, const float* bias,
                                  const void* add1, const void* add2, int N, int K, int act, int out_f32, int rt,
                                  int parts, int reduce) {
    SplitkProblem p{};
    p.y = y; p.part = part; p.x = (const bf16_t*)x; p.W = (const bf16_t*)W; p.bias = bias;
    p.add1 = (const bf16_t*)add1; p.add2 = (const bf16_t*)add2;
    p.N = N; p.K = K; p.act = act; p.out_f32 = out_f32;
    const int nkb = (K + 63) / 64;
    p.blocks_per_part = (nkb + parts - 1) / parts;
    p.parts = (nkb + p.blocks_per_part - 1) / p.blocks_per_part;  // ranges that are not empty
    p.tiles = (N + 64 * rt - 1) / (64 * rt);
    p.direct = reduce && p.parts == 1;
    return p;
}

template <int MT, int RT, int U, int D>
static int launch_cfg(const SplitkProblem& a, const SplitkProblem& b, int M, int reduce, hipStream_t s) {
    const size_t lds = (size_t)2 * MT * 16 * (U * 64 + 8) * sizeof(bf16_t);
    // rows of W a multiple of 4 KB long are the ones that crowd memory channels: there every workgroup starts at a
    // stage of its own (PTA_SPLITK_ROT: stages between neighbours, 0 switches it off)
    static const int rot_env = getenv("PTA_SPLITK_ROT") ? atoi(getenv("PTA_SPLITK_ROT")) : -1;
    const int rot_stride = rot_env >= 0 ? rot_env : 1;
    const bool rotate = rot_stride > 0 && (a.K % 2048 == 0 || (b.N > 0 && b.K % 2048 == 0));
    auto kern = rotate ? gemm_splitk_kernel<MT, RT, U, D, true> : gemm_splitk_kernel<MT, RT, U, D, false>;
    if (lds > 64 * 1024) {
        static bool raised[2] = {false, false};  // per instantiation
        if (!raised[rotate]) {
            if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
                return pta_fail("gemm_splitk_bf16: cannot have %zu bytes of LDS", lds);
            raised[rotate] = true;
        }
    }
    // rows beyond the MT tiles of a workgroup go to further chunks of workgroups, all of the same size
    const int chunks = (M + MT * 16 - 1) / (MT * 16), chunk_rows = ((M + chunks - 1) / chunks + 15) / 16 * 16;
    const dim3 grid((a.tiles * a.parts + b.tiles * b.parts) * chunks);
    hipLaunchKernelGGL(kern, grid, dim3(SK_THREADS), lds, s, a, b, M, chunks, chunk_rows, rot_stride);
    if (reduce && a.parts > 1) {
        const long MN = (long)M * a.N;
        hipLaunchKernelGGL(gemm_splitk_reduce_kernel, dim3((unsigned)((MN + 255) / 256)), dim3(256), 0, s, a.y, a.part,
                           a.bias, a.add1, a.add2, MN, a.N, a.parts, a.act, a.out_f32);
    }
    return pta_check_launch("gemm_splitk_bf16");
}

// sixteen-row tiles of x that a workgroup holds: all rows up to SK_CHUNK_ROWS, else an even share of them
static int tiles_per_chunk(int M) {
    const int chunks = (M + SK_CHUNK_ROWS - 1) / SK_CHUNK_ROWS;
    return ((M + chunks - 1) / chunks + 15) / 16;
}

template <int RT, int U, int D>
static int launch_rows(int MT, const SplitkProblem& a, const SplitkProblem& b, int M, int reduce, hipStream_t s) {
    switch (MT) {
        case 1: return launch_cfg<1, RT, U, D>(a, b, M, reduce, s);
        case 2: return launch_cfg<2, RT, U, D>(a, b, M, reduce, s);
        case 3: return launch_cfg<3, RT, U, D>(a, b, M, reduce, s);
        case 4: return launch_cfg<4, RT, U, D>(a, b, M, reduce, s);
        default:
            // 65 to 128 rows: two stages in flight only (four would not fit the registers)
            if constexpr (D == 2) {
                if (MT <= 6) return launch_cfg<6, RT, U, D>(a, b, M, reduce, s);
                return launch_cfg<8, RT, U, D>(a, b, M, reduce, s);
            } else {
                return pta_fail("gemm_splitk_bf16: more than 64 rows run with two stages in flight, not %d", D);
            }
    }
}

static int check_splitk(const char* what, const void* x, const void* W, int M, int N, int K) {
    PTA_REQUIRE(M > 0 && N > 0 && K > 0, "%s: sizes must be positive (M=%d N=%d K=%d)", what, M, N, K);
    PTA_REQUIRE(M <= SK_MAX_ROWS, "%s: at most %d rows, got %d (use the library product)", what, SK_MAX_ROWS, M);
    PTA_REQUIRE(K % 8 == 0 && K >= 8, "%s: K=%d must be a multiple of 8 (16-byte loads)", what, K);
    PTA_REQUIRE(x && W, "%s: null pointer", what);
    PTA_REQUIRE((long)M * K * 2 < 0x7ffffff0L, "%s: x is too large for 32-bit buffer offsets", what);
    PTA_REQUIRE(((uintptr_t)x % 16) == 0 && ((uintptr_t)W % 16) == 0, "%s: x and W must be 16-byte aligned", what);
    return 0;
}

extern "C" int pta_gemm_splitk_bf16(void* y, float* part, const void* x, const void* W, const float* bias,
                                    const void* add1, const void* add2, int M, int N, int K, int act, int out_f32,
                                    int rt, int parts, int stage_blocks, int depth, int reduce, void* stream) {
    if (check_splitk("gemm_splitk_bf16", x, W, M, N, K)) return 1;
    PTA_REQUIRE(y || !reduce, "gemm_splitk_bf16: null pointer");
    PTA_REQUIRE(pta_act_known(act), "gemm_splitk_bf16: unknown activation %d", act);
    PTA_REQUIRE(rt == 0 || rt == 1 || rt == 2, "gemm_splitk_bf16: row tiles per wave must be 0 (choose), 1 or 2, got %d", rt);
    PTA_REQUIRE(stage_blocks == 0 || stage_blocks == 2,
                "gemm_splitk_bf16: 64-element blocks per stage must be 0 (choose) or 2, got %d", stage_blocks);
    PTA_REQUIRE(depth == 0 || depth == 2 || depth == 4, "gemm_splitk_bf16: stages in flight must be 0 (choose), 2 or 4, got %d", depth);
    PTA_REQUIRE(parts >= 0 && parts <= 64, "gemm_splitk_bf16: parts must be 0 (choose) or 1..64, got %d", parts);
    if (rt == 0) rt = pick_rt(N);
    if (parts == 0) parts = pick_parts(N, K, rt);
    if (depth == 0 || M > 64) depth = 2;  // measured: more stages in flight per wave do not pay, more workgroups do
    SplitkProblem a = make_problem(y, part, x, W, bias, add1, add2, N, K, act, out_f32, rt, parts, reduce);
    PTA_REQUIRE(a.direct || part, "gemm_splitk_bf16: %d ranges of K need the workspace for partial sums", a.parts);
    // One range of K ends in the matrix kernel itself, whose epilogue knows the exact GELU only (every activation
    // there would cost it its unrolled loops): another activation, and the additions after it, run as a pass over y.
    const bool after = a.direct && act != PTA_ACT_NONE && act != PTA_ACT_GELU;
    if (after) {
        PTA_REQUIRE(!out_f32, "gemm_splitk_bf16: activation %d needs a bfloat16 result", act);
        a.act = PTA_ACT_NONE;
        a.add1 = a.add2 = nullptr;
    }
    const SplitkProblem none{};
    hipStream_t s = (hipStream_t)stream;
    const int MT = tiles_per_chunk(M);
    int rc;
    if (rt == 1 && depth == 2) rc = launch_rows<1, 2, 2>(MT, a, none, M, reduce, s);
    else if (rt == 1) rc = launch_rows<1, 2, 4>(MT, a, none, M, reduce, s);
    else if (depth == 2) rc = launch_rows<2, 2, 2>(MT, a, none, M, reduce, s);
    else rc = launch_rows<2, 2, 4>(MT, a, none, M, reduce, s);
    if (rc || !after) return rc;
    return pta_epilogue(y, N, nullptr, add1, add2, M, N, act, PTA_BF16, stream);
}

// Ranges of K for the two products of a pair launch: each by its own length, and more of both if the launch
// would have too few workgroups.
// Counts that a caller has fixed for the pairs of one shape: no rule tells which neighbour of its choice is the
// fastest (N = 4,096 with K = 4,096 and 16,384 at 64 rows: 2 and 7 ranges by the rule; 4 and 8 make the
// decode step 7 % faster, 2 and 10 make it 3 % slower with as many workgroups), so the Python side times them once.
struct PairChoice { int p1, p2, rt; };
static std::map<std::array<int, 4>, PairChoice> pair_parts_fixed;
static std::mutex pair_parts_lock;

static bool parts_valid(int K, int p) { return p >= 1 && clamp_parts(p, K) == p && effective_parts(K, p) == p; }

// Fixes, for every later pair launch of this shape, the ranges of K of the two products and how many tiles of
// sixteen rows of W a wave holds in steps of more than 32 rows (rt 1 or 2: 64 or 128 rows of W a workgroup; the
// taller tile loads the activations half as often and has half as many workgroups).  p1 = p2 = 0 forgets the
// shape.  Returns 1 (no error text) for counts that the kernel does not take.  The ranges decide the order of
// summation; the tile height does not.
extern "C" int pta_gemm_splitk_pair_fix(int N1, int K1, int N2, int K2, int p1, int p2, int rt) {
    if (N1 <= 0 || K1 <= 0 || N2 <= 0 || K2 <= 0) return 1;
    std::lock_guard<std::mutex> hold(pair_parts_lock);
    const std::array<int, 4> key{N1, K1, N2, K2};
    if (p1 == 0 && p2 == 0) {
        pair_parts_fixed.erase(key);
        return 0;
    }
    if (!parts_valid(K1, p1) || !parts_valid(K2, p2) || (rt != 1 && rt != 2)) return 1;
    pair_parts_fixed[key] = {p1, p2, rt};
    return 0;
}

extern "C" int pta_gemm_splitk_pair_fix_parts(int N1, int K1, int N2, int K2, int p1, int p2) {
    return pta_gemm_splitk_pair_fix(N1, K1, N2, K2, p1, p2, 1);
}

// returns the row tiles per wave for steps of more than 32 rows
static int pick_pair_parts(int N1, int K1, int N2, int K2, int* p1, int* p2) {
    {
        std::lock_guard<std::mutex> hold(pair_parts_lock);
        const auto it = pair_parts_fixed.find({N1, K1, N2, K2});
        if (it != pair_parts_fixed.end()) {
            *p1 = it->second.p1;
            *p2 = it->second.p2;
            return it->second.rt;
        }
    }
    const int g1 = (N1 + 63) / 64, g2 = (N2 + 63) / 64;
    const int range = range_for(min(g1, g2));
    int a = clamp_parts((K1 + range / 2) / range, K1), b = clamp_parts((K2 + range / 2) / range, K2);
    const int total = g1 * a + g2 * b;
    if (total < splitk_target()) {
        const int more = (splitk_target() + total - 1) / total;
        a = clamp_parts(a * more, K1);
        b = clamp_parts(b * more, K2);
    }
    *p1 = effective_parts(K1, a);
    *p2 = effective_parts(K2, b);
    return 1;
}

// Steps of up to 128 rows may run with the activations stationary (gemm_stationary_bf16.hip), which cuts K into
// ranges of its own, by the class of the step's rows (up to 16, 32, 64, 128).  The rule: ranges of about 1,400
// elements, of the same length in both products, but no more of them than leave every wave at most the row tiles
// it can hold with one workgroup per compute unit (past that the launch needs a second round of workgroups).
// Measured against the staged kernel (us, staged -> stationary with the rule's ranges): K = 4,544 with N = 4,672
// + 18,176 at 8 / 32 / 64 / 128 rows 45.3 -> 40.5, 47.1 -> 43.1, 58.2 -> 46.5, 75.4 -> 56.0; K = 4,544 + 18,176
// with N = 4,544: 44.9 -> 41.6, 48.8 -> 44.9, 57.5 -> 48.0, 72.6 -> 55.6; K = 4,096 with N = 6,144 + 16,384: 42.3
// -> 38.4, 45.6 -> 40.1, 51.7 -> 45.1, 64.8 -> 55.1; K = 8,192 with N = 9,216 + 32,768: 141.8 -> 137.5, 158.5 ->
// 154.6, 178.9 -> 163.5, 188.7 -> 185.7.  Which count of ranges is fastest varies by a few percent around the
// rule's (and at 128 rows of the last shape three ranges in two rounds beat one by a tenth), so the Python side
// times the neighbours per class and fixes what wins, or the staged kernel where that wins.
#define STATIONARY_MAX_ROWS 128
#define STATIONARY_CLASSES 4
#define STATIONARY_RANGE 1400
static int stationary_class(int M) { return M <= 16 ? 0 : M <= 32 ? 1 : M <= 64 ? 2 : 3; }
struct StationaryChoice { int q1[STATIONARY_CLASSES], q2[STATIONARY_CLASSES]; };  // 0: the staged kernel
static std::map<std::array<int, 4>, StationaryChoice> pair_stationary_fixed;

// Without a fixed choice the launch is used from 33 rows on (classes 2 and 3): below, the staged kernel with timed
// ranges is as fast or faster at most shapes.
#define STATIONARY_RULE_FROM_CLASS 2
static void stationary_rule(int N1, int K1, int N2, int K2, int cls, int* q1, int* q2) {
    const int kmin = min(K1, K2), f1 = max(1, (K1 + kmin / 2) / kmin), f2 = max(1, (K2 + kmin / 2) / kmin);
    const long tiles = (long)((N1 + 15) / 16) * f1 + (long)((N2 + 15) / 16) * f2;
    const long room = (long)pta_compute_units() * 8 * (cls == 3 ? 2 : 3);  // waves x row tiles a wave holds
    int base = max(1, (kmin + STATIONARY_RANGE / 2) / STATIONARY_RANGE);
    base = max(1, (int)min((long)base, room / max(1L, tiles)));
    while (base > 1 && (base * f1 > 16 || base * f2 > 16)) --base;
    *q1 = effective_parts(K1, min(16, base * f1));
    *q2 = effective_parts(K2, min(16, base * f2));
}

// Fixes, for every later pair launch of this shape with rows of class cls (0: up to 16 rows, 1: 32, 2: 64, 3:
// 128), the ranges of K of the launch with stationary activations; q1 = q2 = 0: the staged kernel for the class;
// cls = -1 forgets the shape.  Returns 1 (no error text) for counts that the kernel does not take.
extern "C" int pta_gemm_splitk_pair_fix_stationary(int N1, int K1, int N2, int K2, int cls, int q1, int q2) {
    if (N1 <= 0 || K1 <= 0 || N2 <= 0 || K2 <= 0) return 1;
    std::lock_guard<std::mutex> hold(pair_parts_lock);
    const std::array<int, 4> key{N1, K1, N2, K2};
    if (cls == -1) {
        pair_stationary_fixed.erase(key);
        return 0;
    }
    if (cls < 0 || cls >= STATIONARY_CLASSES) return 1;
    const bool staged = q1 == 0 && q2 == 0;
    if (!staged && (q1 < 1 || q2 < 1 || q1 > 16 || q2 > 16 || effective_parts(K1, q1) != q1 || effective_parts(K2, q2) != q2))
        return 1;
    auto it = pair_stationary_fixed.find(key);
    if (it == pair_stationary_fixed.end()) {
        StationaryChoice c{};
        for (int i = STATIONARY_RULE_FROM_CLASS; i < STATIONARY_CLASSES; ++i) stationary_rule(N1, K1, N2, K2, i, &c.q1[i], &c.q2[i]);
        it = pair_stationary_fixed.emplace(key, c).first;
    }
    it->second.q1[cls] = q1;
    it->second.q2[cls] = q2;
    return 0;
}

// The ranges of a pair launch of M rows and its kind: 3 with stationary activations, else the tiles of sixteen
// rows of W per wave of the staged kernel (1 or 2).  M = 0 asks for the staged kernel's ranges.
static int pick_pair_parts_rows(int N1, int K1, int N2, int K2, int M, int* p1, int* p2) {
    if (M >= 1 && M <= STATIONARY_MAX_ROWS && K1 % 8 == 0 && K2 % 8 == 0) {
        const int cls = stationary_class(M);
        int q1, q2;
        bool fixed = false;
        {
            std::lock_guard<std::mutex> hold(pair_parts_lock);
            const auto it = pair_stationary_fixed.find({N1, K1, N2, K2});
            if (it != pair_stationary_fixed.end()) {
                q1 = it->second.q1[cls];
                q2 = it->second.q2[cls];
                fixed = true;
            }
        }
        if (!fixed) {
            q1 = q2 = 0;
            if (cls >= STATIONARY_RULE_FROM_CLASS) stationary_rule(N1, K1, N2, K2, cls, &q1, &q2);
        }
        if (q1 > 0 && q2 > 0) {
            *p1 = q1;
            *p2 = q2;
            return 3;
        }
    }
    const int rt = pick_pair_parts(N1, K1, N2, K2, p1, p2);
    return M > 32 ? rt : 1;
}

extern "C" int pta_gemm_splitk_pair_parts(int N1, int K1, int N2, int K2, int M, int* p1, int* p2) {
    if (N1 <= 0 || K1 <= 0 || N2 <= 0 || K2 <= 0 || M < 0) return pta_fail("gemm_splitk_pair_parts: sizes must be positive");
    pick_pair_parts_rows(N1, K1, N2, K2, M, p1, p2);
    return 0;
}

extern "C" int pta_gemm_stationary_rule(int N1, int K1, int N2, int K2, int cls, int* q1, int* q2) {
    if (N1 <= 0 || K1 <= 0 || N2 <= 0 || K2 <= 0 || cls < 0 || cls >= STATIONARY_CLASSES)
        return pta_fail("gemm_stationary_rule: sizes must be positive and the class of rows 0 to %d", STATIONARY_CLASSES - 1);
    stationary_rule(N1, K1, N2, K2, cls, q1, q2);
    return 0;
}

// Two products of one launch, both left as partial sums: part1 [parts1, M, N1] of x1 . W1^T and part2
// [parts2, M, N2] of x2 . W2^T, with the ranges pta_gemm_splitk_pair_parts gives for M rows.
extern "C" int pta_gemm_splitk_pair_bf16(float* part1, const void* x1, const void* W1, int N1, int K1, float* part2,
                                         const void* x2, const void* W2, int N2, int K2, int M, void* stream) {
    if (check_splitk("gemm_splitk_pair_bf16", x1, W1, M, N1, K1)) return 1;
    if (check_splitk("gemm_splitk_pair_bf16", x2, W2, M, N2, K2)) return 1;
    PTA_REQUIRE(part1 && part2, "gemm_splitk_pair_bf16: null workspace");
    int p1, p2;
    const int kind = pick_pair_parts_rows(N1, K1, N2, K2, M, &p1, &p2);
    if (kind == 3) return pta_gemm_stationary_pair_bf16(part1, x1, W1, N1, K1, p1, part2, x2, W2, N2, K2, p2, M, stream);
    const SplitkProblem a = make_problem(nullptr, part1, x1, W1, nullptr, nullptr, nullptr, N1, K1, 0, 0, kind, p1, 0);
    const SplitkProblem b = make_problem(nullptr, part2, x2, W2, nullptr, nullptr, nullptr, N2, K2, 0, 0, kind, p2, 0);
    if (kind == 2) return launch_rows<2, 2, 2>(tiles_per_chunk(M), a, b, M, 0, (hipStream_t)stream);
    return launch_rows<1, 2, 2>(tiles_per_chunk(M), a, b, M, 0, (hipStream_t)stream);
}

// The same pair run to the end: y1 = act1(x1 . W1^T + bias1), y2 = act2(x2 . W2^T + bias2) in bfloat16; the two
// products share the matrix launch and the launch that adds their partial sums.
extern "C" int pta_gemm_splitk_pair_reduced_bf16(void* y1, float* part1, const void* x1, const void* W1,
                                                 const float* bias1, int N1, int K1, int act1, void* y2, float* part2,
                                                 const void* x2, const void* W2, const float* bias2, int N2, int K2,
                                                 int act2, int M, void* stream) {
    PTA_REQUIRE(y1 && y2, "gemm_splitk_pair_reduced_bf16: null output");
    PTA_REQUIRE(pta_act_known(act1) && pta_act_known(act2),
                "gemm_splitk_pair_reduced_bf16: unknown activation");
    const int rc = pta_gemm_splitk_pair_bf16(part1, x1, W1, N1, K1, part2, x2, W2, N2, K2, M, stream);
    if (rc) return rc;
    const long MN1 = (long)M * N1, MN2 = (long)M * N2;
    int P1, P2;
    pick_pair_parts_rows(N1, K1, N2, K2, M, &P1, &P2);
    hipLaunchKernelGGL(gemm_splitk_reduce2_kernel, dim3((unsigned)((MN1 + MN2 + 255) / 256)), dim3(256), 0,
                       (hipStream_t)stream, (bf16_t*)y1, part1, bias1, MN1, N1, P1, act1, (bf16_t*)y2, part2, bias2, MN2, N2,
                       P2, act2);
    return pta_check_launch("gemm_splitk_pair_reduced_bf16");
}

// what the launches that take fused query_key_value rows to their end ask of their arguments
static int check_qkv_tail(const char* what, const void* q_out, const PtaRotation& rot,
                          const int* token_pos, const int* token_seq,
                          const int* block_table, const void* k_pool, const void* v_pool, int nh, int nkv, int d,
                          int layout, int write_cache) {
    PTA_REQUIRE(nh > 0 && nkv > 0 && d > 0 && nh % nkv == 0, "%s: heads %d, kv heads %d, head size %d", what, nh, nkv, d);
    if (pta_check_rotation(what, rot, d, token_seq)) return 1;
    PTA_REQUIRE(d % 2 == 0, "%s: head size %d must be even", what, d);
    PTA_REQUIRE(layout >= 0 && layout <= 2, "%s: unknown layout %d", what, layout);
    PTA_REQUIRE(layout != PTA_QKV_TAIL || nkv == 1, "%s: the tail layout has one kv head, got %d", what, nkv);
    PTA_REQUIRE(layout != PTA_QKV_INTERLEAVED || nkv == nh, "%s: the interleaved layout needs kv heads == heads", what);
    PTA_REQUIRE(q_out && token_pos, "%s: null pointer", what);
    PTA_REQUIRE(!write_cache || (k_pool && v_pool && block_table && token_seq), "%s: null cache pointer", what);
    return 0;
}

// The same pair with the first product a fused query_key_value projection taken to its end: queries rotated in
// q_out [M, heads, d], keys and values in the cache pages (as pta_qkv_rope_cache leaves them); even head sizes.
extern "C" int pta_gemm_splitk_pair_reduced_qkv_bf16(void* q_out, float* part1, const void* x1, const void* W1,
                                                     const float* bias1, int K1, const PtaRotation* rotation,
                                                     const int* token_pos, const int* token_seq, const int* block_table,
                                                     int bt_stride, void* k_pool, void* v_pool, int nh, int nkv, int d,
                                                     int layout, int write_cache, void* y2, float* part2, const void* x2,
                                                     const void* W2, const float* bias2, int N2, int K2, int act2, int M,
                                                     void* stream) {
    const PtaRotation rot = pta_rotation_of(rotation);
    if (check_qkv_tail("gemm_splitk_pair_reduced_qkv_bf16", q_out, rot, token_pos, token_seq, block_table, k_pool, v_pool, nh,
                       nkv, d, layout, write_cache))
        return 1;
    PTA_REQUIRE(y2, "gemm_splitk_pair_reduced_qkv_bf16: null pointer");
    PTA_REQUIRE(pta_act_known(act2), "gemm_splitk_pair_reduced_qkv_bf16: unknown activation %d", act2);
    const int N1 = (nh + 2 * nkv) * d;
    const int rc = pta_gemm_splitk_pair_bf16(part1, x1, W1, N1, K1, part2, x2, W2, N2, K2, M, stream);
    if (rc) return rc;
    const long MN1 = (long)M * N1, MN2 = (long)M * N2;
    int P1, P2;
    pick_pair_parts_rows(N1, K1, N2, K2, M, &P1, &P2);
    const QkvTail tail{(bf16_t*)q_out, rot, token_pos, token_seq, block_table, bt_stride, (bf16_t*)k_pool,
                       (bf16_t*)v_pool, nh, nkv, d, layout, write_cache};
    hipLaunchKernelGGL(gemm_splitk_reduce2_qkv_kernel, dim3((unsigned)((MN1 / 2 + MN2 + 255) / 256)), dim3(256), 0,
                       (hipStream_t)stream, tail, part1, bias1, MN1, N1, P1, (bf16_t*)y2, part2, bias2, MN2, N2, P2, act2);
    return pta_check_launch("gemm_splitk_pair_reduced_qkv_bf16");
}

// A fused query_key_value projection on its own (17 to 256 rows), taken to its end by the launch that adds its
// partial sums: part [pta_gemm_splitk_parts(N, K, 0, 0), M, N] is the workspace, N = (nh + 2 nkv) d.
extern "C" int pta_gemm_splitk_reduced_qkv_bf16(void* q_out, float* part, const void* x, const void* W,
                                                const float* bias, int K, const PtaRotation* rotation,
                                                const int* token_pos, const int* token_seq, const int* block_table,
                                                int bt_stride, void* k_pool, void* v_pool, int nh, int nkv, int d,
                                                int layout, int write_cache, int M, void* stream) {
    const PtaRotation rot = pta_rotation_of(rotation);
    if (check_qkv_tail("gemm_splitk_reduced_qkv_bf16", q_out, rot, token_pos, token_seq, block_table, k_pool, v_pool, nh, nkv,
                       d, layout, write_cache))
        return 1;
    PTA_REQUIRE(part, "gemm_splitk_reduced_qkv_bf16: null workspace");
    const int N = (nh + 2 * nkv) * d;
    const int rc = pta_gemm_splitk_bf16(nullptr, part, x, W, nullptr, nullptr, nullptr, M, N, K, PTA_ACT_NONE, 0, 0, 0, 0,
                                        0, 0, stream);
    if (rc) return rc;
    const long MN = (long)M * N;
    const QkvTail tail{(bf16_t*)q_out, rot, token_pos, token_seq, block_table, bt_stride, (bf16_t*)k_pool,
                       (bf16_t*)v_pool, nh, nkv, d, layout, write_cache};
    hipLaunchKernelGGL(gemm_splitk_reduce2_qkv_kernel, dim3((unsigned)((MN / 2 + 255) / 256)), dim3(256), 0,
                       (hipStream_t)stream, tail, part, bias, MN, N, pta_gemm_splitk_parts(N, K, 0, 0), (bf16_t*)nullptr,
                       (const float*)nullptr, (const float*)nullptr, 0L, 1, 1, 0);
    return pta_check_launch("gemm_splitk_reduced_qkv_bf16");
}

// ---- the same product for callers that cannot allocate ---------------------------------------------------
// The 32-bit partial sums of the ranges of K lie in a file-scope device array instead of a workspace that the
// caller brings.  Every GPU holds its own copy of the array at its own address until the process ends; its
// address is asked from the runtime once per device, with that device current, and only that address is ever
// handed to a kernel or a runtime call (the array's name in host code is a stand-in, no device address).
#define PTA_STATIC_PART_FLOATS (4 * 1024 * 1024)  // 16 MiB per GPU
#define PTA_MAX_DEVICES 64
static __device__ __align__(256) float scratch[PTA_STATIC_PART_FLOATS];
static float* scratch_ptr[PTA_MAX_DEVICES] = {nullptr};
static std::mutex scratch_lock;

// the current device's copy of `scratch`; null after storing the reason
static float* static_workspace() {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= PTA_MAX_DEVICES) {
        pta_fail("gemm_splitk_bf16_static: no current device (or more than %d devices)", PTA_MAX_DEVICES);
        return nullptr;
    }
    std::lock_guard<std::mutex> hold(scratch_lock);
    if (!scratch_ptr[dev]) {
        void* p = nullptr;
        const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) {
            pta_fail("gemm_splitk_bf16_static: the workspace's address on device %d is not known: %s", dev,
                     hipGetErrorString(e));
            return nullptr;
        }
        scratch_ptr[dev] = (float*)p;
    }
    return scratch_ptr[dev];
}

extern "C" long pta_gemm_splitk_static_floats(void) { return PTA_STATIC_PART_FLOATS; }

extern "C" int pta_gemm_splitk_bf16_static(void* y, const void* x, const void* W, const float* bias, const void* add1,
                                           const void* add2, int M, int N, int K, int act, int out_f32, void* stream) {
    if (check_splitk("gemm_splitk_bf16_static", x, W, M, N, K)) return 1;
    const long need = (long)pta_gemm_splitk_parts(N, K, 0, 0) * M * N;
    PTA_REQUIRE(need <= (long)PTA_STATIC_PART_FLOATS,
                "gemm_splitk_bf16_static: %d ranges of K x %d rows x %d features are %ld partial sums, the built-in "
                "workspace holds %d (bring a workspace to pta_gemm_splitk_bf16 instead)",
                pta_gemm_splitk_parts(N, K, 0, 0), M, N, need, PTA_STATIC_PART_FLOATS);
    float* part = static_workspace();
    if (!part) return 1;
    // every partial sum that the reduction reads is written by this call's matrix launch first, so nothing of
    // the array has to start at zero
    return pta_gemm_splitk_bf16(y, part, x, W, bias, add1, add2, M, N, K, act, out_f32, 0, 0, 0, 0, 1, stream);
}
