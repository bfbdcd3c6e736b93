// y[M,N] = act(x[M,K] . W[N,K]^T + bias) + add1 + add2 for a decode batch of up to 64 rows,
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

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef int i32x4_t __attribute__((ext_vector_type(4)));

union Frag8 {
    uint4 u;
    bf16x8_t v;
    i32x4_t i;
};

#define SK_THREADS 256

template <int MT, int RT, int U, int D>
__global__ __launch_bounds__(SK_THREADS) void gemm_splitk_kernel(
    void* __restrict__ y, float* __restrict__ part, const bf16_t* __restrict__ x, const bf16_t* __restrict__ W,
    const float* __restrict__ bias, const bf16_t* __restrict__ add1, const bf16_t* __restrict__ add2, int M, int N,
    int K, int act, int out_f32, int blocks_per_part, int direct) {
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
    const int n_base = blockIdx.x * (64 * RT) + wave * (16 * RT);
    const int nkb = (K + 63) >> 6;
    const int kb0 = blockIdx.y * blocks_per_part, kb1 = min(kb0 + blocks_per_part, nkb);
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

    auto load_x = [&](int stage, i32x4_t(&xr)[PIECES]) {
        const int k_stage = k_begin + stage * KS;
#pragma unroll
        for (int j = 0; j < PIECES; ++j) {
            const int q = tid + j * SK_THREADS, row = q / (KS / 8), k = k_stage + (q % (KS / 8)) * 8;
            const int off = (k < k_end && row < M) ? (row * K + k) * 2 : 0x7ffffff0;
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
        const int k_stage = k_begin + stage * KS + g * 8;
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
            const int m = mt * 16 + r, n = n_base + t * 16 + g * 4;
            if (m >= M || n >= N) continue;
            const long o = (long)m * N + n;
            if (!direct) {
                const long idx = (long)blockIdx.y * M * N + o;
                float* dst = part + idx;
                if (n + 3 < N && (idx & 3) == 0) *reinterpret_cast<f32x4_t*>(dst) = acc[t][mt];
                else
                    for (int i = 0; i < 4 && n + i < N; ++i) dst[i] = acc[t][mt][i];
                continue;
            }
            for (int i = 0; i < 4 && n + i < N; ++i) {
                float v = acc[t][mt][i];
                if (!out_f32) v = round_to_bf16(v);
                if (bias) { v += bias[n + i]; if (!out_f32) v = round_to_bf16(v); }
                if (act == PTA_ACT_GELU) v = gelu_erf(v);
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
    if (act == PTA_ACT_GELU) v = gelu_erf(v);
    if (add1) v += bf16_bits_to_f32(add1[o]);
    if (add2) v += bf16_bits_to_f32(add2[o]);
    if (out_f32) ((float*)y)[o] = v;
    else ((bf16_t*)y)[o] = f32_to_bf16_bits(v);
}

static int pick_rt(int N) { return N >= 16384 ? 2 : 1; }

// Ranges of K (workgroups along gridDim.y): enough for about two workgroups per compute unit, but no
// range shorter than 512 elements and no more partial sums than about a sixth of W's bytes at 64 rows.
static int pick_parts(int N, int K, int rt) {
    const int groups = (N + 64 * rt - 1) / (64 * rt);
    int P = (512 + groups - 1) / groups;
    P = min(P, max(1, K / 512));
    P = min(P, max(1, K / 900));
    return max(1, min(P, 16));
}

// ranges that are not empty when K is cut into `parts` ranges of whole 64-element blocks
static int effective_parts(int K, int parts) {
    const int nkb = (K + 63) / 64, per = (nkb + parts - 1) / parts;
    return (nkb + per - 1) / per;
}

extern "C" int pta_gemm_splitk_parts(int N, int K, int parts, int rt) {
    if (N <= 0 || K <= 0) return 0;
    if (rt <= 0) rt = pick_rt(N);
    return effective_parts(K, parts > 0 ? parts : pick_parts(N, K, rt));
}

template <int MT, int RT, int U, int D>
static int launch_cfg(void* y, float* part, const bf16_t* x, const bf16_t* W, const float* bias, const bf16_t* add1,
                      const bf16_t* add2, int M, int N, int K, int act, int out_f32, int P, int reduce, hipStream_t s) {
    const int nkb = (K + 63) / 64;
    const int per = (nkb + P - 1) / P;
    const int parts = (nkb + per - 1) / per;  // ranges that are not empty
    const size_t lds = (size_t)2 * MT * 16 * (U * 64 + 8) * sizeof(bf16_t);
    auto kern = gemm_splitk_kernel<MT, RT, U, D>;
    if (lds > 64 * 1024) {
        static bool raised = false;  // per instantiation
        if (!raised) {
            if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
                return pta_fail("gemm_splitk_bf16: cannot have %zu bytes of LDS", lds);
            raised = true;
        }
    }
    const dim3 grid((N + 64 * RT - 1) / (64 * RT), parts);
    hipLaunchKernelGGL(kern, grid, dim3(SK_THREADS), lds, s, y, part, x, W, bias, add1, add2, M, N, K, act, out_f32, per,
                       (int)(reduce && parts == 1));
    if (reduce && parts > 1) {
        const long MN = (long)M * N;
        hipLaunchKernelGGL(gemm_splitk_reduce_kernel, dim3((unsigned)((MN + 255) / 256)), dim3(256), 0, s, y, part, bias,
                           add1, add2, MN, N, parts, act, out_f32);
    }
    return pta_check_launch("gemm_splitk_bf16");
}

template <int RT, int U, int D>
static int launch_rows(int MT, void* y, float* part, const bf16_t* x, const bf16_t* W, const float* bias,
                       const bf16_t* add1, const bf16_t* add2, int M, int N, int K, int act, int out_f32, int P,
                       int reduce, hipStream_t s) {
    switch (MT) {
        case 1: return launch_cfg<1, RT, U, D>(y, part, x, W, bias, add1, add2, M, N, K, act, out_f32, P, reduce, s);
        case 2: return launch_cfg<2, RT, U, D>(y, part, x, W, bias, add1, add2, M, N, K, act, out_f32, P, reduce, s);
        case 3: return launch_cfg<3, RT, U, D>(y, part, x, W, bias, add1, add2, M, N, K, act, out_f32, P, reduce, s);
        default: return launch_cfg<4, RT, U, D>(y, part, x, W, bias, add1, add2, M, N, K, act, out_f32, P, reduce, s);
    }
}

extern "C" int pta_gemm_splitk_bf16(void* y, float* part, const void* x, const void* W, const float* bias,
                                    const void* add1, const void* add2, int M, int N, int K, int act, int out_f32,
                                    int rt, int parts, int stage_blocks, int depth, int reduce, void* stream) {
    PTA_REQUIRE(M > 0 && N > 0 && K > 0, "gemm_splitk_bf16: sizes must be positive (M=%d N=%d K=%d)", M, N, K);
    PTA_REQUIRE(M <= 64, "gemm_splitk_bf16: at most 64 rows, got %d (use the library product)", M);
    PTA_REQUIRE(K % 8 == 0 && K >= 8, "gemm_splitk_bf16: K=%d must be a multiple of 8 (16-byte loads)", K);
    PTA_REQUIRE(x && W && (y || !reduce), "gemm_splitk_bf16: null pointer");
    PTA_REQUIRE((long)M * K * 2 < 0x7ffffff0L, "gemm_splitk_bf16: x is too large for 32-bit buffer offsets");
    PTA_REQUIRE(((uintptr_t)x % 16) == 0 && ((uintptr_t)W % 16) == 0, "gemm_splitk_bf16: x and W must be 16-byte aligned");
    PTA_REQUIRE(act == PTA_ACT_NONE || act == PTA_ACT_GELU, "gemm_splitk_bf16: unknown activation %d", act);
    PTA_REQUIRE(rt == 0 || rt == 1 || rt == 2, "gemm_splitk_bf16: row tiles per wave must be 0 (choose), 1 or 2, got %d", rt);
    PTA_REQUIRE(stage_blocks == 0 || stage_blocks == 2,
                "gemm_splitk_bf16: 64-element blocks per stage must be 0 (choose) or 2, got %d", stage_blocks);
    PTA_REQUIRE(depth == 0 || depth == 2 || depth == 4, "gemm_splitk_bf16: stages in flight must be 0 (choose), 2 or 4, got %d", depth);
    PTA_REQUIRE(parts >= 0 && parts <= 64, "gemm_splitk_bf16: parts must be 0 (choose) or 1..64, got %d", parts);
    if (rt == 0) rt = pick_rt(N);
    if (parts == 0) parts = pick_parts(N, K, rt);
    if (stage_blocks == 0) stage_blocks = 2;
    PTA_REQUIRE((parts == 1 && reduce) || part, "gemm_splitk_bf16: %d ranges of K need the workspace for partial sums", parts);
    parts = effective_parts(K, parts);  // what the caller's workspace must hold
    hipStream_t s = (hipStream_t)stream;
    const int MT = (M + 15) / 16;
    const bf16_t *xb = (const bf16_t*)x, *wb = (const bf16_t*)W, *a1 = (const bf16_t*)add1, *a2 = (const bf16_t*)add2;
    if (depth == 0) depth = 2;  // measured: more stages in flight per wave do not pay, more workgroups do
#define SK_CASE(RT_, U_, D_)                                                                                      \
    if (rt == RT_ && stage_blocks == U_ && depth == D_)                                                           \
        return launch_rows<RT_, U_, D_>(MT, y, part, xb, wb, bias, a1, a2, M, N, K, act, out_f32, parts, reduce, s);
    SK_CASE(1, 2, 2) SK_CASE(1, 2, 4) SK_CASE(2, 2, 2) SK_CASE(2, 2, 4)
#undef SK_CASE
    return pta_fail("gemm_splitk_bf16: no kernel for rt=%d stage_blocks=%d depth=%d", rt, stage_blocks, depth);
}
