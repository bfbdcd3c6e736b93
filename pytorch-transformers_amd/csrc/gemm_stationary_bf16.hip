// The two products of a pair launch for a decode batch of 17 to 128 rows, left as 32-bit partial sums, with the
// activations stationary: part[p, M, N] = x[M, range p of K] . W[N, range p of K]^T.
//
// The kernel that walks K in stages (gemm_splitk_bf16.hip) copies every stage's slice of x into LDS once per
// workgroup of 64 rows of W, with a barrier per stage: at 64 rows of x a workgroup pulls as many bytes of x out of
// L2 as of W out of memory.  Here a launch has about as many workgroups as the chip has compute units, each of
// eight waves, and each wave owns up to TMAX tiles of sixteen rows of W whose 32-bit sums it keeps in registers
// while the workgroup walks its range of K in phases: a phase's slice of x, [rows, KP], lies in one of two LDS
// buffers (the next phase's is fetched meanwhile and written at the phase's end, one barrier per phase), and
// within a phase a wave takes its tiles one after the other, W rows straight from global memory into the A
// operand registers, PF steps of 32 elements ahead and across tile and phase boundaries.  A slice of x is thus
// read once per workgroup and phase for all its tiles (some 22 at the shapes this was written for), and K needs to
// be cut into ranges only as far as the row tiles alone leave compute units idle: fewer partial sums.
//
// Rows of x past M and elements past the range's end arrive as zeros (buffer loads out of bounds); W addresses
// are clamped into the range instead, so a step past the end multiplies weights that are in cache by zeros.
#include "common.h"
#include "pta_kernels.h"

#include <algorithm>
#include <type_traits>

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef int i32x4_t __attribute__((ext_vector_type(4)));

union SFrag8 {
    uint4 u;
    bf16x8_t v;
    i32x4_t i;
};

#define ST_WAVES 8
#define ST_THREADS (ST_WAVES * 64)
#define ST_LDS_BYTES (152 * 1024)

struct StationaryProblem {
    float* part;
    const bf16_t* x;
    const bf16_t* W;
    int N, K;
    int parts;            // ranges of K
    int blocks_per_part;  // 64-element blocks of K per range
    int groups;           // workgroups per range; workgroup g takes the row tiles g, g + groups, ...
};

// MT: sixteen-row tiles of x.  KP: elements of K per phase (a multiple of 64).  PF: 32-element steps of W in flight
// per wave; it is even and divides the steps of a phase, so that a step's registers are known when the kernel is
// compiled.  Every phase runs all its steps: past the range's end x is zero.
// SINGLE: the workgroup's whole range of K is one phase (the host has seen to it that it fits): one LDS buffer, and
// after the first no barrier at all.  The barriers cost more than they look: the waves of a workgroup stream their
// tiles at the pace memory gives each of them, and at every phase's end all wait for the slowest (K = 4,544 in
// nine phases: 51 us; in one phase, at 8 rows, 42 us, which is what a kernel that only reads W in this walk takes).
template <int MT, int KP, int PF, int ST_TMAX, bool SINGLE>
__global__ __launch_bounds__(ST_THREADS) void gemm_stationary_kernel(StationaryProblem pa, StationaryProblem pb, int M) {
    constexpr int MP = MT * 16;
    constexpr int LDW = KP + 8;  // 16 bytes of padding keep the sixteen rows of a 16-byte read on distinct banks
    constexpr int STEPS = KP / 32;
    static_assert(STEPS % PF == 0 && PF % 2 == 0, "the loads in flight must divide a phase's steps and be even");
    constexpr int PIECES = MP * (KP / 8) / ST_THREADS;  // 16-byte pieces of a slice per thread
    static_assert(MP * (KP / 8) % ST_THREADS == 0, "a slice of x must divide over the threads");
    extern __shared__ __attribute__((aligned(16))) bf16_t xs[];  // [2][MP][LDW], [MP][LDW] if SINGLE

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r = lane & 15, g4 = lane >> 4;
    const int first = pa.groups * pa.parts;
    const bool second = (int)blockIdx.x >= first;
    const StationaryProblem& pr = second ? pb : pa;
    float* __restrict__ part = pr.part;
    const bf16_t* __restrict__ x = pr.x;
    const bf16_t* __restrict__ W = pr.W;
    const int N = pr.N, K = pr.K, groups = pr.groups;
    const int idx = (int)blockIdx.x - (second ? first : 0);
    const int range = idx % pr.parts, group = idx / pr.parts;
    const int nkb = (K + 63) >> 6;
    const int kb0 = range * pr.blocks_per_part, kb1 = min(kb0 + pr.blocks_per_part, nkb);
    const int k_begin = kb0 * 64, k_end = min(kb1 * 64, K);
    const int phases = SINGLE ? 1 : (k_end - k_begin + KP - 1) / KP;
    // steps of a phase: all of them, or with one phase as many as the range has, in whole rounds of PF
    const int nsteps = SINGLE ? min(STEPS, (((k_end - k_begin + 31) >> 5) + PF - 1) / PF * PF) : STEPS;
    const int n_tiles = (N + 15) >> 4;
    // this wave's tiles: group + groups * (wave + 8 j)
    const int t0 = group + groups * wave, t_stride = groups * ST_WAVES;
    const int n_my = t0 < n_tiles ? min(ST_TMAX, (n_tiles - t0 + t_stride - 1) / t_stride) : 0;

    __amdgpu_buffer_rsrc_t xres = __builtin_amdgcn_make_buffer_rsrc((void*)x, 0, M * K * 2, 0x00020000);
    i32x4_t xr[PIECES];
    auto load_x = [&](int phase) {
        const int k0 = k_begin + phase * KP;
#pragma unroll
        for (int j = 0; j < PIECES; ++j) {
            const int q = tid + j * ST_THREADS, row = q / (KP / 8), k = k0 + (q % (KP / 8)) * 8;
            const int off = (k < k_end && row < M && phase < phases) ? (row * K + k) * 2 : 0x7ffffff0;
            xr[j] = __builtin_amdgcn_raw_buffer_load_b128(xres, off, 0, 0);
        }
    };
    auto store_x = [&](int buf) {
#pragma unroll
        for (int j = 0; j < PIECES; ++j) {
            const int q = tid + j * ST_THREADS, row = q / (KP / 8), c8 = q % (KP / 8);
            *reinterpret_cast<i32x4_t*>(&xs[(buf * MP + row) * LDW + c8 * 8]) = xr[j];
        }
    };

    // the cursor of the W loads runs PF steps ahead of the matrix cores through (phase, tile, step)
    SFrag8 w[PF];
    int p_phase = 0, p_tile = 0, p_step = 0;
    const bf16_t* p_row = W + (long)min(t0 * 16 + r, N - 1) * K;
    auto prefetch = [&](SFrag8& dst) {
        const int k = min(k_begin + p_phase * KP + p_step * 32 + g4 * 8, k_end - 8);
        dst.u = *reinterpret_cast<const uint4*>(p_row + k);
        if (++p_step >= nsteps) {
            p_step = 0;
            if (++p_tile >= n_my) { p_tile = 0; ++p_phase; }
            p_row = W + (long)min((t0 + t_stride * p_tile) * 16 + r, N - 1) * K;
        }
    };
    if (n_my > 0) {
#pragma unroll
        for (int u = 0; u < PF; ++u) prefetch(w[u]);
    }
    load_x(0);
    store_x(0);
    __syncthreads();

    f32x4_t acc[ST_TMAX][MT];
#pragma unroll
    for (int t = 0; t < ST_TMAX; ++t)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) acc[t][mt] = f32x4_t{0.f, 0.f, 0.f, 0.f};

    // The phases for a wave with NT tiles, NT known when the kernel is compiled: the next phase's slice of x is asked
    // for at the start of the wave's last round of steps of the phase and written to LDS at the phase's end, so
    // that the compiler can count the W loads that are younger than it (one round's) and lets the wave wait for
    // the slice alone.  Asked for at the phase's start, a loop of unknown length lies between the slice's loads
    // and their use, the count is unknown, and the wave waits for every load it has in flight, W rows included,
    // at every phase's end.
    auto run = [&](auto tiles_c) {
        constexpr int NT = decltype(tiles_c)::value;
        for (int phase = 0; phase < phases; ++phase) {
            const int buf = phase & 1;
            // a step's B fragments are read from LDS while the step before it is on the matrix cores: two sets of
            // registers that alternate, and a scheduling barrier per step, without which the compiler reads all of
            // a round's fragments first and runs out of registers
            bf16x8_t b[2][MT];
            auto read_b = [&](bf16x8_t(&dst)[MT], int step) {
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
                    dst[mt] = *reinterpret_cast<const bf16x8_t*>(&xs[(buf * MP + mt * 16 + r) * LDW + step * 32 + g4 * 8]);
            };
            if constexpr (NT == 0 && !SINGLE) load_x(phase + 1);
            if constexpr (NT > 0) read_b(b[0], 0);
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                auto round = [&](int s0) {
#pragma unroll
                    for (int u = 0; u < PF; ++u) {
                        const int next = s0 + u + 1;
                        read_b(b[(u + 1) & 1], next == nsteps ? 0 : next);  // the next tile starts at the slice's start
#pragma unroll
                        for (int mt = 0; mt < MT; ++mt)
                            acc[t][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w[u].v, b[u & 1][mt], acc[t][mt], 0, 0, 0);
                        prefetch(w[u]);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                };
                for (int s0 = 0; s0 < nsteps - PF; s0 += PF) round(s0);
                if constexpr (!SINGLE) {
                    if (t == NT - 1) {
                        load_x(phase + 1);  // zeros past the last phase
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
                round(nsteps - PF);
            }
            if constexpr (!SINGLE) {
                __builtin_amdgcn_sched_barrier(0);
                store_x(buf ^ 1);
                __syncthreads();
            }
        }
    };
    switch (n_my) {
        case 0: run(std::integral_constant<int, 0>{}); break;
        case 1: run(std::integral_constant<int, 1>{}); break;
        case 2: run(std::integral_constant<int, 2>{}); break;
        default:
            if constexpr (ST_TMAX >= 3) run(std::integral_constant<int, 3>{});
            break;
    }

    // lane: row m = mt*16 + r of x, columns tile*16 + g4*4 + 0..3
#pragma unroll
    for (int t = 0; t < ST_TMAX; ++t) {
        if (t >= n_my) break;
        const int n = (t0 + t_stride * t) * 16 + g4 * 4;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const int m = mt * 16 + r;
            if (m >= M || n >= N) continue;
            const long at = ((long)range * M + m) * N + n;
            if (n + 3 < N && (at & 3) == 0) *reinterpret_cast<f32x4_t*>(part + at) = acc[t][mt];
            else
                for (int i = 0; i < 4 && n + i < N; ++i) part[at + i] = acc[t][mt][i];
        }
    }
}

static StationaryProblem make_stationary(float* part, const void* x, const void* W, int N, int K, int parts, int groups) {
    StationaryProblem p{};
    p.part = part; p.x = (const bf16_t*)x; p.W = (const bf16_t*)W; p.N = N; p.K = K;
    const int nkb = (K + 63) / 64;
    p.blocks_per_part = (nkb + parts - 1) / parts;
    p.parts = (nkb + p.blocks_per_part - 1) / p.blocks_per_part;
    p.groups = groups;
    return p;
}

template <int MT, int KP, int PF, int TMAX, bool SINGLE = false>
static int launch_stationary(const StationaryProblem& a, const StationaryProblem& b, int M, hipStream_t s) {
    constexpr size_t lds = (size_t)(SINGLE ? 1 : 2) * MT * 16 * (KP + 8) * sizeof(bf16_t);
    static_assert(lds <= ST_LDS_BYTES, "two slices of x must fit the LDS of a compute unit");
    auto kern = gemm_stationary_kernel<MT, KP, PF, TMAX, SINGLE>;
    if (lds > 64 * 1024) {
        static bool raised = false;
        if (!raised) {
            if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess)
                return pta_fail("gemm_stationary_pair_bf16: cannot have %zu bytes of LDS", lds);
            raised = true;
        }
    }
    hipLaunchKernelGGL(kern, dim3(a.groups * a.parts + b.groups * b.parts), dim3(ST_THREADS), lds, s, a, b, M);
    return pta_check_launch("gemm_stationary_pair_bf16");
}

// workgroups per range of K for the two products: together about one per compute unit, shared by the bytes of
// the two matrices, and at least as many as the tiles a wave can hold ask for
// row tiles of W that a wave holds at most: what the sums of M rows leave registers for
static int stationary_tmax(int M) { return M <= 64 ? 3 : 2; }

extern "C" int pta_gemm_stationary_groups(int N1, int K1, int parts1, int N2, int K2, int parts2, int M, int* g1, int* g2) {
    const int tmax = stationary_tmax(M);
    if (N1 <= 0 || K1 <= 0 || N2 <= 0 || K2 <= 0 || parts1 <= 0 || parts2 <= 0 || parts1 > 64 || parts2 > 64)
        return pta_fail("gemm_stationary_groups: sizes must be positive, ranges 1 to 64");
    // Workgroups per range for the two products: as many as the compute units in all and no more (a few workgroups
    // over start when the first ones end and double the launch's time; half as many, which would read x half as
    // often, take a third longer: a compute unit alone pulls no more than some 21 GB/s out of memory in this walk),
    // shared so that the slower kind of workgroup, by its tiles per wave times the length of its range, is as
    // fast as can be; more than the units only where the tiles a wave can hold ask for it.
    const int units = pta_compute_units(), t1 = (N1 + 15) / 16, t2 = (N2 + 15) / 16;
    const int need1 = (t1 + ST_WAVES * tmax - 1) / (ST_WAVES * tmax), need2 = (t2 + ST_WAVES * tmax - 1) / (ST_WAVES * tmax);
    const double r1 = (double)K1 / parts1, r2 = (double)K2 / parts2;
    double best = 0.0;
    *g1 = need1;
    *g2 = need2;
    for (int a = need1; a == need1 || a * parts1 + need2 * parts2 <= units; ++a) {
        const int b = std::max(need2, (units - a * parts1) / parts2);
        const double rounds = (double)((a * parts1 + b * parts2 + units - 1) / units);
        const double per1 = (double)((t1 + a - 1) / a) / ST_WAVES * r1, per2 = (double)((t2 + b - 1) / b) / ST_WAVES * r2;
        const double cost = std::max(per1, per2) * rounds;
        if (best == 0.0 || cost < best) {
            best = cost;
            *g1 = a;
            *g2 = b;
        }
    }
    return 0;
}

extern "C" int pta_gemm_stationary_pair_bf16(float* part1, const void* x1, const void* W1, int N1, int K1, int parts1,
                                             float* part2, const void* x2, const void* W2, int N2, int K2, int parts2,
                                             int M, void* stream) {
    PTA_REQUIRE(M >= 1 && M <= 128, "gemm_stationary_pair_bf16: 1 to 128 rows, got %d", M);
    PTA_REQUIRE(N1 > 0 && K1 > 0 && N2 > 0 && K2 > 0, "gemm_stationary_pair_bf16: sizes must be positive");
    PTA_REQUIRE(K1 % 8 == 0 && K2 % 8 == 0, "gemm_stationary_pair_bf16: K must be a multiple of 8 (16-byte loads)");
    PTA_REQUIRE(part1 && part2 && x1 && x2 && W1 && W2, "gemm_stationary_pair_bf16: null pointer");
    PTA_REQUIRE(parts1 >= 1 && parts2 >= 1 && parts1 <= 64 && parts2 <= 64, "gemm_stationary_pair_bf16: 1 to 64 ranges of K");
    PTA_REQUIRE((long)M * K1 * 2 < 0x7ffffff0L && (long)M * K2 * 2 < 0x7ffffff0L,
                "gemm_stationary_pair_bf16: x is too large for 32-bit buffer offsets");
    for (const void* p : {x1, x2, W1, W2})
        PTA_REQUIRE(((uintptr_t)p % 16) == 0, "gemm_stationary_pair_bf16: x and W must be 16-byte aligned");
    int g1, g2;
    if (pta_gemm_stationary_groups(N1, K1, parts1, N2, K2, parts2, M, &g1, &g2)) return 1;
    const StationaryProblem a = make_stationary(part1, x1, W1, N1, K1, parts1, g1);
    const StationaryProblem b = make_stationary(part2, x2, W2, N2, K2, parts2, g2);
    hipStream_t s = (hipStream_t)stream;
    // ranges of K that fit LDS whole run as one phase
    const int longest = std::max(a.blocks_per_part, b.blocks_per_part) * 64;
    switch ((M + 15) / 16) {
        case 1: if (longest <= 4608) return launch_stationary<1, 4608, 8, 3, true>(a, b, M, s); break;
        case 2: if (longest <= 2304) return launch_stationary<2, 2304, 8, 3, true>(a, b, M, s); break;
        case 3: if (longest <= 1536) return launch_stationary<3, 1536, 8, 3, true>(a, b, M, s); break;
        case 4: if (longest <= 1152) return launch_stationary<4, 1152, 12, 3, true>(a, b, M, s); break;
        default: break;
    }
    switch ((M + 15) / 16) {
        case 1: return launch_stationary<1, 2048, 8, 3>(a, b, M, s);
        case 2: return launch_stationary<2, 1024, 8, 3>(a, b, M, s);
        case 3: return launch_stationary<3, 768, 8, 3>(a, b, M, s);
        case 4: return launch_stationary<4, 512, 8, 3>(a, b, M, s);
        case 5: case 6: return launch_stationary<6, 384, 6, 2>(a, b, M, s);
        default: return launch_stationary<8, 256, 8, 2>(a, b, M, s);
    }
}
