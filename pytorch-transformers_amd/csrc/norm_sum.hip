// The residual sum and the LayerNorm that reads it, in one pass over bfloat16 rows.
//
//   v    = A + B + add1 + add2 + add3   (terms that are absent are skipped; at least one is given)
//   x    = round(v)                     -> out_x, if wanted
//   out1 = LN(x) * w1 + b1              -> if wanted; out2 with (w2, b2) likewise
//
// A and B are matrix products that their kernels left as 32-bit partial sums over ranges of K,
// [parts, rows, H]; each is summed in the order of its ranges, rounded to bfloat16, and its bias is
// added and rounded again: what the epilogue of a product that ran whole would have stored.  B comes
// first in the sum, then A, then the bfloat16 addends, as in the epilogue of the block's last product
// (feed-forward plus mixer first, then the residual).  `rows` selects source rows (the final norm reads
// only the rows whose logits are wanted).
//
// One workgroup per row (H <= 8192, H % 8 == 0); a thread holds its chunks of eight features in registers,
// loaded and stored sixteen bytes at a time.  Norm weights are loaded before the reductions so that their
// latency hides behind them.  Mean and biased variance in 32-bit, variance from the centred values.
#include "common.h"
#include "pta_kernels.h"

#define NS_THREADS 1024  // at most
#define NS_MAX_H (NS_THREADS * 8)
#define NS_ROWS_MIN 512  // rows from which a wave per row is the faster arrangement

__device__ __forceinline__ void load8f(const float* p, float (&f)[8]) {
    const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
    f[0] = a.x; f[1] = a.y; f[2] = a.z; f[3] = a.w; f[4] = b.x; f[5] = b.y; f[6] = b.z; f[7] = b.w;
}

// round(sum of the parts in order), then the bias added and rounded.  The parts are loaded eight at a
// time before they are added, so that their latencies overlap (a row's workgroup runs on one compute unit,
// and what it waits for is the number of round trips to memory, not the bytes).
__device__ __forceinline__ void product_value(const float* part, int P, long part_stride, const float* bias, long at,
                                              int i, float (&out)[8]) {
    float bv[8];
    if (bias) load8f(bias + i, bv);
    for (int p0 = 0; p0 < P; p0 += 8) {
        float t[8][8];
#pragma unroll
        for (int u = 0; u < 8; ++u) load8f(part + (long)min(p0 + u, P - 1) * part_stride + at, t[u]);
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            if (p0 + u >= P) continue;
#pragma unroll
            for (int e = 0; e < 8; ++e) out[e] = (p0 + u == 0) ? t[u][e] : out[e] + t[u][e];
        }
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) out[e] = round_to_bf16(out[e]);
    if (bias) {
#pragma unroll
        for (int e = 0; e < 8; ++e) out[e] = round_to_bf16(out[e] + bv[e]);
    }
}

// CH chunks of eight features per thread, blockDim.x * CH * 8 >= H.
template <int CH>
__global__ __launch_bounds__(NS_THREADS / CH) void layernorm_sum_kernel(
    bf16_t* __restrict__ out_x, bf16_t* __restrict__ out1, bf16_t* __restrict__ out2, const float* __restrict__ pa,
    int Pa, const float* __restrict__ bias_a, const float* __restrict__ pb, int Pb, const float* __restrict__ bias_b,
    const bf16_t* __restrict__ add1, const bf16_t* __restrict__ add2, const bf16_t* __restrict__ add3,
    const int* __restrict__ rows, const float* __restrict__ w1, const float* __restrict__ b1,
    const float* __restrict__ w2, const float* __restrict__ b2, int M_in, int H, float eps) {
    __shared__ float red[16];
    const int m = blockIdx.x;
    const long src = rows ? (long)rows[m] : (long)m;
    const long part_stride = (long)M_in * H;
    float v[CH][8];
    float gw1[CH][8], gb1[CH][8], gw2[CH][8], gb2[CH][8];
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < CH; ++j) {
        const int i = (threadIdx.x + j * blockDim.x) * 8;
        if (i >= H) continue;
        const long at = src * H + i;
        if (out1) { load8f(w1 + i, gw1[j]); load8f(b1 + i, gb1[j]); }
        if (out2) { load8f(w2 + i, gw2[j]); load8f(b2 + i, gb2[j]); }
        bool any = false;
        if (pb) { product_value(pb, Pb, part_stride, bias_b, at, i, v[j]); any = true; }
        if (pa) {
            float t[8];
            product_value(pa, Pa, part_stride, bias_a, at, i, t);
#pragma unroll
            for (int e = 0; e < 8; ++e) v[j][e] = any ? v[j][e] + t[e] : t[e];
            any = true;
        }
        if (add1) {
            float t[8];
            unpack8(*reinterpret_cast<const uint4*>(add1 + at), t);
#pragma unroll
            for (int e = 0; e < 8; ++e) v[j][e] = any ? v[j][e] + t[e] : t[e];
            any = true;
        }
        if (add2) {
            float t[8];
            unpack8(*reinterpret_cast<const uint4*>(add2 + at), t);
#pragma unroll
            for (int e = 0; e < 8; ++e) v[j][e] = any ? v[j][e] + t[e] : t[e];
            any = true;
        }
        if (add3) {
            float t[8];
            unpack8(*reinterpret_cast<const uint4*>(add3 + at), t);
#pragma unroll
            for (int e = 0; e < 8; ++e) v[j][e] = any ? v[j][e] + t[e] : t[e];
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            v[j][e] = round_to_bf16(v[j][e]);
            s += v[j][e];
        }
        if (out_x) *reinterpret_cast<uint4*>(out_x + (long)m * H + i) = pack8(v[j]);
    }
    if (!out1) return;
    const float mean = block_sum(s, red) / (float)H;
    float q = 0.f;
#pragma unroll
    for (int j = 0; j < CH; ++j) {
        const int i = (threadIdx.x + j * blockDim.x) * 8;
        if (i >= H) continue;
#pragma unroll
        for (int e = 0; e < 8; ++e) { const float d = v[j][e] - mean; q += d * d; }
    }
    const float var = block_sum(q, red) / (float)H;
    const float rstd = 1.0f / sqrtf(var + eps);
#pragma unroll
    for (int j = 0; j < CH; ++j) {
        const int i = (threadIdx.x + j * blockDim.x) * 8;
        if (i >= H) continue;
        float o[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) o[e] = (v[j][e] - mean) * rstd * gw1[j][e] + gb1[j][e];
        *reinterpret_cast<uint4*>(out1 + (long)m * H + i) = pack8(o);
        if (out2) {
#pragma unroll
            for (int e = 0; e < 8; ++e) o[e] = (v[j][e] - mean) * rstd * gw2[j][e] + gb2[j][e];
            *reinterpret_cast<uint4*>(out2 + (long)m * H + i) = pack8(o);
        }
    }
}


// The same for a decode step's usual terms (two products of at most NB and NA ranges, up to three tensors), with every
// load of a thread's chunk asked for before the first is used.  A row's workgroup runs on one compute unit and what it
// waits for is round trips to memory, not bytes: one product after the other, then the tensors, each wait a trip;
// here the weights' loads are asked for when the sum is formed and arrive behind the two reductions, and everything
// else is one trip.  The additions are the same, in the same order: the same bits.  Measured in whole decode steps
// at 32 layers of 4,544 features, 8 rows: 3.416 -> 3.384 ms a step (a microsecond a layer; most of this kernel's nine
// are what any kernel boundary costs).
// TH: the most threads of a launch (what the registers of a thread are bounded by: 12 ranges in flight need more
// than the 128 that 1,024 threads leave each).
template <int NB, int NA, int TH = NS_THREADS>
__global__ __launch_bounds__(TH) void layernorm_sum_ahead_kernel(
    bf16_t* __restrict__ out_x, bf16_t* __restrict__ out1, bf16_t* __restrict__ out2, const float* __restrict__ pa,
    int Pa, const float* __restrict__ bias_a, const float* __restrict__ pb, int Pb, const float* __restrict__ bias_b,
    const bf16_t* __restrict__ add1, const bf16_t* __restrict__ add2, const bf16_t* __restrict__ add3,
    const int* __restrict__ rows, const float* __restrict__ w1, const float* __restrict__ b1,
    const float* __restrict__ w2, const float* __restrict__ b2, int M_in, int H, float eps) {
    __shared__ float red[16];
    const int m = blockIdx.x;
    const long src = rows ? (long)rows[m] : (long)m;
    const long part_stride = (long)M_in * H;
    const int i = threadIdx.x * 8;
    const bool live = i < H;
    const long at = src * H + (live ? i : 0);
    // of the first product's ranges at most FLY are on their way at once: a range past them is asked for into the
    // registers of the range that was just added (16 at once need more registers than a wave has)
    constexpr int FLY = NB < 12 ? NB : 12;
    float tb[FLY][8], ta[NA][8], v[8];
    uint4 r1 = make_uint4(0u, 0u, 0u, 0u), r2 = r1, r3 = r1;
#pragma unroll
    for (int u = 0; u < FLY; ++u) load8f(pb + (long)min(u, Pb - 1) * part_stride + at, tb[u]);
    if (pa) {
#pragma unroll
        for (int u = 0; u < NA; ++u) load8f(pa + (long)min(u, Pa - 1) * part_stride + at, ta[u]);
    }
    if (add1) r1 = *reinterpret_cast<const uint4*>(add1 + at);
    if (add2) r2 = *reinterpret_cast<const uint4*>(add2 + at);
    if (add3) r3 = *reinterpret_cast<const uint4*>(add3 + at);
    // the first product: its ranges in order, rounded, then its bias added and rounded
#pragma unroll
    for (int u = 0; u < NB; ++u) {
        if (u < Pb) {
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] = u == 0 ? tb[u % FLY][e] : v[e] + tb[u % FLY][e];
        }
        if (u + FLY < NB) load8f(pb + (long)min(u + FLY, Pb - 1) * part_stride + at, tb[u % FLY]);
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = round_to_bf16(v[e]);
    if (bias_b) {
        float bv[8];
        load8f(bias_b + (live ? i : 0), bv);
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = round_to_bf16(v[e] + bv[e]);
    }
    if (pa) {
        float t[8];
#pragma unroll
        for (int u = 0; u < NA; ++u) {
            if (u >= Pa) continue;
#pragma unroll
            for (int e = 0; e < 8; ++e) t[e] = u == 0 ? ta[u][e] : t[e] + ta[u][e];
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) t[e] = round_to_bf16(t[e]);
        if (bias_a) {
            float bv[8];
            load8f(bias_a + (live ? i : 0), bv);
#pragma unroll
            for (int e = 0; e < 8; ++e) t[e] = round_to_bf16(t[e] + bv[e]);
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] += t[e];
    }
    const uint4* adds[3] = {&r1, &r2, &r3};
    const bool has[3] = {add1 != nullptr, add2 != nullptr, add3 != nullptr};
#pragma unroll
    for (int k = 0; k < 3; ++k) {
        if (!has[k]) continue;
        float t[8];
        unpack8(*adds[k], t);
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] += t[e];
    }
    float s = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        v[e] = round_to_bf16(v[e]);
        s += live ? v[e] : 0.f;
    }
    if (out_x && live) *reinterpret_cast<uint4*>(out_x + (long)m * H + i) = pack8(v);
    if (!out1) return;
    float gw1[8], gb1[8], gw2[8], gb2[8];
    load8f(w1 + (live ? i : 0), gw1);
    load8f(b1 + (live ? i : 0), gb1);
    if (out2) { load8f(w2 + (live ? i : 0), gw2); load8f(b2 + (live ? i : 0), gb2); }
    const float mean = block_sum(s, red) / (float)H;
    float q = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) { const float d = v[e] - mean; q += live ? d * d : 0.f; }
    const float var = block_sum(q, red) / (float)H;
    const float rstd = 1.0f / sqrtf(var + eps);
    if (!live) return;
    float o[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) o[e] = (v[e] - mean) * rstd * gw1[e] + gb1[e];
    *reinterpret_cast<uint4*>(out1 + (long)m * H + i) = pack8(o);
    if (out2) {
#pragma unroll
        for (int e = 0; e < 8; ++e) o[e] = (v[e] - mean) * rstd * gw2[e] + gb2[e];
        *reinterpret_cast<uint4*>(out2 + (long)m * H + i) = pack8(o);
    }
}


// Many rows and no products (prompts): one wave per row, four rows per workgroup.  A lane holds every 64th
// chunk of eight features of its row (MAXCH of them at most), all loads of a row are in flight at once, and
// the two reductions stay inside the wave: no LDS, no barrier.
template <int MAXCH>
__global__ __launch_bounds__(256) void layernorm_rows_kernel(
    bf16_t* __restrict__ out_x, bf16_t* __restrict__ out1, bf16_t* __restrict__ out2, const bf16_t* __restrict__ add1,
    const bf16_t* __restrict__ add2, const bf16_t* __restrict__ add3, const float* __restrict__ w1,
    const float* __restrict__ b1, const float* __restrict__ w2, const float* __restrict__ b2, int M, int H, float eps) {
    const int lane = threadIdx.x & 63;
    const long m = (long)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (m >= M) return;
    const int chunks = H / 8;
    uint4 r1[MAXCH], r2[MAXCH], r3[MAXCH];
#pragma unroll
    for (int j = 0; j < MAXCH; ++j) {
        const int ch = min(lane + j * 64, chunks - 1);
        r1[j] = *reinterpret_cast<const uint4*>(add1 + m * H + ch * 8);
        if (add2) r2[j] = *reinterpret_cast<const uint4*>(add2 + m * H + ch * 8);
        if (add3) r3[j] = *reinterpret_cast<const uint4*>(add3 + m * H + ch * 8);
    }
    float v[MAXCH][8];
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < MAXCH; ++j) {
        const bool live = lane + j * 64 < chunks;
        unpack8(r1[j], v[j]);
        if (add2) {  // the terms are added in 32-bit, in their order, and the sum is rounded once
            float t[8];
            unpack8(r2[j], t);
#pragma unroll
            for (int e = 0; e < 8; ++e) v[j][e] += t[e];
            if (add3) {
                unpack8(r3[j], t);
#pragma unroll
                for (int e = 0; e < 8; ++e) v[j][e] += t[e];
            }
#pragma unroll
            for (int e = 0; e < 8; ++e) v[j][e] = round_to_bf16(v[j][e]);
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) s += live ? v[j][e] : 0.f;
        if (out_x && live) *reinterpret_cast<uint4*>(out_x + m * H + (lane + j * 64) * 8) = pack8(v[j]);
    }
    if (!out1) return;
    const float mean = wave_sum(s) / (float)H;
    float q = 0.f;
#pragma unroll
    for (int j = 0; j < MAXCH; ++j) {
        if (lane + j * 64 >= chunks) continue;
#pragma unroll
        for (int e = 0; e < 8; ++e) { const float d = v[j][e] - mean; q += d * d; }
    }
    const float rstd = 1.0f / sqrtf(wave_sum(q) / (float)H + eps);
#pragma unroll
    for (int j = 0; j < MAXCH; ++j) {
        const int i = (lane + j * 64) * 8;
        if (i >= H) continue;
        float gw[8], gb[8], o[8];
        load8f(w1 + i, gw); load8f(b1 + i, gb);
#pragma unroll
        for (int e = 0; e < 8; ++e) o[e] = (v[j][e] - mean) * rstd * gw[e] + gb[e];
        *reinterpret_cast<uint4*>(out1 + m * H + i) = pack8(o);
        if (out2) {
            load8f(w2 + i, gw); load8f(b2 + i, gb);
#pragma unroll
            for (int e = 0; e < 8; ++e) o[e] = (v[j][e] - mean) * rstd * gw[e] + gb[e];
            *reinterpret_cast<uint4*>(out2 + m * H + i) = pack8(o);
        }
    }
}

template <int MAXCH>
static void launch_rows(void* out_x, void* out1, void* out2, const void* add1, const void* add2, const void* add3,
                        const float* w1, const float* b1, const float* w2, const float* b2, int M, int H, float eps,
                        hipStream_t s) {
    hipLaunchKernelGGL(layernorm_rows_kernel<MAXCH>, dim3((M + 3) / 4), dim3(256), 0, s, (bf16_t*)out_x, (bf16_t*)out1,
                       (bf16_t*)out2, (const bf16_t*)add1, (const bf16_t*)add2, (const bf16_t*)add3, w1, b1, w2, b2, M, H, eps);
}

extern "C" int pta_layernorm_sum_ok(int H) { return H > 0 && H % 8 == 0 && H <= NS_MAX_H; }

extern "C" int pta_layernorm_sum_rows_min(void) { return NS_ROWS_MIN; }

extern "C" int pta_layernorm_sum(void* out_x, void* out1, void* out2, const float* pa, int Pa, const float* bias_a,
                                 const float* pb, int Pb, const float* bias_b, const void* add1, const void* add2,
                                 const void* add3, const int* rows, const float* w1, const float* b1, const float* w2, const float* b2,
                                 int M_in, int M, int H, float eps, void* stream) {
    PTA_REQUIRE(M > 0 && M_in > 0 && H > 0, "layernorm_sum: M=%d M_in=%d H=%d must be positive", M, M_in, H);
    PTA_REQUIRE(pta_layernorm_sum_ok(H), "layernorm_sum: H=%d must be a multiple of 8 up to %d", H,
                NS_MAX_H);
    PTA_REQUIRE(pa || pb || add1 || add2 || add3, "layernorm_sum: nothing to sum");
    PTA_REQUIRE(!add3 || (add1 && add2), "layernorm_sum: a third tensor comes after a first and a second");
    PTA_REQUIRE((!pa || Pa > 0) && (!pb || Pb > 0), "layernorm_sum: a product needs at least one part");
    PTA_REQUIRE(out_x || out1, "layernorm_sum: no output wanted");
    PTA_REQUIRE(!out1 || (w1 && b1), "layernorm_sum: the norm needs weight and bias");
    PTA_REQUIRE(!out2 || (out1 && w2 && b2), "layernorm_sum: a second output needs the first, and its own weight and bias");
    PTA_REQUIRE(rows || M == M_in, "layernorm_sum: without row selection M (%d) must equal M_in (%d)", M, M_in);
    const void* ptrs[] = {out_x, out1, out2, pa, pb, add1, add2, add3, bias_a, bias_b, w1, b1, w2, b2};
    for (const void* p : ptrs) PTA_REQUIRE(((uintptr_t)p % 16) == 0, "layernorm_sum: pointers must be 16-byte aligned");
    // Many rows of plain tensors: a wave per row.  Measured at 2,048 rows of 4,544 against a workgroup per row:
    // 18 us against 27.  The two kernels add a row's squares in different orders, so a row's norm may differ in its
    // last bit between a prompt and a decode step, as their matrix products already do.
    if (!pa && !pb && !rows && add1 && M >= NS_ROWS_MIN) {
        const int per_lane = (H / 8 + 63) / 64;
        hipStream_t s = (hipStream_t)stream;
        if (per_lane <= 4) launch_rows<4>(out_x, out1, out2, add1, add2, add3, w1, b1, w2, b2, M, H, eps, s);
        else if (per_lane <= 9) launch_rows<9>(out_x, out1, out2, add1, add2, add3, w1, b1, w2, b2, M, H, eps, s);
        else launch_rows<16>(out_x, out1, out2, add1, add2, add3, w1, b1, w2, b2, M, H, eps, s);
        return pta_check_launch("layernorm_sum");
    }
    // A decode step's usual sum (a first product of up to 16 ranges, a second of up to 4, tensors): every load at once,
    // or of 13 to 16 ranges twelve at once and the rest behind them (16 at once, 168 registers and some spilled, took
    // 11.3 us where one range after the other takes 9.1).
    static const bool ahead = !getenv("PTA_NORM_AHEAD") || atoi(getenv("PTA_NORM_AHEAD")) != 0;
    const int threads = (H / 8 + 63) / 64 * 64;
    constexpr int WIDE_THREADS = 640;  // rows of up to 5,120 features
    if (ahead && pb && (Pb <= 8 || (Pb <= 16 && threads <= WIDE_THREADS)) && (!pa || Pa <= 4) && H <= NS_MAX_H) {
        auto kern = pa ? layernorm_sum_ahead_kernel<8, 4> : layernorm_sum_ahead_kernel<8, 1>;
        if (Pb > 12) kern = pa ? layernorm_sum_ahead_kernel<16, 4, WIDE_THREADS> : layernorm_sum_ahead_kernel<16, 1, WIDE_THREADS>;
        else if (Pb > 8) kern = pa ? layernorm_sum_ahead_kernel<12, 4, WIDE_THREADS> : layernorm_sum_ahead_kernel<12, 1, WIDE_THREADS>;
        hipLaunchKernelGGL(kern, dim3(M), dim3(threads), 0, (hipStream_t)stream,
                           (bf16_t*)out_x, (bf16_t*)out1, (bf16_t*)out2, pa, Pa, bias_a, pb, Pb, bias_b, (const bf16_t*)add1,
                           (const bf16_t*)add2, (const bf16_t*)add3, rows, w1, b1, w2, b2, M_in, H, eps);
        return pta_check_launch("layernorm_sum");
    }
    // One chunk per thread for every row count.  Measured at 2,048 rows of 4,544: 1 chunk 26 us, 2 chunks 34 us,
    // 4 chunks 26 us; and with one choice a row's norm has the same bits in a prompt and in a decode step.
    const int chunks = H / 8;
    hipLaunchKernelGGL(layernorm_sum_kernel<1>, dim3(M), dim3((chunks + 63) / 64 * 64), 0, (hipStream_t)stream,
                       (bf16_t*)out_x, (bf16_t*)out1, (bf16_t*)out2, pa, Pa, bias_a, pb, Pb, bias_b, (const bf16_t*)add1,
                       (const bf16_t*)add2, (const bf16_t*)add3, rows, w1, b1, w2, b2, M_in, H, eps);
    return pta_check_launch("layernorm_sum");
}
