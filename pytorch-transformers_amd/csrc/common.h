// Shared device helpers for the gfx950 kernels: bfloat16 bits, typed loads and
// stores, wave and block reductions, and the error channel of the C entry points.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#define PTA_WAVE 64
#define PTA_PAGE 64  // tokens per cache page; must equal cache.paged.PAGE_SIZE

enum PtaDtype { PTA_F32 = 0, PTA_BF16 = 1 };

// orders of the rows of a fused query_key_value projection (described in rope_cache.hip)
enum PtaQkvLayout { PTA_QKV_GROUPED = 0, PTA_QKV_TAIL = 1, PTA_QKV_INTERLEAVED = 2 };

// activations of an epilogue, by the reference's names (src/transformers/activations.py:200-220)
enum PtaAct {
    PTA_ACT_NONE = 0,        // "linear"
    PTA_ACT_GELU = 1,        // "gelu", "gelu_python": the exact erf form
    PTA_ACT_GELU_TANH = 2,   // "gelu_new", "gelu_pytorch_tanh", "gelu_fast", "gelu_accurate"
    PTA_ACT_QUICK_GELU = 3,  // x * sigmoid(1.702 x)
    PTA_ACT_RELU = 4,
    PTA_ACT_RELU2 = 5,       // relu(x)^2
    PTA_ACT_RELU6 = 6,
    PTA_ACT_SILU = 7,        // "silu", "swish"
    PTA_ACT_SIGMOID = 8,
    PTA_ACT_TANH = 9,
    PTA_ACT_LEAKY_RELU = 10, // slope 0.01
    PTA_ACT_MISH = 11,       // x * tanh(softplus(x))
    PTA_ACT_GELU_10 = 12,    // exact GELU clipped to [-10, 10]
    PTA_ACT_LAPLACE = 13,    // the normal distribution function with mean 0.707107, deviation 0.282095
    PTA_ACT_COUNT = 14
};

typedef uint16_t bf16_t;  // raw bits of a bfloat16

__host__ __device__ __forceinline__ float bf16_bits_to_f32(bf16_t v) {
    union { uint32_t u; float f; } c;
    c.u = ((uint32_t)v) << 16;
    return c.f;
}

// round to nearest, ties to even; NaN stays NaN.  On the device this is gfx950's own conversion instruction
// (one for two values where the compiler can pair them); the host spells the same rounding out.
__host__ __device__ __forceinline__ bf16_t f32_to_bf16_bits(float f) {
#if defined(__HIP_DEVICE_COMPILE__)
    union { __bf16 b; bf16_t u; } c;
    c.b = (__bf16)f;
    return c.u;
#else
    union { uint32_t u; float f; } c;
    c.f = f;
    uint32_t u = c.u;
    if ((u & 0x7fffffffu) > 0x7f800000u) return (bf16_t)((u >> 16) | 0x0040u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (bf16_t)(u >> 16);
#endif
}

__host__ __device__ __forceinline__ float round_to_bf16(float f) { return bf16_bits_to_f32(f32_to_bf16_bits(f)); }

template <typename T> struct Io;
template <> struct Io<float> {
    static __device__ __forceinline__ float ld(const float* p) { return *p; }
    static __device__ __forceinline__ void st(float* p, float v) { *p = v; }
    static __device__ __forceinline__ float round(float v) { return v; }
};
template <> struct Io<bf16_t> {
    static __device__ __forceinline__ float ld(const bf16_t* p) { return bf16_bits_to_f32(*p); }
    static __device__ __forceinline__ void st(bf16_t* p, float v) { *p = f32_to_bf16_bits(v); }
    static __device__ __forceinline__ float round(float v) { return round_to_bf16(v); }
};

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}

// Sum over a block of up to 1024 threads; every thread gets the result.  `red`
// is LDS of at least 16 floats.  The order of additions depends on the block
// size only.
__device__ __forceinline__ float block_sum(float v, float* red) {
    v = wave_sum(v);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    __syncthreads();
    if (lane == 0) red[wave] = v;
    __syncthreads();
    float t = 0.f;
    for (int i = 0; i < nw; ++i) t += red[i];
    return t;
}
__device__ __forceinline__ float block_max(float v, float* red) {
    v = wave_max(v);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
    __syncthreads();
    if (lane == 0) red[wave] = v;
    __syncthreads();
    float t = red[0];
    for (int i = 1; i < nw; ++i) t = fmaxf(t, red[i]);
    return t;
}

// eight bfloat16 in sixteen bytes <-> eight floats
__device__ __forceinline__ void unpack8(const uint4& u, float (&f)[8]) {
    const uint32_t w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        f[2 * p] = bf16_bits_to_f32((bf16_t)(w[p] & 0xffffu));
        f[2 * p + 1] = bf16_bits_to_f32((bf16_t)(w[p] >> 16));
    }
}
__device__ __forceinline__ uint4 pack8(const float (&f)[8]) {
    typedef __bf16 bf16_pair __attribute__((ext_vector_type(2)));
    typedef float f32_pair __attribute__((ext_vector_type(2)));
    uint32_t w[4];
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        union { bf16_pair b; uint32_t u; } c;
        c.b = __builtin_convertvector(f32_pair{f[2 * p], f[2 * p + 1]}, bf16_pair);  // one instruction for the two
        w[p] = c.u;
    }
    return make_uint4(w[0], w[1], w[2], w[3]);
}

// exact GELU, 0.5 x (1 + erf(x / sqrt 2))  (src/transformers/activations.py:59-78)
__device__ __forceinline__ float gelu_erf(float x) { return 0.5f * x * (1.0f + erff(x * 0.70710678118654752440f)); }

// Every activation in 32-bit, rounded once by whoever stores it (src/transformers/activations.py:25-195; softplus
// with torch's threshold of 20, beyond which it is the identity).
__device__ __forceinline__ float apply_act(float x, int act) {
    switch (act) {
        case PTA_ACT_GELU: return gelu_erf(x);
        case PTA_ACT_GELU_TANH: return 0.5f * x * (1.0f + tanhf(0.79788456080286535588f * (x + 0.044715f * x * x * x)));
        case PTA_ACT_QUICK_GELU: return x / (1.0f + expf(-1.702f * x));
        case PTA_ACT_RELU: return fmaxf(x, 0.f);
        case PTA_ACT_RELU2: { const float r = fmaxf(x, 0.f); return r * r; }
        case PTA_ACT_RELU6: return fminf(fmaxf(x, 0.f), 6.f);
        case PTA_ACT_SILU: return x / (1.0f + expf(-x));
        case PTA_ACT_SIGMOID: return 1.0f / (1.0f + expf(-x));
        case PTA_ACT_TANH: return tanhf(x);
        case PTA_ACT_LEAKY_RELU: return x >= 0.f ? x : 0.01f * x;
        case PTA_ACT_MISH: return x * tanhf(x > 20.f ? x : log1pf(expf(x)));
        case PTA_ACT_GELU_10: return fminf(fmaxf(gelu_erf(x), -10.f), 10.f);
        case PTA_ACT_LAPLACE: return 0.5f * (1.0f + erff((x - 0.707107f) / (0.282095f * 1.41421356237309504880f)));
        default: return x;
    }
}

// ---- host side ---------------------------------------------------------
// Entry points return 0 on success; otherwise pta_last_error() holds the reason.
int pta_fail(const char* fmt, ...);
int pta_check_launch(const char* what);
int pta_compute_units();
static inline bool pta_act_known(int act) { return act >= 0 && act < PTA_ACT_COUNT; }

#define PTA_REQUIRE(cond, ...) \
    do { if (!(cond)) return pta_fail(__VA_ARGS__); } while (0)
