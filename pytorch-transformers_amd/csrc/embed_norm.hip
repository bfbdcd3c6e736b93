// Embedding lookup and LayerNorm for gfx950.
//
// LayerNorm: one workgroup per row, statistics in 32-bit, two passes over the
// row for the variance (mean first, then squared distances), so the result
// does not depend on which other rows are in the launch.  One pass over x can
// feed two affine outputs (the ln_attn / ln_mlp pair of the parallel block),
// and rows can be gathered by index (the final norm runs on wanted rows only).
#include "common.h"
#include "pta_kernels.h"

template <typename T>
__global__ void embed_kernel(T* __restrict__ out, const T* __restrict__ table, const int* __restrict__ ids,
                             int H) {
    const int m = blockIdx.x;
    const long row = ids[m];
    const T* src = table + row * (long)H;
    T* dst = out + (long)m * H;
    for (int i = threadIdx.x; i < H; i += blockDim.x) dst[i] = src[i];
}

extern "C" int pta_embed(void* out, const void* table, const int* ids, int M, int H, int dtype, void* stream) {
    PTA_REQUIRE(M > 0 && H > 0, "embed: M=%d H=%d must be positive", M, H);
    hipStream_t s = (hipStream_t)stream;
    if (dtype == PTA_F32)
        hipLaunchKernelGGL(embed_kernel<float>, dim3(M), dim3(256), 0, s, (float*)out, (const float*)table, ids, H);
    else if (dtype == PTA_BF16)
        hipLaunchKernelGGL(embed_kernel<bf16_t>, dim3(M), dim3(256), 0, s, (bf16_t*)out, (const bf16_t*)table, ids, H);
    else
        return pta_fail("embed: unknown dtype %d", dtype);
    return pta_check_launch("embed");
}

// y = (x - mean) / sqrt(var + eps) * w + b, biased variance (torch.nn.LayerNorm as built at
// src/transformers/models/falcon/modeling_falcon.py:603-612, :843).  w and b are 32-bit.
template <typename T>
__global__ void layernorm_kernel(T* __restrict__ out1, T* __restrict__ out2, const T* __restrict__ x,
                                 const int* __restrict__ rows, const float* __restrict__ w1,
                                 const float* __restrict__ b1, const float* __restrict__ w2,
                                 const float* __restrict__ b2, int H, float eps) {
    __shared__ float red[16];
    const int m = blockIdx.x;
    const long src_row = rows ? (long)rows[m] : (long)m;
    const T* xr = x + src_row * H;
    float s = 0.f;
    for (int i = threadIdx.x; i < H; i += blockDim.x) s += Io<T>::ld(xr + i);
    const float mean = block_sum(s, red) / (float)H;
    float q = 0.f;
    for (int i = threadIdx.x; i < H; i += blockDim.x) {
        const float d = Io<T>::ld(xr + i) - mean;
        q += d * d;
    }
    const float var = block_sum(q, red) / (float)H;
    const float rstd = 1.0f / sqrtf(var + eps);
    T* o1 = out1 + (long)m * H;
    T* o2 = out2 ? out2 + (long)m * H : nullptr;
    for (int i = threadIdx.x; i < H; i += blockDim.x) {
        const float n = (Io<T>::ld(xr + i) - mean) * rstd;
        Io<T>::st(o1 + i, n * w1[i] + b1[i]);
        if (o2) Io<T>::st(o2 + i, n * w2[i] + b2[i]);
    }
}

// The same, for rows of at most LN_THREADS * LN_VPT features: the row is read once and held in
// registers, in the same thread-strided order, so the statistics are the same bits as above.
#define LN_THREADS 512
#define LN_VPT 16
template <typename T>
__global__ __launch_bounds__(LN_THREADS) void layernorm_reg_kernel(
    T* __restrict__ out1, T* __restrict__ out2, const T* __restrict__ x, const int* __restrict__ rows,
    const float* __restrict__ w1, const float* __restrict__ b1, const float* __restrict__ w2,
    const float* __restrict__ b2, int H, float eps) {
    __shared__ float red[16];
    const int m = blockIdx.x;
    const long src_row = rows ? (long)rows[m] : (long)m;
    const T* xr = x + src_row * H;
    float xv[LN_VPT];
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < LN_VPT; ++j) {
        const int i = threadIdx.x + j * LN_THREADS;
        xv[j] = i < H ? Io<T>::ld(xr + i) : 0.f;
        if (i < H) s += xv[j];
    }
    const float mean = block_sum(s, red) / (float)H;
    float q = 0.f;
#pragma unroll
    for (int j = 0; j < LN_VPT; ++j) {
        const int i = threadIdx.x + j * LN_THREADS;
        if (i < H) { const float d = xv[j] - mean; q += d * d; }
    }
    const float var = block_sum(q, red) / (float)H;
    const float rstd = 1.0f / sqrtf(var + eps);
    T* o1 = out1 + (long)m * H;
    T* o2 = out2 ? out2 + (long)m * H : nullptr;
#pragma unroll
    for (int j = 0; j < LN_VPT; ++j) {
        const int i = threadIdx.x + j * LN_THREADS;
        if (i < H) {
            const float n = (xv[j] - mean) * rstd;
            Io<T>::st(o1 + i, n * w1[i] + b1[i]);
            if (o2) Io<T>::st(o2 + i, n * w2[i] + b2[i]);
        }
    }
}

extern "C" int pta_layernorm(void* out1, void* out2, const void* x, const int* rows, const float* w1,
                             const float* b1, const float* w2, const float* b2, int M, int H, float eps,
                             int dtype, void* stream) {
    PTA_REQUIRE(M > 0 && H > 0, "layernorm: M=%d H=%d must be positive", M, H);
    PTA_REQUIRE(out1 && x && w1 && b1, "layernorm: null pointer");
    PTA_REQUIRE(!out2 || (w2 && b2), "layernorm: a second output needs its own weight and bias");
    hipStream_t s = (hipStream_t)stream;
    const bool in_regs = H > 1024 && H <= LN_THREADS * LN_VPT;
    const int threads = H >= 2048 ? 512 : 256;
    if (dtype != PTA_F32 && dtype != PTA_BF16) return pta_fail("layernorm: unknown dtype %d", dtype);
    if (in_regs && dtype == PTA_F32)
        hipLaunchKernelGGL(layernorm_reg_kernel<float>, dim3(M), dim3(LN_THREADS), 0, s, (float*)out1, (float*)out2,
                           (const float*)x, rows, w1, b1, w2, b2, H, eps);
    else if (in_regs)
        hipLaunchKernelGGL(layernorm_reg_kernel<bf16_t>, dim3(M), dim3(LN_THREADS), 0, s, (bf16_t*)out1, (bf16_t*)out2,
                           (const bf16_t*)x, rows, w1, b1, w2, b2, H, eps);
    else if (dtype == PTA_F32)
        hipLaunchKernelGGL(layernorm_kernel<float>, dim3(M), dim3(threads), 0, s, (float*)out1, (float*)out2,
                           (const float*)x, rows, w1, b1, w2, b2, H, eps);
    else
        hipLaunchKernelGGL(layernorm_kernel<bf16_t>, dim3(M), dim3(threads), 0, s, (bf16_t*)out1, (bf16_t*)out2,
                           (const bf16_t*)x, rows, w1, b1, w2, b2, H, eps);
    return pta_check_launch("layernorm");
}

// In place on y [M, N] (rows ld apart): y = act(round(y + bias)) + add1 + add2, the part of a linear layer
// that follows a library matrix product.  The reference adds the bias as an op of its own, so
// the sum is rounded to the storage type before the activation
// (src/transformers/models/falcon/modeling_falcon.py:67-72).
template <typename T>
__global__ void epilogue_kernel(T* __restrict__ y, const float* __restrict__ bias, const T* __restrict__ add1,
                                const T* __restrict__ add2, long total, int N, long ld, int act) {
    const long stride = (long)gridDim.x * blockDim.x;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
        T* at = y + (i / N) * ld + i % N;
        float v = Io<T>::ld(at);
        if (bias) v = Io<T>::round(v + bias[i % N]);
        if (act) v = apply_act(v, act);
        if (add1) v += Io<T>::ld(add1 + i);
        if (add2) v += Io<T>::ld(add2 + i);
        Io<T>::st(at, v);
    }
}

// The same on bfloat16 rows whose length is a multiple of 8: sixteen bytes per thread and access.
__global__ void epilogue_bf16x8_kernel(bf16_t* __restrict__ y, const float* __restrict__ bias,
                                       const bf16_t* __restrict__ add1, const bf16_t* __restrict__ add2, long groups,
                                       int N, long ld, int act) {
    const long stride = (long)gridDim.x * blockDim.x;
    for (long gi = (long)blockIdx.x * blockDim.x + threadIdx.x; gi < groups; gi += stride) {
        const long i = gi * 8;
        const int n = (int)(i % N);
        bf16_t* at = y + (i / N) * ld + n;
        uint4 yv = *reinterpret_cast<const uint4*>(at);
        uint4 a1 = add1 ? *reinterpret_cast<const uint4*>(add1 + i) : make_uint4(0u, 0u, 0u, 0u);
        uint4 a2 = add2 ? *reinterpret_cast<const uint4*>(add2 + i) : make_uint4(0u, 0u, 0u, 0u);
        uint32_t* yw = reinterpret_cast<uint32_t*>(&yv);
        const uint32_t* w1 = reinterpret_cast<const uint32_t*>(&a1);
        const uint32_t* w2 = reinterpret_cast<const uint32_t*>(&a2);
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            float v[2] = {bf16_bits_to_f32((bf16_t)(yw[p] & 0xffffu)), bf16_bits_to_f32((bf16_t)(yw[p] >> 16))};
            const float x1[2] = {bf16_bits_to_f32((bf16_t)(w1[p] & 0xffffu)), bf16_bits_to_f32((bf16_t)(w1[p] >> 16))};
            const float x2[2] = {bf16_bits_to_f32((bf16_t)(w2[p] & 0xffffu)), bf16_bits_to_f32((bf16_t)(w2[p] >> 16))};
#pragma unroll
            for (int e = 0; e < 2; ++e) {
                if (bias) v[e] = round_to_bf16(v[e] + bias[n + 2 * p + e]);
                if (act) v[e] = apply_act(v[e], act);
                v[e] += x1[e];  // an absent addend was loaded as zeros
                v[e] += x2[e];
            }
            yw[p] = (uint32_t)f32_to_bf16_bits(v[0]) | ((uint32_t)f32_to_bf16_bits(v[1]) << 16);
        }
        *reinterpret_cast<uint4*>(at) = yv;
    }
}

extern "C" int pta_epilogue(void* y, int ld_y, const float* bias, const void* add1, const void* add2, int M, int N,
                            int act, int dtype, void* stream) {
    PTA_REQUIRE(M > 0 && N > 0, "epilogue: M=%d N=%d must be positive", M, N);
    PTA_REQUIRE(ld_y >= N, "epilogue: rows of %d elements cannot lie %d apart", N, ld_y);
    PTA_REQUIRE(pta_act_known(act), "epilogue: unknown activation %d", act);
    if (dtype == PTA_BF16 && N % 8 == 0 && ld_y % 8 == 0 && ((uintptr_t)y % 16) == 0 && ((uintptr_t)add1 % 16) == 0 &&
        ((uintptr_t)add2 % 16) == 0) {
        const long groups = (long)M * N / 8;
        long nb = (groups + 255) / 256;
        if (nb > 16384) nb = 16384;
        hipLaunchKernelGGL(epilogue_bf16x8_kernel, dim3((unsigned)nb), dim3(256), 0, (hipStream_t)stream, (bf16_t*)y, bias,
                           (const bf16_t*)add1, (const bf16_t*)add2, groups, N, ld_y, act);
        return pta_check_launch("epilogue");
    }
    const long total = (long)M * N;
    long blocks = (total + 255) / 256;
    if (blocks > 65536) blocks = 65536;
    hipStream_t s = (hipStream_t)stream;
    if (dtype == PTA_F32)
        hipLaunchKernelGGL(epilogue_kernel<float>, dim3((unsigned)blocks), dim3(256), 0, s, (float*)y, bias,
                           (const float*)add1, (const float*)add2, total, N, ld_y, act);
    else if (dtype == PTA_BF16)
        hipLaunchKernelGGL(epilogue_kernel<bf16_t>, dim3((unsigned)blocks), dim3(256), 0, s, (bf16_t*)y, bias,
                           (const bf16_t*)add1, (const bf16_t*)add2, total, N, ld_y, act);
    else
        return pta_fail("epilogue: unknown dtype %d", dtype);
    return pta_check_launch("epilogue");
}
