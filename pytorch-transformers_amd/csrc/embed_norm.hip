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

// The same on bfloat16 rows whose length is a multiple of 8: sixteen bytes per thread and access.  A thread has
// one group of eight columns in EPI_ROWS rows, so four loads of y are in flight at once and no index is divided
// (one group per thread, found by dividing a 64-bit index: 37 us for 2,048 x 18,176 with GELU; this: see below).
#define EPI_ROWS 4
template <int ACT>  // the activation is fixed at compile time: a switch per element costs more than the activation
__global__ __launch_bounds__(256) void epilogue_bf16x8_kernel(bf16_t* __restrict__ y, const float* __restrict__ bias,
                                                              const bf16_t* __restrict__ add1,
                                                              const bf16_t* __restrict__ add2, int M, int N, long ld) {
    const int n = ((int)blockIdx.x * 256 + (int)threadIdx.x) * 8;
    if (n >= N) return;
    const int m0 = (int)blockIdx.y * EPI_ROWS;
    uint4 yv[EPI_ROWS], a1[EPI_ROWS], a2[EPI_ROWS];
#pragma unroll
    for (int r = 0; r < EPI_ROWS; ++r) {
        const int m = min(m0 + r, M - 1);
        yv[r] = *reinterpret_cast<const uint4*>(y + (long)m * ld + n);
        a1[r] = add1 ? *reinterpret_cast<const uint4*>(add1 + (long)m * N + n) : make_uint4(0u, 0u, 0u, 0u);
        a2[r] = add2 ? *reinterpret_cast<const uint4*>(add2 + (long)m * N + n) : make_uint4(0u, 0u, 0u, 0u);
    }
    float b[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) b[e] = bias ? bias[n + e] : 0.f;
#pragma unroll
    for (int r = 0; r < EPI_ROWS; ++r) {
        if (m0 + r >= M) break;
        float v[8], x1[8], x2[8];
        unpack8(yv[r], v);
        unpack8(a1[r], x1);
        unpack8(a2[r], x2);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            if (bias) v[e] = round_to_bf16(v[e] + b[e]);
            if (ACT != PTA_ACT_NONE) v[e] = apply_act(v[e], ACT);
            v[e] += x1[e];  // an absent addend was loaded as zeros
            v[e] += x2[e];
        }
        *reinterpret_cast<uint4*>(y + (long)(m0 + r) * ld + n) = pack8(v);
    }
}

template <int ACT>
static void launch_epilogue_x8(int act, dim3 grid, hipStream_t s, bf16_t* y, const float* bias, const bf16_t* add1,
                               const bf16_t* add2, int M, int N, long ld) {
    if constexpr (ACT < PTA_ACT_COUNT) {
        if (act == ACT)
            hipLaunchKernelGGL(epilogue_bf16x8_kernel<ACT>, grid, dim3(256), 0, s, y, bias, add1, add2, M, N, ld);
        else
            launch_epilogue_x8<ACT + 1>(act, grid, s, y, bias, add1, add2, M, N, ld);
    }
}

extern "C" int pta_epilogue(void* y, int ld_y, const float* bias, const void* add1, const void* add2, int M, int N,
                            int act, int dtype, void* stream) {
    PTA_REQUIRE(M > 0 && N > 0, "epilogue: M=%d N=%d must be positive", M, N);
    PTA_REQUIRE(ld_y >= N, "epilogue: rows of %d elements cannot lie %d apart", N, ld_y);
    PTA_REQUIRE(pta_act_known(act), "epilogue: unknown activation %d", act);
    if (dtype == PTA_BF16 && N % 8 == 0 && ld_y % 8 == 0 && ((uintptr_t)y % 16) == 0 && ((uintptr_t)add1 % 16) == 0 &&
        ((uintptr_t)add2 % 16) == 0) {
        const dim3 grid((unsigned)((N / 8 + 255) / 256), (unsigned)((M + EPI_ROWS - 1) / EPI_ROWS));
        PTA_REQUIRE(grid.y <= 65535u * 16u, "epilogue: too many rows (%d) for one launch", M);
        launch_epilogue_x8<0>(act, grid, (hipStream_t)stream, (bf16_t*)y, bias, (const bf16_t*)add1, (const bf16_t*)add2, M, N,
                              (long)ld_y);
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
