// C[M,N] = act(A[M,K] . W[N,K]^T + bias) + add1 + add2 in true 32-bit: plain FMA on
// the vector units, no matrix-core mode of reduced precision.  Every output element
// sums its K products in the order k = 0 .. K-1 in one accumulator, whatever M is and
// wherever the element lies in the grid, so a row's result is bitwise the same alone
// and in any batch.  The 32-bit path of the whole model runs its projections, MLP and
// output head through this kernel.
#include "common.h"
#include "pta_kernels.h"

#define G_BM 64
#define G_BN 64
#define G_BK 16

__global__ __launch_bounds__(256) void gemm_f32_kernel(float* __restrict__ C, const float* __restrict__ A,
                                                       const float* __restrict__ W,
                                                       const float* __restrict__ bias,
                                                       const float* __restrict__ add1,
                                                       const float* __restrict__ add2, int M, int N, int K,
                                                       int act) {
    __shared__ float As[G_BK][G_BM + 4];
    __shared__ float Ws[G_BK][G_BN + 4];
    const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
    const int m0 = blockIdx.y * G_BM, n0 = blockIdx.x * G_BN;
    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

    for (int k0 = 0; k0 < K; k0 += G_BK) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int idx = tid + i * 256;
            const int r = idx >> 4, kk = idx & 15;
            const int gk = k0 + kk;
            const int gm = m0 + r, gn = n0 + r;
            As[kk][r] = (gm < M && gk < K) ? A[(long)gm * K + gk] : 0.f;
            Ws[kk][r] = (gn < N && gk < K) ? W[(long)gn * K + gk] : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < G_BK; ++kk) {
            float a[4], w[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) { a[i] = As[kk][ty * 4 + i]; w[i] = Ws[kk][tx * 4 + i]; }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int gm = m0 + ty * 4 + i;
        if (gm >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int gn = n0 + tx * 4 + j;
            if (gn >= N) continue;
            float v = acc[i][j];
            if (bias) v += bias[gn];
            if (act) v = apply_act(v, act);
            const long o = (long)gm * N + gn;
            if (add1) v += add1[o];
            if (add2) v += add2[o];
            C[o] = v;
        }
    }
}

extern "C" int pta_gemm_f32(float* C, const float* A, const float* W, const float* bias, const float* add1,
                            const float* add2, int M, int N, int K, int act, void* stream) {
    PTA_REQUIRE(M > 0 && N > 0 && K > 0, "gemm_f32: sizes must be positive (M=%d N=%d K=%d)", M, N, K);
    PTA_REQUIRE(C && A && W, "gemm_f32: null pointer");
    PTA_REQUIRE(pta_act_known(act), "gemm_f32: unknown activation %d", act);
    const int gy = (M + G_BM - 1) / G_BM, gx = (N + G_BN - 1) / G_BN;
    PTA_REQUIRE(gy <= 65535, "gemm_f32: M=%d is too large for one launch", M);
    hipLaunchKernelGGL(gemm_f32_kernel, dim3(gx, gy), dim3(256), 0, (hipStream_t)stream, C, A, W, bias, add1, add2,
                       M, N, K, act);
    return pta_check_launch("gemm_f32");
}
