// y = x @ W^T for row-major x [M, K] and W [N, K] (the nn.Linear layout of the reference,
// rollout/monkey_patch/qwen3.py:21). This file holds the plain tiled kernel: products and
// sums in true 32-bit FMA, K walked in order, so a row's result does not depend on M.
// It is the only matrix product of the float32 path and the fallback of the bfloat16 path.
#include "common.h"

#define BM 64
#define BN 64
#define BK 16

template <typename TI, typename TO>
__global__ __launch_bounds__(256) void gemm_nt_kernel(const TI* __restrict__ A,
                                                      const TI* __restrict__ W,
                                                      TO* __restrict__ C, int M, int N, int K) {
    __shared__ float As[BK][BM + 4];
    __shared__ float Ws[BK][BN + 4];
    const int tid = threadIdx.x;
    const int tx = tid & 15, ty = tid >> 4;
    const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    const int lr = tid >> 2;            // 0..63: row of the tile this thread loads
    const int lk = (tid & 3) * 4;       // 0,4,8,12: first of its 4 k
    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

    for (int k0 = 0; k0 < K; k0 += BK) {
        {
            const int m = m0 + lr;
            const TI* p = A + (size_t)m * K + k0 + lk;
#pragma unroll
            for (int i = 0; i < 4; ++i)
                As[lk + i][lr] = (m < M && k0 + lk + i < K) ? to_f(p[i]) : 0.f;
            const int n = n0 + lr;
            const TI* q = W + (size_t)n * K + k0 + lk;
#pragma unroll
            for (int i = 0; i < 4; ++i)
                Ws[lk + i][lr] = (n < N && k0 + lk + i < K) ? to_f(q[i]) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < BK; ++k) {
            float a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = As[k][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) b[j] = Ws[k][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = m0 + ty * 4 + i;
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx * 4 + j;
            if (n < N) C[(size_t)m * N + n] = from_f<TO>(acc[i][j]);
        }
    }
}

// in_dtype / out_dtype: RA_DTYPE_F32 or RA_DTYPE_BF16 (x and W share in_dtype)
extern "C" int ra_gemm_nt(const void* A, const void* W, void* C, int M, int N, int K, int in_dtype,
                          int out_dtype, void* stream) {
    if (M <= 0 || N <= 0) return RA_OK;
    if (K <= 0) return RA_ERR_ARG;
    dim3 block(256), grid((N + BN - 1) / BN, (M + BM - 1) / BM);
    hipStream_t s = (hipStream_t)stream;
    if (in_dtype == RA_DTYPE_F32 && out_dtype == RA_DTYPE_F32)
        hipLaunchKernelGGL((gemm_nt_kernel<float, float>), grid, block, 0, s, (const float*)A,
                           (const float*)W, (float*)C, M, N, K);
    else if (in_dtype == RA_DTYPE_BF16 && out_dtype == RA_DTYPE_BF16)
        hipLaunchKernelGGL((gemm_nt_kernel<bf16, bf16>), grid, block, 0, s, (const bf16*)A,
                           (const bf16*)W, (bf16*)C, M, N, K);
    else if (in_dtype == RA_DTYPE_BF16 && out_dtype == RA_DTYPE_F32)
        hipLaunchKernelGGL((gemm_nt_kernel<bf16, float>), grid, block, 0, s, (const bf16*)A,
                           (const bf16*)W, (float*)C, M, N, K);
    else
        return RA_ERR_ARG;
    return ra_launch_status();
}
