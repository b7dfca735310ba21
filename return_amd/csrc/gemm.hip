// y = x @ W^T for row-major x [M, K] and W [N, K] (the nn.Linear layout of the reference,
// rollout/monkey_patch/qwen3.py:21). This file holds the plain tiled kernel: products and
// sums in true 32-bit FMA, K walked in order, so a row's result does not depend on M.
// It is the matrix product of the float32 path and the fallback of the bfloat16 path. For up to
// 16 rows of x in float32 (decoding) there is a second kernel that streams W once with 16-byte
// loads; it sums a row's products in another order than the tiled kernel, 32-bit all the same.
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

// ------------------------------------------------------------------ few rows, float32
// y[m, n] = sum_k x[m, k] W[n, k] for M <= MR rows, all float32, K % 4 == 0. A workgroup of four
// waves takes 16 rows of W, four per wave; x goes through LDS in blocks of 512 columns for all
// four waves; a lane multiplies the four floats at k = 4 lane (+256) of its rows of W with the same
// four floats of every row of x, and the lanes' sums are added at the end (lane order, fixed).
typedef float gv_f4 __attribute__((ext_vector_type(4)));
#define GV_KC 512
template <int MR>
__global__ __launch_bounds__(256) void gemv_f32_kernel(const float* __restrict__ x, const float* __restrict__ W,
                                                       float* __restrict__ y, int M, int N, int K) {
    __shared__ __attribute__((aligned(16))) float x_s[MR][GV_KC];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int n0 = (blockIdx.x * 4 + wave) * 4;
    const float* wr[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) wr[r] = W + (size_t)min(n0 + r, N - 1) * K;      // clamped: loads stay inside W
    float acc[4][MR];
#pragma unroll
    for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int m = 0; m < MR; ++m) acc[r][m] = 0.f;
    const gv_f4 zero = {0.f, 0.f, 0.f, 0.f};
    for (int k0 = 0; k0 < K; k0 += GV_KC) {
        __syncthreads();                                     // every wave has left the last block of x
        for (int e = tid; e < MR * (GV_KC / 4); e += 256) {
            const int m = e / (GV_KC / 4), k = k0 + 4 * (e % (GV_KC / 4));
            *reinterpret_cast<gv_f4*>(&x_s[m][k - k0]) =
                (m < M && k < K) ? *reinterpret_cast<const gv_f4*>(x + (size_t)m * K + k) : zero;
        }
        __syncthreads();
#pragma unroll
        for (int h = 0; h < GV_KC / 256; ++h) {
            const int kl = 256 * h + 4 * lane, k = k0 + kl;
            gv_f4 w[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) w[r] = k < K ? *reinterpret_cast<const gv_f4*>(wr[r] + k) : zero;
#pragma unroll
            for (int m = 0; m < MR; ++m) {
                const gv_f4 xv = *reinterpret_cast<const gv_f4*>(&x_s[m][kl]);
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    acc[r][m] = fmaf(w[r][0], xv[0], acc[r][m]);
                    acc[r][m] = fmaf(w[r][1], xv[1], acc[r][m]);
                    acc[r][m] = fmaf(w[r][2], xv[2], acc[r][m]);
                    acc[r][m] = fmaf(w[r][3], xv[3], acc[r][m]);
                }
            }
        }
    }
#pragma unroll
    for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int m = 0; m < MR; ++m) {
            const float s = wave_sum(acc[r][m]);
            if (lane == 0 && m < M && n0 + r < N) y[(size_t)m * N + n0 + r] = s;
        }
}

// in_dtype / out_dtype: RA_DTYPE_F32 or RA_DTYPE_BF16 (x and W share in_dtype)
extern "C" int ra_gemm_nt(const void* A, const void* W, void* C, int M, int N, int K, int in_dtype,
                          int out_dtype, void* stream) {
    if (M <= 0 || N <= 0) return RA_OK;
    if (K <= 0) return RA_ERR_ARG;
    dim3 block(256), grid((N + BN - 1) / BN, (M + BM - 1) / BM);
    hipStream_t s = (hipStream_t)stream;
    if (in_dtype == RA_DTYPE_F32 && out_dtype == RA_DTYPE_F32 && M <= 16 && K % 4 == 0) {
        const dim3 g16((N + 15) / 16);
        const float *xa = (const float*)A, *wa = (const float*)W;
        float* ya = (float*)C;
        if (M <= 1) hipLaunchKernelGGL(gemv_f32_kernel<1>, g16, block, 0, s, xa, wa, ya, M, N, K);
        else if (M <= 2) hipLaunchKernelGGL(gemv_f32_kernel<2>, g16, block, 0, s, xa, wa, ya, M, N, K);
        else if (M <= 4) hipLaunchKernelGGL(gemv_f32_kernel<4>, g16, block, 0, s, xa, wa, ya, M, N, K);
        else if (M <= 8) hipLaunchKernelGGL(gemv_f32_kernel<8>, g16, block, 0, s, xa, wa, ya, M, N, K);
        else hipLaunchKernelGGL(gemv_f32_kernel<16>, g16, block, 0, s, xa, wa, ya, M, N, K);
        return ra_launch_status();
    }
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
