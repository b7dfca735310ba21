// y = x @ W^T for many rows, bfloat16 in, fp32 accumulate, fp32 or bfloat16 out: a tiled MFMA
// product. Layout of the reference's F.linear (rollout/monkey_patch/qwen3.py:21): x [M, K],
// W [N, K], y [M, N]. It serves where the library has nothing to offer (fp32 results from
// bf16 operands, as the output head needs for more than 64 rows) and stands beside the
// library for bf16 results.
//
// Workgroup tile 128 x 128, k-step 32, four waves as 2 x 2, each wave 64 x 64 as 4 x 4 MFMA
// 16x16x32 bf16 tiles. Both operands are contraction-major in memory, so a lane's MFMA operand
// (row r, k = 8g .. 8g+7) is one 16-byte piece of a row; tiles are staged in LDS with rows padded
// by 16 bytes, two buffers, the next k-step travelling through registers while this one is used.
// Needs K % 8 == 0; M, N arbitrary (edges are clamped on load and masked on store).
#include "common.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef uint32_t uint4_t __attribute__((ext_vector_type(4)));

#define GM_BM 128
#define GM_BN 128
#define GM_BK 32
#define GM_LD (GM_BK + 8)        // LDS row stride in elements

template <typename TO>
__global__ __launch_bounds__(256) void gemm_mfma_kernel(const bf16* __restrict__ A,
                                                        const bf16* __restrict__ W,
                                                        TO* __restrict__ C, int M, int N, int K) {
    __shared__ __attribute__((aligned(16))) uint16_t a_s[2][GM_BM * GM_LD];
    __shared__ __attribute__((aligned(16))) uint16_t w_s[2][GM_BN * GM_LD];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, n = lane & 15, g = lane >> 4;
    const int wm = wave >> 1, wn = wave & 1;                 // this wave's 64 x 64 quadrant
    const int m0 = blockIdx.y * GM_BM, n0 = blockIdx.x * GM_BN;

    // staging: 128 rows x 4 pieces of 16 bytes per operand; a thread moves 2 pieces of each
    const int ld_row = tid >> 1, ld_p = (tid & 1) * 2;       // pieces ld_p, ld_p + 1 of row ld_row
    const bf16* a_src = A + (size_t)min(m0 + ld_row, M - 1) * K + ld_p * 8;
    const bf16* w_src = W + (size_t)min(n0 + ld_row, N - 1) * K + ld_p * 8;
    const uint4_t zero = {0u, 0u, 0u, 0u};
    uint4_t ar[2], wr[2];

    float4_t acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = float4_t{0.f, 0.f, 0.f, 0.f};

#define GM_FETCH(k0_)                                                                        \
    _Pragma("unroll") for (int p = 0; p < 2; ++p) {                                          \
        const bool in_ = (k0_) + (ld_p + p) * 8 < K;                                         \
        ar[p] = in_ ? *reinterpret_cast<const uint4_t*>(a_src + (k0_) + p * 8) : zero;       \
        wr[p] = in_ ? *reinterpret_cast<const uint4_t*>(w_src + (k0_) + p * 8) : zero;       \
    }
#define GM_STAGE(buf_)                                                                       \
    _Pragma("unroll") for (int p = 0; p < 2; ++p) {                                          \
        *reinterpret_cast<uint4_t*>(&a_s[buf_][ld_row * GM_LD + (ld_p + p) * 8]) = ar[p];    \
        *reinterpret_cast<uint4_t*>(&w_s[buf_][ld_row * GM_LD + (ld_p + p) * 8]) = wr[p];    \
    }

    GM_FETCH(0)
    GM_STAGE(0)
    if (GM_BK < K) { GM_FETCH(GM_BK) }
    __syncthreads();

    int it = 0;
    for (int k0 = 0; k0 < K; k0 += GM_BK, ++it) {
        const int cur = it & 1;
        if (k0 + GM_BK < K) {
            GM_STAGE(cur ^ 1)
            if (k0 + 2 * GM_BK < K) { GM_FETCH(k0 + 2 * GM_BK) }
        }
        bf16x8_t af[4], wf[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            af[i] = *reinterpret_cast<const bf16x8_t*>(&a_s[cur][(wm * 64 + i * 16 + n) * GM_LD + 8 * g]);
            wf[i] = *reinterpret_cast<const bf16x8_t*>(&w_s[cur][(wn * 64 + i * 16 + n) * GM_LD + 8 * g]);
        }
        // W rows are the A operand (result rows = columns of y), x rows the B operand:
        // acc[i][j][e] = y[m = m0 + wm*64 + j*16 + n][col = n0 + wn*64 + i*16 + 4g + e]
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[i], af[j], acc[i][j], 0, 0, 0);
        __syncthreads();
    }
#undef GM_FETCH
#undef GM_STAGE
    MFMA_SETTLE();
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int m = m0 + wm * 64 + j * 16 + n;
        if (m >= M) continue;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int col = n0 + wn * 64 + i * 16 + 4 * g;
            TO* dst = C + (size_t)m * N + col;
            if (col + 3 < N && (N & 3) == 0) {
                if constexpr (sizeof(TO) == 4) {
                    *reinterpret_cast<float4_t*>(dst) = acc[i][j];
                } else {
                    uint2 w;
                    w.x = (uint32_t)f2bf_bits(acc[i][j][0]) | ((uint32_t)f2bf_bits(acc[i][j][1]) << 16);
                    w.y = (uint32_t)f2bf_bits(acc[i][j][2]) | ((uint32_t)f2bf_bits(acc[i][j][3]) << 16);
                    *reinterpret_cast<uint2*>(dst) = w;
                }
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (col + e < N) dst[e] = from_f<TO>(acc[i][j][e]);
            }
        }
    }
}

extern "C" int ra_gemm_tile_bf16(const void* X, const void* W, void* C, int M, int N, int K, int splits,
                                 int out_dtype, void* stream);

// More than 128 rows go to the product with tiles of 256 x 256 (gemm_tile.hip) where it takes the sizes
// and has at least 160 tiles to spread over the CUs (2,048 x 4,096 are 128 tiles: there the small tiles
// are as fast or faster).
extern "C" int ra_gemm_mfma_bf16(const void* A, const void* W, void* C, int M, int N, int K,
                                 int out_dtype, void* stream) {
    if (M <= 0 || N <= 0) return RA_OK;
    if (K <= 0 || K % 8 != 0) return RA_ERR_ARG;
    if (M > GM_BM && K % 32 == 0 && (size_t)M * K * 2 <= 0x7fffffffull && (size_t)N * K * 2 <= 0x7fffffffull &&
        (long long)((M + 255) / 256) * ((N + 255) / 256) >= 160)
        return ra_gemm_tile_bf16(A, W, C, M, N, K, 1, out_dtype, stream);
    dim3 grid((N + GM_BN - 1) / GM_BN, (M + GM_BM - 1) / GM_BM), block(256);
    if (grid.y > 65535) return RA_ERR_ARG;
    hipStream_t st = (hipStream_t)stream;
    if (out_dtype == RA_DTYPE_F32)
        hipLaunchKernelGGL(gemm_mfma_kernel<float>, grid, block, 0, st, (const bf16*)A,
                           (const bf16*)W, (float*)C, M, N, K);
    else if (out_dtype == RA_DTYPE_BF16)
        hipLaunchKernelGGL(gemm_mfma_kernel<bf16>, grid, block, 0, st, (const bf16*)A,
                           (const bf16*)W, (bf16*)C, M, N, K);
    else
        return RA_ERR_ARG;
    return ra_launch_status();
}
