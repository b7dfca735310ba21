// y = x @ W^T for few rows of x (M <= 64), bfloat16 in, fp32 accumulate: the decode-time
// matrix product, bound by streaming W once from HBM. Layout as in the reference's
// F.linear (rollout/monkey_patch/qwen3.py:21): x [M, K], W [N, K], y [M, N].
//
// A workgroup takes 16 rows of W at a time; its waves split K in blocks of 256 elements.
// W is the A operand of MFMA 16x16x32 bf16: lane (n, g) loads 16 contiguous bytes of row n
// at k = k0 + 8g, which is exactly its operand; x is the B operand, loaded the same way from
// row m = lane % 16 (x is small and stays in cache). The contraction does not care how k is
// distributed over lanes as long as both operands agree. Partial tiles of the waves are
// added through LDS in wave order, so the result does not depend on scheduling.
// Needs K % 8 == 0 (16-byte loads); other K go to the plain kernel.
//
// GATED: W is [2I, K] with the gate rows first (rollout/monkey_patch/qwen3.py:103); a tile
// takes 16 gate rows and the 16 up rows that belong to them and writes silu(g) * u
// (rollout/fused.py:103-114) as [M, I], so the [M, 2I] intermediate never reaches memory.
#include "common.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));

#define SK_UNROLL 8                      // MFMA steps (of 32 k) per wave iteration
#define SK_KB (32 * SK_UNROLL)           // k elements per wave iteration

template <int WAVES, int MB, typename TO, bool GATED>
__global__ __launch_bounds__(WAVES * 64) void gemm_skinny_kernel(
    const bf16* __restrict__ x, const bf16* __restrict__ W, TO* __restrict__ out, int M, int N,
    int K, int n_tiles) {
    // N: rows of the result (= rows of W, or half of them when GATED)
    constexpr int NG = GATED ? 2 : 1;
    __shared__ float red[WAVES][NG][MB][16][17];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int n = lane & 15, g = lane >> 4;
    const bf16x8_t zero = {0, 0, 0, 0, 0, 0, 0, 0};

    for (int tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
        const int n0 = tile * 16;
        const int row = min(n0 + n, N - 1);                 // clamped: loads stay inside W
        const bf16* wp = W + (size_t)row * K + g * 8;
        const bf16* wp_up = wp + (size_t)N * K;               // GATED: the up row of the same column
        const bf16* xp[MB];
        bool x_ok[MB];
#pragma unroll
        for (int b = 0; b < MB; ++b) {
            const int m = b * 16 + n;
            x_ok[b] = m < M;
            xp[b] = x + (size_t)min(m, M - 1) * K + g * 8;
        }
        float4_t c[NG][MB];
#pragma unroll
        for (int z = 0; z < NG; ++z)
#pragma unroll
            for (int b = 0; b < MB; ++b) c[z][b] = float4_t{0.f, 0.f, 0.f, 0.f};

        for (int kb = wave * SK_KB; kb < K; kb += WAVES * SK_KB) {
            bf16x8_t a[NG][SK_UNROLL];
            bf16x8_t bx[MB][SK_UNROLL];
#pragma unroll
            for (int u = 0; u < SK_UNROLL; ++u) {
                const int k = kb + u * 32;
                const bool in = k + g * 8 < K;               // K % 8 == 0: a lane's 8 are in or out together
                a[0][u] = in ? *reinterpret_cast<const bf16x8_t*>(wp + k) : zero;
                if constexpr (GATED) a[1][u] = in ? *reinterpret_cast<const bf16x8_t*>(wp_up + k) : zero;
#pragma unroll
                for (int b = 0; b < MB; ++b)
                    bx[b][u] = (in && x_ok[b]) ? *reinterpret_cast<const bf16x8_t*>(xp[b] + k) : zero;
            }
#pragma unroll
            for (int u = 0; u < SK_UNROLL; ++u)
#pragma unroll
                for (int b = 0; b < MB; ++b)
#pragma unroll
                    for (int z = 0; z < NG; ++z)
                        c[z][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[z][u], bx[b][u], c[z][b], 0, 0, 0);
        }
        MFMA_SETTLE();
        // c[z][b][i] = partial y[m = 16b + n][row n0 + 4g + i]
#pragma unroll
        for (int z = 0; z < NG; ++z)
#pragma unroll
            for (int b = 0; b < MB; ++b)
#pragma unroll
                for (int i = 0; i < 4; ++i) red[wave][z][b][4 * g + i][n] = c[z][b][i];
        __syncthreads();
        for (int e = threadIdx.x; e < MB * 256; e += WAVES * 64) {
            const int b = e >> 8, mm = (e >> 4) & 15, r = e & 15;     // r fastest: neighbours write neighbours
            const int m = b * 16 + mm, col = n0 + r;
            if (m < M && col < N) {
                float s = 0.f;
#pragma unroll
                for (int w = 0; w < WAVES; ++w) s += red[w][0][b][r][mm];
                if constexpr (GATED) {
                    float u = 0.f;
#pragma unroll
                    for (int w = 0; w < WAVES; ++w) u += red[w][1][b][r][mm];
                    s = s / (1.0f + expf(-s)) * u;        // gate and up stay 32-bit until here
                }
                out[(size_t)m * N + col] = from_f<TO>(s);
            }
        }
        __syncthreads();
    }
}

template <int WAVES, int MB, typename TO, bool GATED>
static void launch_skinny(int grid, hipStream_t st, const bf16* x, const bf16* W, TO* out, int M,
                          int N, int K, int n_tiles) {
    hipLaunchKernelGGL((gemm_skinny_kernel<WAVES, MB, TO, GATED>), dim3(grid), dim3(WAVES * 64), 0,
                       st, x, W, out, M, N, K, n_tiles);
}

template <int WAVES, typename TO>
static int pick_mb(int grid, hipStream_t st, const bf16* x, const bf16* W, TO* out, int M, int N,
                   int K, int n_tiles) {
    switch ((M + 15) / 16) {
        case 1: launch_skinny<WAVES, 1, TO, false>(grid, st, x, W, out, M, N, K, n_tiles); break;
        case 2: launch_skinny<WAVES, 2, TO, false>(grid, st, x, W, out, M, N, K, n_tiles); break;
        case 3: launch_skinny<WAVES, 3, TO, false>(grid, st, x, W, out, M, N, K, n_tiles); break;
        case 4: launch_skinny<WAVES, 4, TO, false>(grid, st, x, W, out, M, N, K, n_tiles); break;
        default: return RA_ERR_ARG;
    }
    return RA_OK;
}

extern "C" int ra_gemm_skinny_bf16(const void* x, const void* W, void* out, int M, int N, int K,
                                   int out_dtype, int max_grid, void* stream) {
    if (M <= 0 || N <= 0) return RA_OK;
    if (M > 64 || K <= 0 || K % 8 != 0) return RA_ERR_ARG;
    const int n_tiles = (N + 15) / 16;
    hipStream_t st = (hipStream_t)stream;
    const bf16* xx = (const bf16*)x;
    const bf16* ww = (const bf16*)W;
    int rc;
    if (n_tiles <= 1024) {                       // few tiles: more waves per tile keep more bytes in flight
        const int grid = n_tiles;
        rc = out_dtype == RA_DTYPE_F32 ? pick_mb<8, float>(grid, st, xx, ww, (float*)out, M, N, K, n_tiles)
                                       : pick_mb<8, bf16>(grid, st, xx, ww, (bf16*)out, M, N, K, n_tiles);
    } else {
        const int grid = max_grid > 0 ? min(n_tiles, max_grid) : n_tiles;
        rc = out_dtype == RA_DTYPE_F32 ? pick_mb<4, float>(grid, st, xx, ww, (float*)out, M, N, K, n_tiles)
                                       : pick_mb<4, bf16>(grid, st, xx, ww, (bf16*)out, M, N, K, n_tiles);
    }
    if (rc != RA_OK) return rc;
    return ra_launch_status();
}

// out [M, I] = silu(x @ Wg^T) * (x @ Wu^T) for W = [Wg; Wu] of shape [2I, K]; M <= 16.
extern "C" int ra_gemm_skinny_gated_bf16(const void* x, const void* W, void* out, int M, int I, int K,
                                         void* stream) {
    if (M <= 0 || I <= 0) return RA_OK;
    if (M > 16 || K <= 0 || K % 8 != 0) return RA_ERR_ARG;
    const int n_tiles = (I + 15) / 16;
    hipStream_t st = (hipStream_t)stream;
    if (n_tiles <= 512)
        launch_skinny<8, 1, bf16, true>(n_tiles, st, (const bf16*)x, (const bf16*)W, (bf16*)out, M, I, K, n_tiles);
    else
        launch_skinny<4, 1, bf16, true>(n_tiles, st, (const bf16*)x, (const bf16*)W, (bf16*)out, M, I, K, n_tiles);
    return ra_launch_status();
}
