// y = x @ W^T for up to 16 rows of x (32 with K up to 4,096) with W read as one sweep through memory: the decode-time
// product of a small batch, which is bound by reading W once.
// Layout as in the reference's F.linear (rollout/monkey_patch/qwen3.py:21): x [M, K], W [N, K],
// y [M, N].
//
// One workgroup of eight waves per CU. Result column c belongs to workgroup c % gridDim, so that at
// any time the workgroups together read gridDim consecutive rows of W, one contiguous run of memory
// (measured here: such a sweep reads 201 MB in 31 µs; the same bytes as 16 rows x 512 B per wave,
// the order of an MFMA operand read straight from memory, take 35 µs). Wave w has columns
// 512w .. 512w+511 of K: a row of W is one load of 1 KB per wave, sixteen rows (a tile) are on their
// way per lane while the tile before is multiplied; a row of the next tile is asked for as soon as
// the same row of this one has arrived, so the loads on their way never run out. The tile goes through a part of LDS that is the
// wave's own (16 rows of 512 + 8 elements), from where it is read back as A operands of MFMA
// 16x16x32 bf16 (lane (n, g): 16 bytes of row n at 32j + 8g); the wave's columns of x are B operands
// that stay in registers for all tiles. The eight waves' partial tiles are added through LDS in wave
// order, as in the x-resident product.
// Results: bfloat16 or fp32 [M, N]; GATED (W = [Wg; Wu], rollout/monkey_patch/qwen3.py:103): a tile
// is 8 gate rows and the 8 up rows of the same columns, the result silu(g) * u as [M, N]
// (rollout/fused.py:103-114).
// K beyond the 4,096 columns that eight waves cover at once (gemm_sweep_long_kernel): a tile's rows
// are taken in spans of 4,096 columns, one after the other, each with its own B operands (read again
// for every tile; they come from L2).
// Needs K % 8 == 0.
#include "common.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));

#define SW_WAVES 8
#define SW_THREADS (SW_WAVES * 64)
#define SW_KW 512                         // columns of K per wave
#define SW_STRIDE (SW_KW + 8)             // row stride of a wave's tile in LDS (elements): rows shift by 4 banks
#define SW_STEPS (SW_KW / 32)             // MFMA steps per tile

// order between the LDS accesses of one wave: LDS serves a wave in order, the compiler must too
#define SW_WAVE_SYNC()                                           \
    do {                                                         \
        __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");   \
        __builtin_amdgcn_wave_barrier();                         \
    } while (0)

// MB: blocks of 16 rows of x (1 or 2)
template <int MB, bool GATED, typename TO>
__global__ __launch_bounds__(SW_THREADS) void gemm_sweep_kernel(
    const bf16* __restrict__ x, const bf16* __restrict__ W, TO* __restrict__ out, int M, int N, int K) {
    constexpr int COLS = GATED ? 8 : 16;                        // result columns of a tile
    constexpr int RS = 16 * MB + 1;                             // row stride of the waves' tiles in LDS (floats)
    constexpr bool TWO_BUFFERS = MB == 1;                       // of those tiles (LDS has room for one set with MB == 2)
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, n = lane & 15, g = lane >> 4;
    uint16_t* stage = reinterpret_cast<uint16_t*>(lds_raw) + (size_t)wave * 16 * SW_STRIDE;
    float* red_both = reinterpret_cast<float*>(lds_raw + (size_t)SW_WAVES * 16 * SW_STRIDE * 2);   // [1 or 2][wave][16 rows][RS]
    const int G = gridDim.x, b = blockIdx.x;
    const int my_cols = N > b ? (N - 1 - b) / G + 1 : 0;
    const int n_tiles = (my_cols + COLS - 1) / COLS;
    if (n_tiles == 0) return;
    const int kb = wave * SW_KW;
    const bool k_in = kb + lane * 8 < K;                        // K % 8 == 0: a lane's 8 columns are in or out together
    const bf16x8_t zero = {0, 0, 0, 0, 0, 0, 0, 0};

    // row i of tile t: column b + G (COLS t + i % COLS), GATED: rows 8.. are the up rows
    bf16x8_t wreg[16];
    auto fetch_row = [&](int t, int i) {
        const int col = b + G * (t * COLS + (GATED ? (i & 7) : i));
        const size_t row = (GATED && i >= 8) ? (size_t)N + col : (size_t)col;
        wreg[i] = (k_in && col < N) ? *reinterpret_cast<const bf16x8_t*>(W + row * K + kb + lane * 8) : zero;
    };
#pragma unroll
    for (int i = 0; i < 16; ++i) fetch_row(0, i);

    // the wave's columns of x as B operands: lane (n, g) holds x[n][kb + 32j + 8g ..], rows beyond M as zeros
    bf16x8_t bx[MB][SW_STEPS];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int j = 0; j < SW_STEPS; ++j) {
            const int k = kb + 32 * j + 8 * g, m = 16 * mb + n;
            bx[mb][j] = (m < M && k < K) ? *reinterpret_cast<const bf16x8_t*>(x + (size_t)m * K + k) : zero;
        }

    for (int t = 0; t < n_tiles; ++t) {
        SW_WAVE_SYNC();                                         // the tile before has been read out of the wave's LDS
        // row by row: as soon as a row has arrived and gone into LDS, the same row of the next tile is
        // asked for, so that the loads on their way never run out at a tile's end
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            *reinterpret_cast<bf16x8_t*>(&stage[i * SW_STRIDE + lane * 8]) = wreg[i];
            if (t + 1 < n_tiles) fetch_row(t + 1, i);
        }
        SW_WAVE_SYNC();                                         // the tile is complete in LDS
        float4_t c[MB];
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) c[mb] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int j = 0; j < SW_STEPS; ++j) {
            const bf16x8_t a = *reinterpret_cast<const bf16x8_t*>(&stage[n * SW_STRIDE + 32 * j + 8 * g]);
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) c[mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, bx[mb][j], c[mb], 0, 0, 0);
        }
        MFMA_SETTLE();
        // c[mb][i] = partial y[m = 16 mb + n][tile row 4g + i]: every wave puts its tile down, then the
        // threads add the waves' tiles in wave order. With two buffers in turn a buffer is written again
        // two tiles on, which is after the next tile's barrier, and that its readers reach only when
        // they have read; with one, a second barrier ends the tile.
        float* red = red_both + (TWO_BUFFERS ? (t & 1) * (SW_WAVES * 16 * RS) : 0);
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int i = 0; i < 4; ++i) red[(wave * 16 + 4 * g + i) * RS + 16 * mb + n] = c[mb][i];
        __syncthreads();
        if (tid < 16 * MB * COLS) {
            const int mm = tid / COLS, r = tid % COLS;        // r fastest: neighbours write neighbours' columns
            const int col = b + G * (t * COLS + r);
            if (mm < M && col < N) {
                float s = 0.f;
#pragma unroll
                for (int w = 0; w < SW_WAVES; ++w) s += red[(w * 16 + r) * RS + mm];
                if constexpr (GATED) {
                    float up = 0.f;
#pragma unroll
                    for (int w = 0; w < SW_WAVES; ++w) up += red[(w * 16 + 8 + r) * RS + mm];
                    s = s / (1.0f + expf(-s)) * up;           // gate and up stay 32-bit until here
                }
                out[(size_t)mm * N + col] = from_f<TO>(s);
            }
        }
        if constexpr (!TWO_BUFFERS) __syncthreads();
    }
}


#define SW_SPAN (SW_WAVES * SW_KW)        // columns of K that the eight waves cover at once

template <bool GATED, typename TO>
__global__ __launch_bounds__(SW_THREADS) void gemm_sweep_long_kernel(
    const bf16* __restrict__ x, const bf16* __restrict__ W, TO* __restrict__ out, int M, int N, int K) {
    constexpr int COLS = GATED ? 8 : 16;
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, n = lane & 15, g = lane >> 4;
    uint16_t* stage = reinterpret_cast<uint16_t*>(lds_raw) + (size_t)wave * 16 * SW_STRIDE;
    float* red_both = reinterpret_cast<float*>(lds_raw + (size_t)SW_WAVES * 16 * SW_STRIDE * 2);
    const int G = gridDim.x, b = blockIdx.x;
    const int my_cols = N > b ? (N - 1 - b) / G + 1 : 0;
    const int n_tiles = (my_cols + COLS - 1) / COLS;
    if (n_tiles == 0) return;
    const int spans = (K + SW_SPAN - 1) / SW_SPAN;
    const int kb = wave * SW_KW;
    const bf16x8_t zero = {0, 0, 0, 0, 0, 0, 0, 0};

    bf16x8_t wreg[16];
    auto fetch_row = [&](int t, int p, int i) {
        const int k = p * SW_SPAN + kb + lane * 8;
        const int col = b + G * (t * COLS + (GATED ? (i & 7) : i));
        const size_t row = (GATED && i >= 8) ? (size_t)N + col : (size_t)col;
        wreg[i] = (k < K && col < N) ? *reinterpret_cast<const bf16x8_t*>(W + row * K + k) : zero;
    };
#pragma unroll
    for (int i = 0; i < 16; ++i) fetch_row(0, 0, i);

    for (int t = 0; t < n_tiles; ++t) {
        float4_t c = {0.f, 0.f, 0.f, 0.f};
        for (int p = 0; p < spans; ++p) {
            bf16x8_t bx[SW_STEPS];                              // the span's columns of x as B operands
#pragma unroll
            for (int j = 0; j < SW_STEPS; ++j) {
                const int k = p * SW_SPAN + kb + 32 * j + 8 * g;
                bx[j] = (n < M && k < K) ? *reinterpret_cast<const bf16x8_t*>(x + (size_t)n * K + k) : zero;
            }
            SW_WAVE_SYNC();
            const bool more = p + 1 < spans || t + 1 < n_tiles;
            const int t_next = p + 1 < spans ? t : t + 1, p_next = p + 1 < spans ? p + 1 : 0;
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                *reinterpret_cast<bf16x8_t*>(&stage[i * SW_STRIDE + lane * 8]) = wreg[i];
                if (more) fetch_row(t_next, p_next, i);
            }
            SW_WAVE_SYNC();
#pragma unroll
            for (int j = 0; j < SW_STEPS; ++j) {
                const bf16x8_t a = *reinterpret_cast<const bf16x8_t*>(&stage[n * SW_STRIDE + 32 * j + 8 * g]);
                c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, bx[j], c, 0, 0, 0);
            }
        }
        MFMA_SETTLE();
        float* red = red_both + (t & 1) * (SW_WAVES * 16 * 17);
#pragma unroll
        for (int i = 0; i < 4; ++i) red[(wave * 16 + 4 * g + i) * 17 + n] = c[i];
        __syncthreads();
        if (tid < 16 * COLS) {
            const int mm = tid / COLS, r = tid % COLS;
            const int col = b + G * (t * COLS + r);
            if (mm < M && col < N) {
                float s = 0.f;
#pragma unroll
                for (int w = 0; w < SW_WAVES; ++w) s += red[(w * 16 + r) * 17 + mm];
                if constexpr (GATED) {
                    float up = 0.f;
#pragma unroll
                    for (int w = 0; w < SW_WAVES; ++w) up += red[(w * 16 + 8 + r) * 17 + mm];
                    s = s / (1.0f + expf(-s)) * up;
                }
                out[(size_t)mm * N + col] = from_f<TO>(s);
            }
        }
    }
}

// the waves' W tiles, and their result tiles: two sets of 17 columns or one of 33
static size_t sweep_lds() { return (size_t)SW_WAVES * 16 * SW_STRIDE * 2 + (size_t)2 * SW_WAVES * 16 * 17 * 4; }

// Whether the sweep takes x [M, K]: up to 32 rows with K within one span, up to 16 rows with K up to
// 8 spans, K in whole pieces of 8.
extern "C" int ra_gemm_sweep_fits(int M, int K) {
    if (M < 1 || K <= 0 || K % 8 != 0) return 0;
    return K <= SW_SPAN ? M <= 32 : (M <= 16 && K <= 8 * SW_SPAN);
}

template <bool GATED, typename TO>
static int launch_sweep(int grid, hipStream_t st, const bf16* x, const bf16* W, TO* out, int M, int N, int K) {
    if (K > SW_SPAN) {
        auto long_kern = gemm_sweep_long_kernel<GATED, TO>;
        static bool long_allowed = false;
        if (!long_allowed) {
            if (hipFuncSetAttribute(reinterpret_cast<const void*>(long_kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                    (int)sweep_lds()) != hipSuccess)
                return RA_ERR_ARG;
            long_allowed = true;
        }
        hipLaunchKernelGGL(long_kern, dim3(grid), dim3(SW_THREADS), sweep_lds(), st, x, W, out, M, N, K);
        return RA_OK;
    }
    if (M > 16) {
        auto wide_kern = gemm_sweep_kernel<2, GATED, TO>;
        static bool wide_allowed = false;
        if (!wide_allowed) {
            if (hipFuncSetAttribute(reinterpret_cast<const void*>(wide_kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                    (int)sweep_lds()) != hipSuccess)
                return RA_ERR_ARG;
            wide_allowed = true;
        }
        hipLaunchKernelGGL(wide_kern, dim3(grid), dim3(SW_THREADS), sweep_lds(), st, x, W, out, M, N, K);
        return RA_OK;
    }
    auto kern = gemm_sweep_kernel<1, GATED, TO>;
    static bool allowed = false;                              // per instantiation: more than 64 KB of LDS
    if (!allowed) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)sweep_lds()) != hipSuccess)
            return RA_ERR_ARG;
        allowed = true;
    }
    hipLaunchKernelGGL(kern, dim3(grid), dim3(SW_THREADS), sweep_lds(), st, x, W, out, M, N, K);
    return RA_OK;
}

// gated: W is [2N, K], the result silu(x Wg^T) * (x Wu^T) in bfloat16. grid: workgroups; one per CU
// is what the sweep is measured with.
extern "C" int ra_gemm_sweep_bf16(const void* x, const void* W, void* out, int M, int N, int K, int gated,
                                  int out_dtype, int grid, void* stream) {
    if (M <= 0 || N <= 0) return RA_OK;
    if (!ra_gemm_sweep_fits(M, K) || grid <= 0) return RA_ERR_ARG;
    if (grid > N) grid = N;
    hipStream_t st = (hipStream_t)stream;
    const bf16* xx = (const bf16*)x;
    const bf16* w = (const bf16*)W;
    int rc = RA_ERR_ARG;
    if (gated) {
        if (out_dtype == RA_DTYPE_BF16) rc = launch_sweep<true, bf16>(grid, st, xx, w, (bf16*)out, M, N, K);
    } else if (out_dtype == RA_DTYPE_BF16) {
        rc = launch_sweep<false, bf16>(grid, st, xx, w, (bf16*)out, M, N, K);
    } else if (out_dtype == RA_DTYPE_F32) {
        rc = launch_sweep<false, float>(grid, st, xx, w, (float*)out, M, N, K);
    }
    if (rc != RA_OK) return rc;
    return ra_launch_status();
}
