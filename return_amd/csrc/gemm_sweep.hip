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
//
// Two additions take the RMSNorm kernels out of a decode step (rollout/fused.py:6-17 is the norm,
// rollout/monkey_patch/qwen3.py:59-68 the residual arrangement they belong to). A norm's 1/rms is a
// number per row, so it can be applied to a product's result instead of to its operand:
// norm(h) W^T = rstd * ((h * w_norm) W^T).
//   row scale (any form): the result rows are multiplied by rstd[m] = rsqrt(sum_b psq[m][b] / cols + eps)
//       before anything else is done with them; psq holds partial sums of squares of the row, one per
//       workgroup of the product that made the row, added here in a fixed order.
//   residual epilogue (RESID, plain bfloat16 form): the result (rounded to bfloat16 as a result that is
//       stored would be) is added into the 32-bit residual stream h [M, N]; the workgroup writes
//       xw = bf16(h * w_next) for its columns, the operand of the next product, and the sum of squares of
//       its columns of every row to psq_out[m][workgroup], from which that product forms rstd.
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

// What the two additions need: nullptr where one is not used.
struct SweepNorm {
    const float* psq_in;       // [M, n_in] partial sums of squares of the rows of x's source; nullptr: no row scale
    int n_in;
    float inv_cols;            // 1 / width of that source
    float eps;
    float* h;                  // RESID: residual stream [M, N], updated in place
    const float* w_next;       // RESID: weight [N] of the norm that follows
    float* psq_out;            // RESID: [M, gridDim.x]
};

// rstd of up to 16 * MB rows into LDS (rs), from the partial sums: thread (row, j) adds partials j,
// j + 16, ..., the sixteen threads of a row are then added in a fixed tree.
// The loads are asked for first of all in the kernel (sweep_scales_ask), before any of W, and added
// up after the first rows of W have been asked for (sweep_scales_make): loads come back in the order
// they were asked for, so a wave that waited for these behind its rows of W would ask for the next
// tile's rows a whole round trip late. SW_SHARES partial sums a thread at most (16 x SW_SHARES per row).
#define SW_SHARES 16
__device__ __forceinline__ void sweep_scales_ask(const SweepNorm& nm, int M, float (&share)[SW_SHARES]) {
    const int tid = threadIdx.x, row = min(tid >> 4, M - 1), j = tid & 15;
#pragma unroll
    for (int i = 0; i < SW_SHARES; ++i) {
        const int b = min(j + 16 * i, nm.n_in - 1);           // always a valid place; what lies beyond n_in is not added
        share[i] = nm.psq_in[(size_t)row * nm.n_in + b];
    }
}
__device__ __forceinline__ void sweep_scales_make(const SweepNorm& nm, int rows, const float (&share)[SW_SHARES], float* rs) {
    const int tid = threadIdx.x, row = tid >> 4, j = tid & 15;
    if (row < rows) {
        float t = 0.f;
#pragma unroll
        for (int i = 0; i < SW_SHARES; ++i) t += (j + 16 * i < nm.n_in) ? share[i] : 0.f;
#pragma unroll
        for (int o = 8; o > 0; o >>= 1) t += __shfl_xor(t, o, 16);
        if (j == 0) rs[row] = 1.0f / sqrtf(t * nm.inv_cols + nm.eps);
    }
}

// MB: blocks of 16 rows of x (1 or 2)
template <int MB, bool GATED, typename TO, bool RESID = false>
__global__ __launch_bounds__(SW_THREADS) void gemm_sweep_kernel(
    const bf16* __restrict__ x, const bf16* __restrict__ W, TO* __restrict__ out, int M, int N, int K, SweepNorm nm) {
    static_assert(!RESID || (!GATED && MB == 1), "the residual epilogue belongs to the plain product of up to 16 rows");
    constexpr int COLS = GATED ? 8 : 16;                        // result columns of a tile
    constexpr int RS = 16 * MB + 1;                             // row stride of the waves' tiles in LDS (floats)
    constexpr bool TWO_BUFFERS = MB == 1;                       // of those tiles (LDS has room for one set with MB == 2)
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, n = lane & 15, g = lane >> 4;
    uint16_t* stage = reinterpret_cast<uint16_t*>(lds_raw) + (size_t)wave * 16 * SW_STRIDE;
    float* red_both = reinterpret_cast<float*>(lds_raw + (size_t)SW_WAVES * 16 * SW_STRIDE * 2);   // [1 or 2][wave][16 rows][RS]
    float* rs = red_both + 2 * SW_WAVES * 16 * 17;            // [32] row scales, behind the result tiles
    const int G = gridDim.x, b = blockIdx.x;
    const int my_cols = N > b ? (N - 1 - b) / G + 1 : 0;
    const int n_tiles = (my_cols + COLS - 1) / COLS;
    if (n_tiles == 0) return;                                   // (the launch keeps the grid within N)
    const int kb = wave * SW_KW;
    const bool k_in = kb + lane * 8 < K;                        // K % 8 == 0: a lane's 8 columns are in or out together
    const bf16x8_t zero = {0, 0, 0, 0, 0, 0, 0, 0};

    const bool scaled = nm.psq_in != nullptr;
    float share[SW_SHARES];
    if (scaled) sweep_scales_ask(nm, M, share);

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

    if (scaled) sweep_scales_make(nm, 16 * MB, share, rs);    // (read after the first tile's barrier)
    [[maybe_unused]] float sq = 0.f;                           // RESID: squares of this thread's row over its columns

    for (int t = 0; t < n_tiles; ++t) {
        // RESID: this tile's entries of h and of the next norm's weight are asked for now, before the next
        // tile's rows of W (loads come back in the order they were asked for: asked for in the epilogue,
        // they would make it wait for those rows). Always from a valid place, so that the load stands
        // under no condition; what lies outside the result is not used.
        [[maybe_unused]] float h_old = 0.f, wn = 0.f;
        if constexpr (RESID) {
            const int mm = min(tid / COLS, M - 1), col = min(b + G * (t * COLS + tid % COLS), N - 1);
            h_old = nm.h[(size_t)mm * N + col];
            wn = nm.w_next[col];
        }
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
                const float scale = scaled ? rs[mm] : 1.0f;
                s *= scale;
                if constexpr (GATED) {
                    float up = 0.f;
#pragma unroll
                    for (int w = 0; w < SW_WAVES; ++w) up += red[(w * 16 + 8 + r) * RS + mm];
                    s = s / (1.0f + expf(-s)) * (up * scale); // gate and up stay 32-bit until here
                }
                if constexpr (RESID) {
                    const size_t at = (size_t)mm * N + col;
                    const float hv = h_old + round_to<bf16>(s);
                    nm.h[at] = hv;
                    out[at] = from_f<TO>(hv * wn);
                    sq += hv * hv;
                } else {
                    out[(size_t)mm * N + col] = from_f<TO>(s);
                }
            }
        }
        if constexpr (!TWO_BUFFERS) __syncthreads();
    }
    if constexpr (RESID) {
        // thread (mm, r): the sixteen threads of a row sit in sixteen neighbouring lanes
        if (tid < 16 * COLS) {
#pragma unroll
            for (int o = 8; o > 0; o >>= 1) sq += __shfl_xor(sq, o, 16);
            if ((tid & 15) == 0 && (tid >> 4) < M) nm.psq_out[(size_t)(tid >> 4) * G + b] = sq;
        }
    }
}


#define SW_SPAN (SW_WAVES * SW_KW)        // columns of K that the eight waves cover at once

// HELD: K is at most two spans, and the columns of x of both stay in registers for all tiles.
template <bool GATED, typename TO, bool RESID = false, bool HELD = false>
__global__ __launch_bounds__(SW_THREADS) void gemm_sweep_long_kernel(
    const bf16* __restrict__ x, const bf16* __restrict__ W, TO* __restrict__ out, int M, int N, int K, SweepNorm nm) {
    static_assert(!RESID || !GATED, "the residual epilogue belongs to the plain product");
    constexpr int COLS = GATED ? 8 : 16;
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, n = lane & 15, g = lane >> 4;
    uint16_t* stage = reinterpret_cast<uint16_t*>(lds_raw) + (size_t)wave * 16 * SW_STRIDE;
    float* red_both = reinterpret_cast<float*>(lds_raw + (size_t)SW_WAVES * 16 * SW_STRIDE * 2);
    float* rs = red_both + 2 * SW_WAVES * 16 * 17;
    const int G = gridDim.x, b = blockIdx.x;
    const int my_cols = N > b ? (N - 1 - b) / G + 1 : 0;
    const int n_tiles = (my_cols + COLS - 1) / COLS;
    if (n_tiles == 0) return;
    const int spans = (K + SW_SPAN - 1) / SW_SPAN;
    const int kb = wave * SW_KW;
    const bf16x8_t zero = {0, 0, 0, 0, 0, 0, 0, 0};

    const bool scaled = nm.psq_in != nullptr;
    float share[SW_SHARES];
    if (scaled) sweep_scales_ask(nm, M, share);
    bf16x8_t wreg[16];
    auto fetch_row = [&](int t, int p, int i) {
        const int k = p * SW_SPAN + kb + lane * 8;
        const int col = b + G * (t * COLS + (GATED ? (i & 7) : i));
        const size_t row = (GATED && i >= 8) ? (size_t)N + col : (size_t)col;
        wreg[i] = (k < K && col < N) ? *reinterpret_cast<const bf16x8_t*>(W + row * K + k) : zero;
    };
#pragma unroll
    for (int i = 0; i < 16; ++i) fetch_row(0, 0, i);
    [[maybe_unused]] bf16x8_t held[HELD ? 2 : 1][SW_STEPS];
    if constexpr (HELD) {
#pragma unroll
        for (int p = 0; p < 2; ++p)
#pragma unroll
            for (int j = 0; j < SW_STEPS; ++j) {
                const int k = p * SW_SPAN + kb + 32 * j + 8 * g;
                held[p][j] = (n < M && k < K) ? *reinterpret_cast<const bf16x8_t*>(x + (size_t)n * K + k) : zero;
            }
    }
    if (scaled) sweep_scales_make(nm, 16, share, rs);
    [[maybe_unused]] float sq = 0.f;

    for (int t = 0; t < n_tiles; ++t) {
        [[maybe_unused]] float h_old = 0.f, wn = 0.f;          // (asked for before the tile's loads of W, as in the kernel above)
        if constexpr (RESID) {
            const int mm = min(tid / COLS, M - 1), col = min(b + G * (t * COLS + tid % COLS), N - 1);
            h_old = nm.h[(size_t)mm * N + col];
            wn = nm.w_next[col];
        }
        float4_t c = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int p = 0; p < (HELD ? 2 : spans); ++p) {
            bf16x8_t bx[SW_STEPS];                              // the span's columns of x as B operands
#pragma unroll
            for (int j = 0; j < SW_STEPS; ++j) {
                if constexpr (HELD) {
                    bx[j] = held[p][j];
                } else {
                    const int k = p * SW_SPAN + kb + 32 * j + 8 * g;
                    bx[j] = (n < M && k < K) ? *reinterpret_cast<const bf16x8_t*>(x + (size_t)n * K + k) : zero;
                }
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
                const float scale = scaled ? rs[mm] : 1.0f;
                s *= scale;
                if constexpr (GATED) {
                    float up = 0.f;
#pragma unroll
                    for (int w = 0; w < SW_WAVES; ++w) up += red[(w * 16 + 8 + r) * 17 + mm];
                    s = s / (1.0f + expf(-s)) * (up * scale);
                }
                if constexpr (RESID) {
                    const size_t at = (size_t)mm * N + col;
                    const float hv = h_old + round_to<bf16>(s);
                    nm.h[at] = hv;
                    out[at] = from_f<TO>(hv * wn);
                    sq += hv * hv;
                } else {
                    out[(size_t)mm * N + col] = from_f<TO>(s);
                }
            }
        }
    }
    if constexpr (RESID) {
        if (tid < 16 * COLS) {
#pragma unroll
            for (int o = 8; o > 0; o >>= 1) sq += __shfl_xor(sq, o, 16);
            if ((tid & 15) == 0 && (tid >> 4) < M) nm.psq_out[(size_t)(tid >> 4) * G + b] = sq;
        }
    }
}

#define SW_FEW_TILES 4                    // tiles a workgroup has at most in gemm_sweep_spans_kernel

// K beyond two spans and at most SW_FEW_TILES tiles a workgroup (few result columns, many of K: a down
// projection): span by span, so that a span's columns of x are read once and serve every tile; the tiles'
// sums stay in registers until the last span. (gemm_sweep_long_kernel reads x again for every tile, as many
// bytes as the tile of W.)
template <bool GATED, typename TO, bool RESID = false>
__global__ __launch_bounds__(SW_THREADS) void gemm_sweep_spans_kernel(
    const bf16* __restrict__ x, const bf16* __restrict__ W, TO* __restrict__ out, int M, int N, int K, SweepNorm nm) {
    static_assert(!RESID || !GATED, "the residual epilogue belongs to the plain product");
    constexpr int COLS = GATED ? 8 : 16;
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, n = lane & 15, g = lane >> 4;
    uint16_t* stage = reinterpret_cast<uint16_t*>(lds_raw) + (size_t)wave * 16 * SW_STRIDE;
    float* red_both = reinterpret_cast<float*>(lds_raw + (size_t)SW_WAVES * 16 * SW_STRIDE * 2);
    float* rs = red_both + 2 * SW_WAVES * 16 * 17;
    const int G = gridDim.x, b = blockIdx.x;
    const int my_cols = N > b ? (N - 1 - b) / G + 1 : 0;
    const int n_tiles = (my_cols + COLS - 1) / COLS;          // (the launch keeps it within SW_FEW_TILES)
    if (n_tiles == 0) return;
    const int spans = (K + SW_SPAN - 1) / SW_SPAN;
    const int kb = wave * SW_KW;
    const bf16x8_t zero = {0, 0, 0, 0, 0, 0, 0, 0};

    const bool scaled = nm.psq_in != nullptr;
    float share[SW_SHARES];
    if (scaled) sweep_scales_ask(nm, M, share);
    bf16x8_t wreg[16];
    auto fetch_row = [&](int t, int p, int i) {
        const int k = p * SW_SPAN + kb + lane * 8;
        const int col = b + G * (t * COLS + (GATED ? (i & 7) : i));
        const size_t row = (GATED && i >= 8) ? (size_t)N + col : (size_t)col;
        wreg[i] = (k < K && col < N) ? *reinterpret_cast<const bf16x8_t*>(W + row * K + k) : zero;
    };
#pragma unroll
    for (int i = 0; i < 16; ++i) fetch_row(0, 0, i);
    if (scaled) sweep_scales_make(nm, 16, share, rs);
    float4_t c[SW_FEW_TILES];
#pragma unroll
    for (int t = 0; t < SW_FEW_TILES; ++t) c[t] = float4_t{0.f, 0.f, 0.f, 0.f};

    // RESID: the tiles' entries of h and of the next norm's weight are asked for at the start of the last
    // span, before its rows of W (asked for in the epilogue they would be waited for; see the kernel above)
    [[maybe_unused]] float h_old[SW_FEW_TILES], wn[SW_FEW_TILES];
    for (int p = 0; p < spans; ++p) {
        if constexpr (RESID) {
            if (p == spans - 1) {
#pragma unroll
                for (int t = 0; t < SW_FEW_TILES; ++t) {
                    const int mm = min(tid / COLS, M - 1), col = min(b + G * (min(t, n_tiles - 1) * COLS + tid % COLS), N - 1);
                    h_old[t] = nm.h[(size_t)mm * N + col];
                    wn[t] = nm.w_next[col];
                }
            }
        }
        bf16x8_t bx[SW_STEPS];                                  // the span's columns of x as B operands, for every tile
#pragma unroll
        for (int j = 0; j < SW_STEPS; ++j) {
            const int k = p * SW_SPAN + kb + 32 * j + 8 * g;
            bx[j] = (n < M && k < K) ? *reinterpret_cast<const bf16x8_t*>(x + (size_t)n * K + k) : zero;
        }
#pragma unroll
        for (int t = 0; t < SW_FEW_TILES; ++t) {
            if (t >= n_tiles) break;
            SW_WAVE_SYNC();
            const bool more = t + 1 < n_tiles || p + 1 < spans;
            const int t_next = t + 1 < n_tiles ? t + 1 : 0, p_next = t + 1 < n_tiles ? p : p + 1;
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                *reinterpret_cast<bf16x8_t*>(&stage[i * SW_STRIDE + lane * 8]) = wreg[i];
                if (more) fetch_row(t_next, p_next, i);
            }
            SW_WAVE_SYNC();
#pragma unroll
            for (int j = 0; j < SW_STEPS; ++j) {
                const bf16x8_t a = *reinterpret_cast<const bf16x8_t*>(&stage[n * SW_STRIDE + 32 * j + 8 * g]);
                c[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, bx[j], c[t], 0, 0, 0);
            }
        }
    }
    MFMA_SETTLE();
    [[maybe_unused]] float sq = 0.f;
#pragma unroll
    for (int t = 0; t < SW_FEW_TILES; ++t) {
        if (t >= n_tiles) break;
        float* red = red_both + (t & 1) * (SW_WAVES * 16 * 17);
#pragma unroll
        for (int i = 0; i < 4; ++i) red[(wave * 16 + 4 * g + i) * 17 + n] = c[t][i];
        __syncthreads();
        if (tid < 16 * COLS) {
            const int mm = tid / COLS, r = tid % COLS;
            const int col = b + G * (t * COLS + r);
            if (mm < M && col < N) {
                float s = 0.f;
#pragma unroll
                for (int w = 0; w < SW_WAVES; ++w) s += red[(w * 16 + r) * 17 + mm];
                const float scale = scaled ? rs[mm] : 1.0f;
                s *= scale;
                if constexpr (GATED) {
                    float up = 0.f;
#pragma unroll
                    for (int w = 0; w < SW_WAVES; ++w) up += red[(w * 16 + 8 + r) * 17 + mm];
                    s = s / (1.0f + expf(-s)) * (up * scale);
                }
                if constexpr (RESID) {
                    const size_t at = (size_t)mm * N + col;
                    const float hv = h_old[t] + round_to<bf16>(s);
                    nm.h[at] = hv;
                    out[at] = from_f<TO>(hv * wn[t]);
                    sq += hv * hv;
                } else {
                    out[(size_t)mm * N + col] = from_f<TO>(s);
                }
            }
        }
    }
    if constexpr (RESID) {
        if (tid < 16 * COLS) {
#pragma unroll
            for (int o = 8; o > 0; o >>= 1) sq += __shfl_xor(sq, o, 16);
            if ((tid & 15) == 0 && (tid >> 4) < M) nm.psq_out[(size_t)(tid >> 4) * G + b] = sq;
        }
    }
}

// the waves' W tiles, and their result tiles: two sets of 17 columns or one of 33
static size_t sweep_lds() { return (size_t)SW_WAVES * 16 * SW_STRIDE * 2 + (size_t)2 * SW_WAVES * 16 * 17 * 4 + 32 * 4; }

// Whether the sweep takes x [M, K]: up to 32 rows with K within one span, up to 16 rows with K up to
// 8 spans, K in whole pieces of 8.
extern "C" int ra_gemm_sweep_fits(int M, int K) {
    if (M < 1 || K <= 0 || K % 8 != 0) return 0;
    return K <= SW_SPAN ? M <= 32 : (M <= 16 && K <= 8 * SW_SPAN);
}

template <typename TO, typename KERN>
static int launch_sweep_kernel(KERN kern, bool& allowed, int grid, hipStream_t st, const bf16* x, const bf16* W, TO* out,
                               int M, int N, int K, const SweepNorm& nm) {
    if (!allowed) {                                           // per instantiation: more than 64 KB of LDS
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)sweep_lds()) != hipSuccess)
            return RA_ERR_ARG;
        allowed = true;
    }
    hipLaunchKernelGGL(kern, dim3(grid), dim3(SW_THREADS), sweep_lds(), st, x, W, out, M, N, K, nm);
    return RA_OK;
}

template <bool GATED, typename TO, bool RESID>
static int launch_sweep(int grid, hipStream_t st, const bf16* x, const bf16* W, TO* out, int M, int N, int K,
                        const SweepNorm& nm) {
    if (K > SW_SPAN) {
        if (K <= 2 * SW_SPAN) {
            static bool allowed = false;
            return launch_sweep_kernel(gemm_sweep_long_kernel<GATED, TO, RESID, true>, allowed, grid, st, x, W, out, M, N, K, nm);
        }
        const int cols = GATED ? 8 : 16, workgroups = grid < N ? grid : N;
        const int most_tiles = ((N + workgroups - 1) / workgroups + cols - 1) / cols;
        if (most_tiles >= 2 && most_tiles <= SW_FEW_TILES) {    // (with one tile the two orders are the same, and this one a little slower)
            static bool allowed = false;
            return launch_sweep_kernel(gemm_sweep_spans_kernel<GATED, TO, RESID>, allowed, grid, st, x, W, out, M, N, K, nm);
        }
        static bool allowed = false;
        return launch_sweep_kernel(gemm_sweep_long_kernel<GATED, TO, RESID, false>, allowed, grid, st, x, W, out, M, N, K, nm);
    }
    if constexpr (!RESID) {
        if (M > 16) {
            static bool allowed = false;
            return launch_sweep_kernel(gemm_sweep_kernel<2, GATED, TO, false>, allowed, grid, st, x, W, out, M, N, K, nm);
        }
    }
    static bool allowed = false;
    return launch_sweep_kernel(gemm_sweep_kernel<1, GATED, TO, RESID>, allowed, grid, st, x, W, out, M, N, K, nm);
}

static int sweep_dispatch(const void* x, const void* W, void* out, int M, int N, int K, int gated, int out_dtype,
                          int grid, const SweepNorm& nm, void* stream) {
    if (M <= 0 || N <= 0) return RA_OK;
    if (!ra_gemm_sweep_fits(M, K) || grid <= 0) return RA_ERR_ARG;
    if (grid > N) grid = N;
    hipStream_t st = (hipStream_t)stream;
    const bf16* xx = (const bf16*)x;
    const bf16* w = (const bf16*)W;
    int rc = RA_ERR_ARG;
    if (nm.h != nullptr) {
        if (!gated && out_dtype == RA_DTYPE_BF16 && M <= 16)
            rc = launch_sweep<false, bf16, true>(grid, st, xx, w, (bf16*)out, M, N, K, nm);
    } else if (gated) {
        if (out_dtype == RA_DTYPE_BF16) rc = launch_sweep<true, bf16, false>(grid, st, xx, w, (bf16*)out, M, N, K, nm);
    } else if (out_dtype == RA_DTYPE_BF16) {
        rc = launch_sweep<false, bf16, false>(grid, st, xx, w, (bf16*)out, M, N, K, nm);
    } else if (out_dtype == RA_DTYPE_F32) {
        rc = launch_sweep<false, float, false>(grid, st, xx, w, (float*)out, M, N, K, nm);
    }
    if (rc != RA_OK) return rc;
    return ra_launch_status();
}

// gated: W is [2N, K], the result silu(x Wg^T) * (x Wu^T) in bfloat16. grid: workgroups; one per CU
// is what the sweep is measured with.
extern "C" int ra_gemm_sweep_bf16(const void* x, const void* W, void* out, int M, int N, int K, int gated,
                                  int out_dtype, int grid, void* stream) {
    SweepNorm none = {};
    return sweep_dispatch(x, W, out, M, N, K, gated, out_dtype, grid, none, stream);
}

// The same with the norm's two additions (see the head of this file).
//   psq_in [M, n_in] (nullptr: no row scale), norm_cols, eps: the result rows are multiplied by
//       rsqrt(sum_b psq_in[m][b] / norm_cols + eps).
//   h [M, N] fp32, w_next [N] fp32, psq_out [M, workgroups] fp32 (all three or none; plain bfloat16
//       form, M <= 16): h += result; out = bf16(h * w_next); psq_out[m][b] = workgroup b's share of
//       sum_n h[m][n]^2. The number of workgroups is min(grid, N): psq_out must have that many columns,
//       which ra_gemm_sweep_workgroups(N, grid) returns.
extern "C" int ra_gemm_sweep_workgroups(int N, int grid) { return grid < N ? grid : N; }

extern "C" int ra_gemm_sweep_norm_bf16(const void* x, const void* W, void* out, int M, int N, int K, int gated,
                                       int out_dtype, int grid, const float* psq_in, int n_in, int norm_cols,
                                       float eps, float* h, const float* w_next, float* psq_out, void* stream) {
    if ((h == nullptr) != (w_next == nullptr) || (h == nullptr) != (psq_out == nullptr)) return RA_ERR_ARG;
    if (psq_in != nullptr && (n_in <= 0 || n_in > 16 * SW_SHARES || norm_cols <= 0)) return RA_ERR_ARG;
    if (M > 32) return RA_ERR_ARG;                            // the row scales of a workgroup are at most 32
    SweepNorm nm = {psq_in, n_in, norm_cols > 0 ? 1.0f / (float)norm_cols : 0.f, eps, h, w_next, psq_out};
    return sweep_dispatch(x, W, out, M, N, K, gated, out_dtype, grid, nm, stream);
}
