// y = x @ W^T for few rows of x (M <= 64), bfloat16 in, fp32 accumulate: the decode-time
// matrix product, bound by streaming W once from HBM. Layout as in the reference's
// F.linear (rollout/monkey_patch/qwen3.py:21): x [M, K], W [N, K], y [M, N].
//
// A workgroup (four waves) takes a block of 64 rows of W and one share of K (`k_extent`
// elements); its waves interleave k-blocks of 32*U elements. W is the A operand of MFMA
// 16x16x32 bf16: lane (n, g) loads 16 contiguous bytes of row n at k = k0 + 8g, which is
// exactly its operand; x is the B operand, loaded the same way from row m = lane % 16 and used
// for all four row groups of the block, so x costs a quarter of W's traffic per 16 rows of x.
// The contraction does not care how k is distributed over lanes as long as both operands agree.
// The waves' partial tiles are added in LDS in wave order. When K is split over workgroups
// (small N: the block count alone would not fill the chip), every workgroup writes its tile to
// a workspace and the one that arrives last at the block's counter adds the shares in split
// order and writes the result: the sum never depends on scheduling. The counter is left at zero.
// Needs K % 8 == 0 (16-byte loads); other K go to the plain kernel.
//
// GATED: W is [2I, K] with the gate rows first (rollout/monkey_patch/qwen3.py:103); a block
// takes 32 gate rows and the 32 up rows that belong to them and writes silu(g) * u
// (rollout/fused.py:103-114) as [M, I], so the [M, 2I] intermediate never reaches memory.
//
// Calls that share one workspace must not overlap in time (one stream).
#include "common.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));

#define SK_WAVES 4
#define SK_R 4                           // row groups of 16 per workgroup block
#define SK_TILE (SK_R * 256)             // floats of one 16-row x block: [z][r][m]

template <int MB, int U, typename TO, bool GATED>
__global__ __launch_bounds__(SK_WAVES * 64) void gemm_skinny_kernel(
    const bf16* __restrict__ x, const bf16* __restrict__ W, TO* __restrict__ out,
    float* __restrict__ part, int* __restrict__ counters, int M, int N, int K, int k_extent,
    int n_splits) {
    // N: columns of the result (= rows of W, or half of them when GATED)
    constexpr int COLS = GATED ? 16 * SK_R / 2 : 16 * SK_R;     // result columns per block
    __shared__ float acc_s[MB][SK_R][16][17];                   // [b][z][r][m]
    __shared__ int last_s;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int n = lane & 15, g = lane >> 4;
    const int blk = blockIdx.x, ks = blockIdx.y;
    const int c0 = blk * COLS;
    const bf16x8_t zero = {0, 0, 0, 0, 0, 0, 0, 0};

    const bf16* wp[SK_R];
#pragma unroll
    for (int z = 0; z < SK_R; ++z) {
        int row;
        if constexpr (GATED) {
            const int col = min(c0 + 16 * (z % (SK_R / 2)) + n, N - 1);   // clamped: loads stay inside W
            row = (z < SK_R / 2) ? col : N + col;
        } else {
            row = min(c0 + 16 * z + n, N - 1);
        }
        wp[z] = W + (size_t)row * K + g * 8;
    }
    const bf16* xp[MB];
    bool x_ok[MB];
#pragma unroll
    for (int b = 0; b < MB; ++b) {
        const int m = b * 16 + n;
        x_ok[b] = m < M;
        xp[b] = x + (size_t)min(m, M - 1) * K + g * 8;
    }
    float4_t c[SK_R][MB];
#pragma unroll
    for (int z = 0; z < SK_R; ++z)
#pragma unroll
        for (int b = 0; b < MB; ++b) c[z][b] = float4_t{0.f, 0.f, 0.f, 0.f};

    const int k_lo = ks * k_extent, k_hi = min(K, k_lo + k_extent);
    for (int kb = k_lo + wave * (32 * U); kb < k_hi; kb += SK_WAVES * 32 * U) {
        bf16x8_t a[SK_R][U];
        bf16x8_t bx[MB][U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int k = kb + u * 32;
            const bool in = k + g * 8 < k_hi;                 // K % 8 == 0: a lane's 8 are in or out together
#pragma unroll
            for (int z = 0; z < SK_R; ++z)
                a[z][u] = in ? *reinterpret_cast<const bf16x8_t*>(wp[z] + k) : zero;
#pragma unroll
            for (int b = 0; b < MB; ++b)
                bx[b][u] = (in && x_ok[b]) ? *reinterpret_cast<const bf16x8_t*>(xp[b] + k) : zero;
        }
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int b = 0; b < MB; ++b)
#pragma unroll
                for (int z = 0; z < SK_R; ++z)
                    c[z][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[z][u], bx[b][u], c[z][b], 0, 0, 0);
    }
    MFMA_SETTLE();
    // c[z][b][i] = partial y[m = 16b + n][row 16z + 4g + i of the block]; the waves add theirs in order
#pragma unroll
    for (int w = 0; w < SK_WAVES; ++w) {
        if (wave == w) {
#pragma unroll
            for (int z = 0; z < SK_R; ++z)
#pragma unroll
                for (int b = 0; b < MB; ++b)
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        float* p = &acc_s[b][z][4 * g + i][n];
                        *p = (w == 0) ? c[z][b][i] : *p + c[z][b][i];
                    }
        }
        __syncthreads();
    }

    const float* share = nullptr;              // the shares of this block, split after split
    if (n_splits > 1) {
        float* mine = part + ((size_t)blk * n_splits + ks) * (MB * SK_TILE);
        for (int e = threadIdx.x; e < MB * SK_TILE; e += SK_WAVES * 64)
            mine[e] = acc_s[e >> 10][(e >> 8) & 3][(e >> 4) & 15][e & 15];
        __threadfence();                       // the tile is visible before the counter moves
        __syncthreads();
        if (threadIdx.x == 0) {
            const int seen = atomicAdd(&counters[blk], 1);
            last_s = seen == n_splits - 1;
            if (seen == n_splits - 1) atomicExch(&counters[blk], 0);
        }
        __syncthreads();
        if (!last_s) return;
        __threadfence();                       // read the others' tiles from memory, not from a stale line
        share = part + (size_t)blk * n_splits * (MB * SK_TILE);
    }
    auto value = [&](int b, int z, int r, int mm) -> float {
        if (share == nullptr) return acc_s[b][z][r][mm];
        const float* p = share + ((b * SK_R + z) * 16 + r) * 16 + mm;
        float s = 0.f;
        for (int q = 0; q < n_splits; ++q) s += p[(size_t)q * (MB * SK_TILE)];
        return s;
    };
    for (int e = threadIdx.x; e < MB * 16 * COLS; e += SK_WAVES * 64) {
        const int cc = e % COLS, mrow = e / COLS;             // column fastest: neighbours write neighbours
        const int b = mrow >> 4, mm = mrow & 15, z = cc >> 4, r = cc & 15;
        const int m = mrow, col = c0 + cc;
        if (m < M && col < N) {
            float s = value(b, z, r, mm);
            if constexpr (GATED) {
                const float up = value(b, z + SK_R / 2, r, mm);
                s = s / (1.0f + expf(-s)) * up;               // gate and up stay 32-bit until here
            }
            out[(size_t)m * N + col] = from_f<TO>(s);
        }
    }
}

template <int MB, typename TO, bool GATED>
static void launch_skinny(dim3 grid, hipStream_t st, const bf16* x, const bf16* W, TO* out, float* part,
                          int* counters, int M, int N, int K, int k_extent, int n_splits) {
    constexpr int U = MB == 1 ? 4 : 2;
    hipLaunchKernelGGL((gemm_skinny_kernel<MB, U, TO, GATED>), grid, dim3(SK_WAVES * 64), 0, st, x, W,
                       out, part, counters, M, N, K, k_extent, n_splits);
}

template <typename TO, bool GATED>
static int pick_mb(dim3 grid, hipStream_t st, const bf16* x, const bf16* W, TO* out, float* part,
                   int* counters, int M, int N, int K, int k_extent, int n_splits) {
    switch ((M + 15) / 16) {
        case 1: launch_skinny<1, TO, GATED>(grid, st, x, W, out, part, counters, M, N, K, k_extent, n_splits); break;
        case 2: launch_skinny<2, TO, GATED>(grid, st, x, W, out, part, counters, M, N, K, k_extent, n_splits); break;
        case 3: launch_skinny<3, TO, GATED>(grid, st, x, W, out, part, counters, M, N, K, k_extent, n_splits); break;
        case 4: launch_skinny<4, TO, GATED>(grid, st, x, W, out, part, counters, M, N, K, k_extent, n_splits); break;
        default: return RA_ERR_ARG;
    }
    return RA_OK;
}

// How K is shared out: enough workgroups to fill the chip, shares no shorter than one pass of
// the four waves, and within the workspace and the counters the caller brought.
static void plan_split(int M, int n_blocks, int K, size_t ws_floats, int n_counters, int want_wgs,
                       int* k_extent, int* n_splits) {
    const int mb = (M + 15) / 16;
    const int step = SK_WAVES * 32 * (mb == 1 ? 4 : 2);          // k elements per pass of the workgroup
    int splits = 1;
    if (n_blocks < want_wgs && n_blocks <= n_counters) {
        splits = (want_wgs + n_blocks - 1) / n_blocks;
        const int most = max(1, K / step);
        if (splits > most) splits = most;
        const size_t per_split = (size_t)n_blocks * mb * SK_TILE;
        if ((size_t)splits * per_split > ws_floats) splits = (int)(ws_floats / per_split);
        if (splits < 1) splits = 1;
    }
    int extent = (K + splits - 1) / splits;
    extent = (extent + 31) / 32 * 32;
    *k_extent = extent;
    *n_splits = (K + extent - 1) / extent;
}

// ws: workspace of ws_bytes for the shares of a split K; counters: n_counters ints, zero before
// the first call (every call leaves them zero). want_wgs <= 0: the default.
extern "C" int ra_gemm_skinny_bf16(const void* x, const void* W, void* out, int M, int N, int K,
                                   int out_dtype, void* ws, size_t ws_bytes, void* counters,
                                   int n_counters, int want_wgs, void* stream) {
    if (M <= 0 || N <= 0) return RA_OK;
    if (M > 64 || K <= 0 || K % 8 != 0) return RA_ERR_ARG;
    const int n_blocks = (N + 16 * SK_R - 1) / (16 * SK_R);
    int k_extent, n_splits;
    plan_split(M, n_blocks, K, ws ? ws_bytes / 4 : 0, counters ? n_counters : 0,
               want_wgs > 0 ? want_wgs : 512, &k_extent, &n_splits);
    if (n_splits > 65535) return RA_ERR_ARG;
    hipStream_t st = (hipStream_t)stream;
    const dim3 grid(n_blocks, n_splits);
    int rc;
    if (out_dtype == RA_DTYPE_F32)
        rc = pick_mb<float, false>(grid, st, (const bf16*)x, (const bf16*)W, (float*)out, (float*)ws,
                                   (int*)counters, M, N, K, k_extent, n_splits);
    else if (out_dtype == RA_DTYPE_BF16)
        rc = pick_mb<bf16, false>(grid, st, (const bf16*)x, (const bf16*)W, (bf16*)out, (float*)ws,
                                  (int*)counters, M, N, K, k_extent, n_splits);
    else
        return RA_ERR_ARG;
    if (rc != RA_OK) return rc;
    return ra_launch_status();
}

// out [M, I] = silu(x @ Wg^T) * (x @ Wu^T) for W = [Wg; Wu] of shape [2I, K]; M <= 64.
extern "C" int ra_gemm_skinny_gated_bf16(const void* x, const void* W, void* out, int M, int I, int K,
                                         void* ws, size_t ws_bytes, void* counters, int n_counters,
                                         int want_wgs, void* stream) {
    if (M <= 0 || I <= 0) return RA_OK;
    if (M > 64 || K <= 0 || K % 8 != 0) return RA_ERR_ARG;
    const int n_blocks = (I + 8 * SK_R - 1) / (8 * SK_R);
    int k_extent, n_splits;
    plan_split(M, n_blocks, K, ws ? ws_bytes / 4 : 0, counters ? n_counters : 0,
               want_wgs > 0 ? want_wgs : 512, &k_extent, &n_splits);
    if (n_splits > 65535) return RA_ERR_ARG;
    hipStream_t st = (hipStream_t)stream;
    const int rc = pick_mb<bf16, true>(dim3(n_blocks, n_splits), st, (const bf16*)x, (const bf16*)W,
                                       (bf16*)out, (float*)ws, (int*)counters, M, I, K, k_extent, n_splits);
    if (rc != RA_OK) return rc;
    return ra_launch_status();
}
