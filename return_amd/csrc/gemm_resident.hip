// y = x @ W^T for very few rows (M <= 16) with x resident in LDS: the decode-time product when
// a workgroup takes several tiles of W (many rows of W: gate-up, the output head).
// Layout as in the reference's F.linear (rollout/monkey_patch/qwen3.py:21): x [M, K], W [N, K],
// y [M, N].
//
// A workgroup first copies x into LDS, [8 or 16][K + 8] (rows shifted by four banks). Then it
// walks over tiles of 16 rows of W (tile = blockIdx.x, += gridDim.x): its waves split K in
// blocks of 256 (128 when GATED), W is the A operand of MFMA 16x16x32 bf16 read straight from memory (lane
// (n, g): 16 bytes of row n at k0 + 8g), x the B operand read from LDS, and the waves' partial
// tiles are added through LDS in wave order (one barrier, then every thread adds one element). x is read from the cache once per workgroup
// instead of once per tile, and the loop issues no loads but W's.
// Results: bfloat16 or fp32 [M, N]; GATED (W = [Wg; Wu], rollout/monkey_patch/qwen3.py:103):
// silu(g) * u as [M, N] (rollout/fused.py:103-114).
// Needs K % 8 == 0 and the x block within the LDS a workgroup may have.
#include "common.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef uint32_t uint4_t __attribute__((ext_vector_type(4)));

#define RG_UNROLL 8

template <int WAVES, int MP, bool GATED, typename TO>
__global__ __launch_bounds__(WAVES * 64) void gemm_resident_kernel(
    const bf16* __restrict__ x, const bf16* __restrict__ W, TO* __restrict__ out, int M, int N, int K,
    int n_tiles) {
    constexpr int NG = GATED ? 2 : 1;
    constexpr int MB = 1;                                       // blocks of 16 rows of x (MP = 8 or 16 rows are held)
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    const int XS = K + 8;                                       // row stride of x in LDS (elements)
    uint16_t* x_s = reinterpret_cast<uint16_t*>(lds_raw);
    float* red = reinterpret_cast<float*>(lds_raw + (size_t)MP * XS * 2);   // [WAVES][NG][16][MP + 1]
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, n = lane & 15, g = lane >> 4;
    const bf16x8_t zero = {0, 0, 0, 0, 0, 0, 0, 0};

    // The blocks of W that this wave multiplies, in order: for every tile of the workgroup its k-blocks
    // wave, wave + WAVES, ... The next block is asked for before this one is multiplied, the first one
    // before x is copied, so that W keeps streaming through the copy and through the tiles' ends.
    constexpr int U = GATED ? RG_UNROLL / 2 : RG_UNROLL;    // MFMA steps per block (two operands each when GATED)
    constexpr int KB = 32 * U;
    const int n_kb = K > wave * KB ? (K - wave * KB + WAVES * KB - 1) / (WAVES * KB) : 0;
    bf16x8_t a_next[NG][U];
    int next_tile = blockIdx.x, next_j = 0;
    auto fetch = [&]() {
        if (next_tile >= n_tiles || n_kb == 0) return;
        const int row = min(next_tile * 16 + n, N - 1);     // clamped: loads stay inside W
        const bf16* wp = W + (size_t)row * K + g * 8;
        const bf16* wp_up = wp + (size_t)N * K;             // GATED: the up row of the same column
        const int kb = (wave + next_j * WAVES) * KB;
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int k = kb + u * 32;
            const bool in = k + g * 8 < K;                  // K % 8 == 0: a lane's 8 are in or out together
            a_next[0][u] = in ? *reinterpret_cast<const bf16x8_t*>(wp + k) : zero;
            if constexpr (GATED) a_next[1][u] = in ? *reinterpret_cast<const bf16x8_t*>(wp_up + k) : zero;
        }
    };
    fetch();

    // ---- x into LDS, rows beyond M as zeros
    {
        const int pieces = K / 8;
        for (int e = tid; e < MP * pieces; e += WAVES * 64) {
            const int m = e / pieces, p = e - m * pieces;
            uint4_t v = {0u, 0u, 0u, 0u};
            if (m < M) v = *reinterpret_cast<const uint4_t*>(x + (size_t)m * K + 8 * p);
            *reinterpret_cast<uint4_t*>(&x_s[m * XS + 8 * p]) = v;
        }
    }
    __syncthreads();

    for (int tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
        const int n0 = tile * 16;
        float4_t c[NG][MB];
#pragma unroll
        for (int z = 0; z < NG; ++z)
#pragma unroll
            for (int b = 0; b < MB; ++b) c[z][b] = float4_t{0.f, 0.f, 0.f, 0.f};

        for (int j = 0; j < n_kb; ++j) {
            bf16x8_t a[NG][U];
#pragma unroll
            for (int z = 0; z < NG; ++z)
#pragma unroll
                for (int u = 0; u < U; ++u) a[z][u] = a_next[z][u];
            if (j + 1 < n_kb) {
                next_j = j + 1;
            } else {
                next_tile = tile + gridDim.x;
                next_j = 0;
            }
            fetch();
            const int kb = (wave + j * WAVES) * KB;
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int k = kb + u * 32 + g * 8;
                const bool in = k < K;
#pragma unroll
                for (int b = 0; b < MB; ++b) {
                    bf16x8_t bx = zero;
                    if (in && n < MP) bx = *reinterpret_cast<const bf16x8_t*>(&x_s[(b * 16 + n) * XS + k]);
#pragma unroll
                    for (int z = 0; z < NG; ++z)
                        c[z][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[z][u], bx, c[z][b], 0, 0, 0);
                }
            }
        }
        MFMA_SETTLE();
        // c[z][0][i] = partial y[m = n][row n0 + 4g + i]: every wave puts its tile down, then the
        // threads add the waves' tiles in wave order
        if (n < MP) {
#pragma unroll
            for (int z = 0; z < NG; ++z)
#pragma unroll
                for (int i = 0; i < 4; ++i) red[((wave * NG + z) * 16 + 4 * g + i) * (MP + 1) + n] = c[z][0][i];
        }
        __syncthreads();
        for (int e = tid; e < MP * 16; e += WAVES * 64) {
            const int mm = e >> 4, r = e & 15;                // r fastest: neighbours write neighbours
            const int col = n0 + r;
            if (mm < M && col < N) {
                float s = 0.f;
#pragma unroll
                for (int w = 0; w < WAVES; ++w) s += red[((w * NG + 0) * 16 + r) * (MP + 1) + mm];
                if constexpr (GATED) {
                    float up = 0.f;
#pragma unroll
                    for (int w = 0; w < WAVES; ++w) up += red[((w * NG + 1) * 16 + r) * (MP + 1) + mm];
                    s = s / (1.0f + expf(-s)) * up;           // gate and up stay 32-bit until here
                }
                out[(size_t)mm * N + col] = from_f<TO>(s);
            }
        }
        __syncthreads();
    }
}

template <int WAVES, int MP, bool GATED, typename TO>
static int launch_resident(int grid, size_t lds, hipStream_t st, const bf16* x, const bf16* W, TO* out, int M,
                           int N, int K, int n_tiles) {
    auto kern = gemm_resident_kernel<WAVES, MP, GATED, TO>;
    static size_t allowed = 0;                                // per instantiation: raised when needed
    if (lds > allowed) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)lds) != hipSuccess)
            return RA_ERR_ARG;
        allowed = lds;
    }
    hipLaunchKernelGGL(kern, dim3(grid), dim3(WAVES * 64), lds, st, x, W, out, M, N, K, n_tiles);
    return RA_OK;
}

// LDS bytes for x [M, K] (M rounded up to 8 or 16) plus the reduction buffer
static size_t resident_lds(int M, int K, bool gated) {
    const int mp = M <= 8 ? 8 : 16;
    return (size_t)mp * (K + 8) * 2 + (size_t)8 * (gated ? 2 : 1) * 16 * (mp + 1) * 4;
}

extern "C" int ra_gemm_resident_fits(int M, int K, int gated) {
    return M >= 1 && M <= 16 && K > 0 && K % 8 == 0 && resident_lds(M, K, gated != 0) <= 160 * 1024 - 512;
}

// gated: W is [2N, K], the result silu(x Wg^T) * (x Wu^T) in bfloat16. grid: workgroups (each
// walks over tiles grid apart); <= 0: two per CU.
extern "C" int ra_gemm_resident_bf16(const void* x, const void* W, void* out, int M, int N, int K, int gated,
                                     int out_dtype, int grid, void* stream) {
    if (M <= 0 || N <= 0) return RA_OK;
    if (!ra_gemm_resident_fits(M, K, gated)) return RA_ERR_ARG;
    const int n_tiles = (N + 15) / 16;
    if (grid <= 0) grid = 512;
    if (grid > n_tiles) grid = n_tiles;
    const size_t lds = resident_lds(M, K, gated != 0);
    hipStream_t st = (hipStream_t)stream;
    const bf16* xx = (const bf16*)x;
    const bf16* w = (const bf16*)W;
    int rc = RA_ERR_ARG;
#define GO(GATED_, TO_)                                                                                   \
    rc = M <= 8 ? launch_resident<8, 8, GATED_, TO_>(grid, lds, st, xx, w, (TO_*)out, M, N, K, n_tiles)   \
                : launch_resident<8, 16, GATED_, TO_>(grid, lds, st, xx, w, (TO_*)out, M, N, K, n_tiles)
    if (gated) {
        if (out_dtype != RA_DTYPE_BF16) return RA_ERR_ARG;
        GO(true, bf16);
    } else if (out_dtype == RA_DTYPE_BF16) {
        GO(false, bf16);
    } else if (out_dtype == RA_DTYPE_F32) {
        GO(false, float);
    }
#undef GO
    if (rc != RA_OK) return rc;
    return ra_launch_status();
}
