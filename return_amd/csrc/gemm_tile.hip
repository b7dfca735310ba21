// y = x @ W^T for many rows, bfloat16 in, fp32 accumulate, fp32 or bfloat16 out: the larger of the two
// hand-written MFMA products (gemm_mfma.hip has the smaller, which takes any K % 8 == 0 and wastes less
// on few rows). Layout of the reference's F.linear (rollout/monkey_patch/qwen3.py:21): x [M, K],
// W [N, K], y [M, N]. Like gemm_mfma.hip it stands beside the library, which is faster (1.1 against
// 1.4 PFLOP/s at 2,048 x 24,576 x 4,096 on MI355X) and which the engine uses for products of many rows.
//
// Workgroup tile 256 x 256, k-steps of 32, eight waves as 2 x 4: a wave has 128 rows of x by 64 rows
// of W as 8 x 4 MFMA 16x16x32 tiles (128 accumulator registers). Tiles of both operands go straight
// from memory into LDS (buffer_load ... lds: the 64 lanes' 16 bytes land at consecutive addresses),
// four stages of 32 KB; which 16-byte piece of a row a lane fetches is chosen so that a row's pieces
// lie rotated by (row / 4) % 4 and the operand reads meet no bank conflict without padding. Every
// other k-step asks for two stages (the two halves of the same 128-byte lines). The operands of
// k-step i+1 are read from LDS between the MFMAs of k-step i, an operand of x as soon as two of this
// step's are used up, so that operands take 72 registers and nothing spills; the loop holds no vector
// instruction but MFMAs, LDS reads and the copies. Workgroups go to the XCDs round-robin by their
// number: an XCD gets a run of consecutive tiles, which are blocks of 4 x 8 tiles, so that its L2 holds
// what its tiles share. K may be split over `splits` workgroups per tile, each writing a 32-bit
// share [M, N] of its own. Needs K % (32 splits) == 0 and operands below 2 GiB; M, N arbitrary (rows
// beyond the edge are clamped on load and masked on store).
#include "common.h"
#include <type_traits>

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));

#define GT_BM 256
#define GT_BN 256
#define GT_BK 32
#define GT_STAGES 4
#define GT_HALF (GT_BM * GT_BK * 2)              // bytes of one operand's tile in a stage (16 KB)
#define GT_STAGE (2 * GT_HALF)                   // 32 KB
#define GT_LDS (GT_STAGES * GT_STAGE)            // 128 KB

template <int N>
__device__ __forceinline__ void gt_wait_copies() {
    // s_waitcnt vmcnt(N) alone: expcnt and lgkmcnt at their maxima
    __builtin_amdgcn_s_waitcnt(0x0F70 | N);
}

template <typename TO>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2))) void gemm_tile_kernel(
    const bf16* __restrict__ X, const bf16* __restrict__ W, TO* __restrict__ C, int M, int N, int K,
    int tiles_m, int tiles_n, int k_split, size_t slab) {
    extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];
    const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, n = lane & 15, g = lane >> 4;
    const int wm = wave >> 2, wn = wave & 3;

    // ---- which tile: workgroups go to the 8 XCDs round-robin; an XCD gets a run of consecutive
    // items, and consecutive items are blocks of 4 tile rows by 8 tile columns
    int item;
    {
        const int total = gridDim.x, id = blockIdx.x, xcd = id & 7, slot = id >> 3;
        const int q = total >> 3, r = total & 7;
        item = xcd * q + min(xcd, r) + slot;
    }
    const int per_z = tiles_m * tiles_n;
    const int z = item / per_z, t = item - z * per_z;
    int mt, nt;
    {
        const int GM = 4, span = GM * tiles_n, grp = t / span, first = grp * GM;
        const int gsize = min(tiles_m - first, GM), in = t - grp * span;
        mt = first + in % gsize;
        nt = in / gsize;
    }
    const int m0 = mt * GT_BM, n0 = nt * GT_BN;
    const int kbeg = z * k_split, kend = min(K, kbeg + k_split);
    const int nk = (kend - kbeg) / GT_BK;

    // ---- copies: wave w brings rows 32w .. 32w+31 of both tiles, 16 rows (1 KB) an instruction;
    // lane l writes piece l & 3 of row l >> 2, and reads the piece of x or W that belongs there.
    // A copy's address is the matrix (a buffer), a lane's offset and a uniform offset that moves on with k.
    const __amdgpu_buffer_rsrc_t xres = __builtin_amdgcn_make_buffer_rsrc((void*)X, 0, (int)((size_t)M * K * 2), 0x00020000);
    const __amdgpu_buffer_rsrc_t wres = __builtin_amdgcn_make_buffer_rsrc((void*)W, 0, (int)((size_t)N * K * 2), 0x00020000);
    const int r16 = lane >> 2, pc = (lane & 3) ^ ((r16 >> 2) & 3);
    int xoff[2], woff[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int row = 32 * wave + 16 * i + r16;
        xoff[i] = (int)(((size_t)min(m0 + row, M - 1) * K + kbeg + pc * 8) * 2);
        woff[i] = (int)(((size_t)min(n0 + row, N - 1) * K + kbeg + pc * 8) * 2);
    }
    unsigned char* copy_to = lds + (32 * wave) * 64;
    auto copy_stage = [&](int s, int kk) {            // k-step kk into stage s
        unsigned char* base = copy_to + s * GT_STAGE;
        const int soff = kk * (GT_BK * 2);
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            __builtin_amdgcn_raw_ptr_buffer_load_lds(xres, (void __attribute__((address_space(3)))*)(base + i * 1024), 16,
                                                     xoff[i], soff, 0, 0);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(wres, (void __attribute__((address_space(3)))*)(base + GT_HALF + i * 1024), 16,
                                                     woff[i], soff, 0, 0);
        }
    };

    // ---- operands: lane (n, g) reads row 16 b + n, piece g of the k-step, which lies at piece g ^ (n >> 2)
    const int rd = n * 64 + ((g ^ ((n >> 2) & 3)) * 16);
    // (two bases each, 64 KB apart, so that every read's offset fits the instruction's 16 bits)
    uint32_t xrd_lo = (uint32_t)(uintptr_t)(lds) + (wm * 128) * 64 + rd, xrd_hi = xrd_lo + 2 * GT_STAGE;
    uint32_t wrd_lo = (uint32_t)(uintptr_t)(lds) + GT_HALF + (wn * 64) * 64 + rd, wrd_hi = wrd_lo + 2 * GT_STAGE;
    asm volatile("" : "+v"(xrd_lo), "+v"(xrd_hi), "+v"(wrd_lo), "+v"(wrd_hi));
    typedef const bf16x8_t __attribute__((address_space(3)))* lds_frag_t;
    auto read_x = [&](int s, int b) { return *(lds_frag_t)(uintptr_t)((s < 2 ? xrd_lo : xrd_hi) + (s & 1) * GT_STAGE + b * 1024); };
    auto read_w = [&](int s, int a) { return *(lds_frag_t)(uintptr_t)((s < 2 ? wrd_lo : wrd_hi) + (s & 1) * GT_STAGE + a * 1024); };

    float4_t acc[4][8];
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int b = 0; b < 8; ++b) acc[a][b] = float4_t{0.f, 0.f, 0.f, 0.f};

    // ---- start: three stages under way, the first one's operands in registers
    copy_stage(0, 0);
    if (nk > 1) copy_stage(1, 1);
    if (nk > 2) copy_stage(2, 2);
    if (nk > 2) gt_wait_copies<4>(); else gt_wait_copies<0>();      // stages 0 and 1 have landed
    __builtin_amdgcn_s_barrier();
    bf16x8_t fwA[4], fxA[8], fwB[4], fxB[8];
#pragma unroll
    for (int a = 0; a < 4; ++a) fwA[a] = read_w(0, a);
#pragma unroll
    for (int b = 0; b < 8; ++b) fxA[b] = read_x(0, b);

    // step it: its operands are in registers (fw_c, fx_c); stage it+1 is in LDS and is read into
    // (fw_n, fx_n) between the MFMAs, an operand of x as soon as two of this step's are used up;
    // stages it+2 and it+3 are on their way
    auto step = [&](int it, auto stage_c, auto steady_c, bf16x8_t (&fw_c)[4], bf16x8_t (&fx_c)[8],
                    bf16x8_t (&fw_n)[4], bf16x8_t (&fx_n)[8]) {
        constexpr int stage = decltype(stage_c)::value;       // it & 3
        constexpr bool steady = decltype(steady_c)::value;
        constexpr int nxt = (stage + 1) & 3;
        const bool more = steady || it + 1 < nk;
        // every other step asks for two stages, the halves of the same 128-byte lines of x and W
        if constexpr ((stage & 1) == 0) {
            if (steady || it + 3 < nk) copy_stage((stage + 3) & 3, it + 3);
            if (steady || it + 4 < nk) copy_stage(stage, it + 4);
        }
        if (more) {
#pragma unroll
            for (int a = 0; a < 4; ++a) fw_n[a] = read_w(nxt, a);
            fx_n[0] = read_x(nxt, 0);
            fx_n[1] = read_x(nxt, 1);
        }
#pragma unroll
        for (int b = 0; b < 8; ++b) {
#pragma unroll
            for (int a = 0; a < 4; ++a)
                acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fw_c[a], fx_c[b], acc[a][b], 0, 0, 0);
            if (more && b + 2 < 8) fx_n[b + 2] = read_x(nxt, b + 2);
        }
        if constexpr (steady) {
            __builtin_amdgcn_sched_group_barrier(0x100, 6, 0);
#pragma unroll
            for (int b = 0; b < 6; ++b) {
                __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                if constexpr ((stage & 1) == 0) {
                    if (b < 2) __builtin_amdgcn_sched_group_barrier(0x020, 2, 0);
                    else __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
                }
            }
            __builtin_amdgcn_sched_group_barrier(0x008, 8, 0);
        }
        // stage it+2 must have landed (for everyone) before the next step reads it
        if constexpr (steady) {
            if constexpr ((stage & 1) == 0) gt_wait_copies<8>(); else gt_wait_copies<4>();
        } else {
            gt_wait_copies<0>();
        }
        __builtin_amdgcn_s_barrier();
    };
    using std::integral_constant;
    constexpr integral_constant<bool, true> yes{};
    constexpr integral_constant<bool, false> no{};
    int it = 0;
    for (; it + 6 < nk; it += 4) {
        step(it, integral_constant<int, 0>{}, yes, fwA, fxA, fwB, fxB);
        step(it + 1, integral_constant<int, 1>{}, yes, fwB, fxB, fwA, fxA);
        step(it + 2, integral_constant<int, 2>{}, yes, fwA, fxA, fwB, fxB);
        step(it + 3, integral_constant<int, 3>{}, yes, fwB, fxB, fwA, fxA);
    }
    for (; it < nk; it += 4) {
        step(it, integral_constant<int, 0>{}, no, fwA, fxA, fwB, fxB);
        if (it + 1 < nk) step(it + 1, integral_constant<int, 1>{}, no, fwB, fxB, fwA, fxA);
        if (it + 2 < nk) step(it + 2, integral_constant<int, 2>{}, no, fwA, fxA, fwB, fxB);
        if (it + 3 < nk) step(it + 3, integral_constant<int, 3>{}, no, fwB, fxB, fwA, fxA);
    }
    MFMA_SETTLE();

    // ---- results: acc[a][b][e] = y[m0 + 128 wm + 16 b + n][n0 + 64 wn + 16 a + 4 g + e]
    TO* out = C + (size_t)z * slab;
#pragma unroll
    for (int b = 0; b < 8; ++b) {
        const int m = m0 + wm * 128 + 16 * b + n;
        if (m >= M) continue;
#pragma unroll
        for (int a = 0; a < 4; ++a) {
            const int col = n0 + wn * 64 + 16 * a + 4 * g;
            TO* dst = out + (size_t)m * N + col;
            if (col + 3 < N && (N & 3) == 0) {
                if constexpr (sizeof(TO) == 4) {
                    *reinterpret_cast<float4_t*>(dst) = acc[a][b];
                } else {
                    uint2 w;
                    w.x = (uint32_t)f2bf_bits(acc[a][b][0]) | ((uint32_t)f2bf_bits(acc[a][b][1]) << 16);
                    w.y = (uint32_t)f2bf_bits(acc[a][b][2]) | ((uint32_t)f2bf_bits(acc[a][b][3]) << 16);
                    *reinterpret_cast<uint2*>(dst) = w;
                }
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    if (col + e < N) dst[e] = from_f<TO>(acc[a][b][e]);
            }
        }
    }
}

// splits == 1: C [M, N] (bf16 or fp32). splits > 1: C fp32 [splits, M, N], K % (32 splits) == 0.
// RA_ERR_ARG for what the kernel does not take (the caller then uses another product).
extern "C" int ra_gemm_tile_bf16(const void* X, const void* W, void* C, int M, int N, int K, int splits,
                                 int out_dtype, void* stream) {
    if (M <= 0 || N <= 0) return RA_OK;
    if (K <= 0 || splits < 1 || K % (GT_BK * splits) != 0) return RA_ERR_ARG;
    if ((size_t)M * K * 2 > 0x7fffffffull || (size_t)N * K * 2 > 0x7fffffffull) return RA_ERR_ARG;
    if (splits > 1 && out_dtype != RA_DTYPE_F32) return RA_ERR_ARG;
    const int tm = (M + GT_BM - 1) / GT_BM, tn = (N + GT_BN - 1) / GT_BN;
    const long long total = (long long)tm * tn * splits;
    if (total > 0x7fffffff) return RA_ERR_ARG;
    hipStream_t st = (hipStream_t)stream;
    static bool raised[2] = {false, false};
    if (out_dtype == RA_DTYPE_F32) {
        auto kern = gemm_tile_kernel<float>;
        if (!raised[0]) {
            if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, GT_LDS) != hipSuccess) return RA_ERR_ARG;
            raised[0] = true;
        }
        hipLaunchKernelGGL(kern, dim3((unsigned)total), dim3(512), GT_LDS, st, (const bf16*)X, (const bf16*)W, (float*)C,
                           M, N, K, tm, tn, K / splits, (size_t)M * N);
    } else if (out_dtype == RA_DTYPE_BF16) {
        auto kern = gemm_tile_kernel<bf16>;
        if (!raised[1]) {
            if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, GT_LDS) != hipSuccess) return RA_ERR_ARG;
            raised[1] = true;
        }
        hipLaunchKernelGGL(kern, dim3((unsigned)total), dim3(512), GT_LDS, st, (const bf16*)X, (const bf16*)W, (bf16*)C,
                           M, N, K, tm, tn, K, (size_t)0);
    } else {
        return RA_ERR_ARG;
    }
    return ra_launch_status();
}
