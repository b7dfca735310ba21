// Shared device helpers for the gfx950 kernels of return_amd.
// Storage types: float, or bf16 (raw 16 bits, round-to-nearest-even on store).
// All arithmetic is done in float.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define RA_OK 0
#define RA_ERR_ARG 1
#define RA_ERR_LAUNCH 2

struct bf16 {
    uint16_t x;
};

__device__ __forceinline__ float to_f(float v) { return v; }
__device__ __forceinline__ float to_f(bf16 v) { return __uint_as_float(((uint32_t)v.x) << 16); }

__device__ __forceinline__ uint16_t f2bf_bits(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return 0x7fc0;      // NaN stays NaN
    u += 0x7fffu + ((u >> 16) & 1u);                           // round to nearest even
    return (uint16_t)(u >> 16);
}

template <typename T> __device__ __forceinline__ T from_f(float f);
template <> __device__ __forceinline__ float from_f<float>(float f) { return f; }
template <> __device__ __forceinline__ bf16 from_f<bf16>(float f) {
    bf16 r;
    r.x = f2bf_bits(f);
    return r;
}

// value rounded to the storage type and back: what a later kernel will read
template <typename T> __device__ __forceinline__ float round_to(float f) { return to_f(from_f<T>(f)); }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}

// Sum over a block of up to 1024 threads; every thread gets the result. scratch: >= 16 floats of LDS.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int nwave = (blockDim.x + 63) >> 6;
    v = wave_sum(v);
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float t = 0.f;
    for (int i = 0; i < nwave; ++i) t += scratch[i];      // same order in every thread
    return t;
}
__device__ __forceinline__ float block_max(float v, float* scratch) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int nwave = (blockDim.x + 63) >> 6;
    v = wave_max(v);
    __syncthreads();
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float t = scratch[0];
    for (int i = 1; i < nwave; ++i) t = fmaxf(t, scratch[i]);
    return t;
}

// Maximum and sum over the four 16-lane rows of a wave (lanes l, l^16, l^32, l^48), the result
// in every lane, by the lane swaps of gfx950: v_permlane16_swap exchanges the odd rows of its
// first operand with the even rows of its second, v_permlane32_swap the upper half of the first
// with the lower half of the second; with the same value in both operands the two results hold
// the two partners of every lane. No LDS round trip as with a shuffle. The sum is
// (row0 + row1) + (row2 + row3) in every lane.
typedef unsigned ra_uint2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ float rows_max(float v) {
    ra_uint2_t r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
    r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float rows_sum(float v) {
    ra_uint2_t r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = __uint_as_float(r[0]) + __uint_as_float(r[1]);
    r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// The cache pools are [page][kv head][row in page][D]: the rows that one kv head has in a page lie
// side by side, so that a kernel that walks through the keys of one kv head reads runs of P rows.
// Offset (elements) of the row with slot number page * P + row in page, for kv head kvh.
__host__ __device__ __forceinline__ size_t ra_cache_offset(long long slot, int kvh, int Hkv, int P, int D) {
    const long long page = slot / P;
    return (((size_t)page * Hkv + kvh) * P + (size_t)(slot - page * P)) * D;
}

static inline int ra_launch_status() {
    return hipGetLastError() == hipSuccess ? RA_OK : RA_ERR_LAUNCH;
}

// Placed between the last MFMA of a chain and the first read of its result. hipcc inserts
// the wait states an MFMA result needs only when producer and reader sit in one basic block;
// with a branch in between (a mask, a loop exit) the 16x16x32 bf16 result was read too early
// on gfx950 and its last register still held the previous value. Nothing is scheduled across.
#define MFMA_SETTLE()                        \
    do {                                     \
        __builtin_amdgcn_sched_barrier(0);   \
        asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 7" ::: "memory"); \
        __builtin_amdgcn_sched_barrier(0);   \
    } while (0)

#define RA_DTYPE_F32 0
#define RA_DTYPE_BF16 1
