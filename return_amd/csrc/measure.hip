// A plain streaming read, for measuring what a read-only kernel reaches on the machine at hand:
// the yardstick that a decode step's memory traffic is held against (bench.py reports the
// fraction of this rate beside the fraction of the published peak).
#include "common.h"

typedef uint32_t mu4_t __attribute__((ext_vector_type(4)));

// One workgroup per CU, 512 threads, grid-stride in units of 16 bytes per lane with four loads in
// flight per lane: the chip moves through memory as one front. The loaded words are folded into
// one word per thread so that no load can be dropped; one word per workgroup is stored.
__global__ __launch_bounds__(512) void stream_read_kernel(const mu4_t* __restrict__ src, size_t n_vec,
                                                          uint32_t* __restrict__ out) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    mu4_t acc = {0u, 0u, 0u, 0u};
    for (; i + 3 * stride < n_vec; i += 4 * stride) {
        const mu4_t a = __builtin_nontemporal_load(src + i);
        const mu4_t b = __builtin_nontemporal_load(src + i + stride);
        const mu4_t c = __builtin_nontemporal_load(src + i + 2 * stride);
        const mu4_t d = __builtin_nontemporal_load(src + i + 3 * stride);
        acc ^= a ^ b ^ c ^ d;
    }
    for (; i < n_vec; i += stride) acc ^= __builtin_nontemporal_load(src + i);
    uint32_t w = acc[0] ^ acc[1] ^ acc[2] ^ acc[3];
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) w ^= __shfl_xor(w, o, 64);
    __shared__ uint32_t part[8];
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = w;
    __syncthreads();
    if (threadIdx.x == 0) {
        uint32_t t = 0;
        for (int k = 0; k < 8; ++k) t ^= part[k];
        out[blockIdx.x] = t;
    }
}

// Reads `bytes` bytes (a multiple of 16, 16-byte aligned) at src once; out: `workgroups` 32-bit words.
extern "C" int ra_stream_read(const void* src, long long bytes, void* out, int workgroups, void* stream) {
    if (src == nullptr || out == nullptr || bytes <= 0 || bytes % 16 != 0 || workgroups <= 0 || workgroups > 65535 ||
        ((uintptr_t)src & 15) != 0)
        return RA_ERR_ARG;
    hipLaunchKernelGGL(stream_read_kernel, dim3(workgroups), dim3(512), 0, (hipStream_t)stream,
                       (const mu4_t*)src, (size_t)(bytes / 16), (uint32_t*)out);
    return ra_launch_status();
}
