// Row-wise kernels: embedding gather, residual add + RMSNorm, per-head RMSNorm, rotary
// rotation, cache write, the fused q/k/v preparation, SiLU-mul, residual add.
// Formulas: rollout/fused.py:6-17 (RMSNorm), rollout/attention.py:10-25 (rotation),
// rollout/fused.py:103-114 (SiLU-mul), rollout/cache.py:334-337 (cache write).
#include "common.h"

// ------------------------------------------------------------------ embedding
template <typename T>
__global__ void embed_kernel(const T* __restrict__ table, const int* __restrict__ ids,
                             float* __restrict__ out, int H, int V) {
    const int t = blockIdx.x;
    int id = ids[t];
    if (id < 0 || id >= V) id = 0;          // ids are checked on the host; never read outside the table
    const T* src = table + (size_t)id * H;
    float* dst = out + (size_t)t * H;
    for (int c = threadIdx.x; c < H; c += blockDim.x) dst[c] = to_f(src[c]);
}

// bf16 table, H % 8 == 0: eight columns a thread by one 16-byte load, all of a row's loads on their way at once
__global__ void embed_bf16x8_kernel(const bf16* __restrict__ table, const int* __restrict__ ids,
                                    float* __restrict__ out, int H, int V) {
    const int t = blockIdx.x;
    int id = ids[t];
    if (id < 0 || id >= V) id = 0;
    const bf16* src = table + (size_t)id * H;
    float* dst = out + (size_t)t * H;
    for (int c = threadIdx.x * 8; c < H; c += blockDim.x * 8) {
        const uint4 w = *reinterpret_cast<const uint4*>(src + c);
        const uint32_t u[4] = {w.x, w.y, w.z, w.w};
        float4 lo, hi;
        lo.x = __uint_as_float(u[0] << 16); lo.y = __uint_as_float(u[0] & 0xffff0000u);
        lo.z = __uint_as_float(u[1] << 16); lo.w = __uint_as_float(u[1] & 0xffff0000u);
        hi.x = __uint_as_float(u[2] << 16); hi.y = __uint_as_float(u[2] & 0xffff0000u);
        hi.z = __uint_as_float(u[3] << 16); hi.w = __uint_as_float(u[3] & 0xffff0000u);
        *reinterpret_cast<float4*>(dst + c) = lo;
        *reinterpret_cast<float4*>(dst + c + 4) = hi;
    }
}

extern "C" int ra_embed(const void* table, const int* ids, float* out, int T, int H, int V,
                        int dtype, void* stream) {
    if (T <= 0) return RA_OK;
    if (dtype == RA_DTYPE_BF16 && H % 8 == 0 && (reinterpret_cast<uintptr_t>(table) & 15) == 0 &&
        (reinterpret_cast<uintptr_t>(out) & 15) == 0) {
        const int threads = H / 8 >= 512 ? 512 : (H / 8 >= 256 ? 256 : 64);
        hipLaunchKernelGGL(embed_bf16x8_kernel, dim3(T), dim3(threads), 0, (hipStream_t)stream,
                           (const bf16*)table, ids, out, H, V);
        return ra_launch_status();
    }
    dim3 grid(T), block(256);
    if (dtype == RA_DTYPE_F32)
        hipLaunchKernelGGL(embed_kernel<float>, grid, block, 0, (hipStream_t)stream,
                           (const float*)table, ids, out, H, V);
    else
        hipLaunchKernelGGL(embed_kernel<bf16>, grid, block, 0, (hipStream_t)stream,
                           (const bf16*)table, ids, out, H, V);
    return ra_launch_status();
}

// ------------------------------------------------------------------ residual add + RMSNorm
// For output row m: r = rows ? rows[m] : m;  v = h[r] + delta[r];  out[m] = v * rsqrt(mean(v^2)+eps) * w.
// Without a row list the sum is written back to h (the residual stream moves on);
// with a row list h is left alone (nothing reads it afterwards).
template <typename T>
__global__ void add_rmsnorm_kernel(float* __restrict__ h, const T* __restrict__ delta,
                                   const float* __restrict__ w, float eps, T* __restrict__ out,
                                   const int* __restrict__ rows, int H) {
    __shared__ float scratch[16];
    const int m = blockIdx.x;
    const size_t r = rows ? (size_t)rows[m] : (size_t)m;
    float* hr = h + r * H;
    const T* dr = delta ? delta + r * H : nullptr;
    const bool write_back = (rows == nullptr) && (delta != nullptr);
    float ss = 0.f;
    for (int c = threadIdx.x; c < H; c += blockDim.x) {
        float v = hr[c];
        if (dr) v += to_f(dr[c]);
        if (write_back) hr[c] = v;
        ss += v * v;
    }
    ss = block_sum(ss, scratch);
    const float rstd = 1.0f / sqrtf(ss / (float)H + eps);
    T* o = out + (size_t)m * H;
    for (int c = threadIdx.x; c < H; c += blockDim.x) {
        float v = hr[c];                       // same thread wrote it above
        if (dr && !write_back) v += to_f(dr[c]);
        o[c] = from_f<T>(v * rstd * w[c]);
    }
}

// The same with 16-byte accesses and the row kept in registers between the two phases:
// H % 4 == 0 and H <= 4 * VPT * blockDim. One block per output row.
template <typename T, int VPT>
__global__ void add_rmsnorm_vec_kernel(float* __restrict__ h, const T* __restrict__ delta,
                                       const float* __restrict__ w, float eps, T* __restrict__ out,
                                       const int* __restrict__ rows, int H) {
    __shared__ float scratch[16];
    const int m = blockIdx.x;
    const size_t r = rows ? (size_t)rows[m] : (size_t)m;
    float4* hr = reinterpret_cast<float4*>(h + r * H);
    const bool write_back = (rows == nullptr) && (delta != nullptr);
    const int nv = H >> 2;
    float4 v[VPT];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        const int c = threadIdx.x + i * blockDim.x;
        v[i] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (c < nv) {
            v[i] = hr[c];
            if (delta) {
                if constexpr (sizeof(T) == 2) {
                    const uint2 d = *reinterpret_cast<const uint2*>(delta + r * H + 4 * c);
                    v[i].x += __uint_as_float(d.x << 16);
                    v[i].y += __uint_as_float(d.x & 0xffff0000u);
                    v[i].z += __uint_as_float(d.y << 16);
                    v[i].w += __uint_as_float(d.y & 0xffff0000u);
                } else {
                    const float4 d = *reinterpret_cast<const float4*>(delta + r * H + 4 * c);
                    v[i].x += d.x; v[i].y += d.y; v[i].z += d.z; v[i].w += d.w;
                }
            }
            if (write_back) hr[c] = v[i];
            ss += v[i].x * v[i].x + v[i].y * v[i].y + v[i].z * v[i].z + v[i].w * v[i].w;
        }
    }
    ss = block_sum(ss, scratch);
    const float rstd = 1.0f / sqrtf(ss / (float)H + eps);
    T* o = out + (size_t)m * H;
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
        const int c = threadIdx.x + i * blockDim.x;
        if (c < nv) {
            const float4 ww = reinterpret_cast<const float4*>(w)[c];
            const float a = v[i].x * rstd * ww.x, b = v[i].y * rstd * ww.y;
            const float cc = v[i].z * rstd * ww.z, d = v[i].w * rstd * ww.w;
            if constexpr (sizeof(T) == 2) {
                uint2 p;
                p.x = (uint32_t)f2bf_bits(a) | ((uint32_t)f2bf_bits(b) << 16);
                p.y = (uint32_t)f2bf_bits(cc) | ((uint32_t)f2bf_bits(d) << 16);
                *reinterpret_cast<uint2*>(o + 4 * c) = p;
            } else {
                *reinterpret_cast<float4*>(o + 4 * c) = make_float4(a, b, cc, d);
            }
        }
    }
}

extern "C" int ra_add_rmsnorm(float* h, const void* delta, const float* w, float eps, void* out,
                              const int* rows, int M, int H, int dtype, void* stream) {
    if (M <= 0) return RA_OK;
    hipStream_t st = (hipStream_t)stream;
    if (H % 4 == 0 && H <= 16384) {
        const int nv = H / 4;
        const int threads = nv <= 256 ? 256 : (nv <= 512 ? 512 : 1024);
        dim3 grid(M), block(threads);
        const bool one = nv <= threads;              // one vector per thread, else up to four
        if (dtype == RA_DTYPE_F32) {
            if (one) hipLaunchKernelGGL((add_rmsnorm_vec_kernel<float, 1>), grid, block, 0, st, h, (const float*)delta, w, eps, (float*)out, rows, H);
            else hipLaunchKernelGGL((add_rmsnorm_vec_kernel<float, 4>), grid, block, 0, st, h, (const float*)delta, w, eps, (float*)out, rows, H);
        } else {
            if (one) hipLaunchKernelGGL((add_rmsnorm_vec_kernel<bf16, 1>), grid, block, 0, st, h, (const bf16*)delta, w, eps, (bf16*)out, rows, H);
            else hipLaunchKernelGGL((add_rmsnorm_vec_kernel<bf16, 4>), grid, block, 0, st, h, (const bf16*)delta, w, eps, (bf16*)out, rows, H);
        }
        return ra_launch_status();
    }
    dim3 grid(M), block(H >= 2048 ? 512 : 256);
    if (dtype == RA_DTYPE_F32)
        hipLaunchKernelGGL(add_rmsnorm_kernel<float>, grid, block, 0, st, h,
                           (const float*)delta, w, eps, (float*)out, rows, H);
    else
        hipLaunchKernelGGL(add_rmsnorm_kernel<bf16>, grid, block, 0, st, h,
                           (const bf16*)delta, w, eps, (bf16*)out, rows, H);
    return ra_launch_status();
}

// The same where the part before left its result as n_slabs 32-bit shares [n_slabs, rows of h, H] (a
// product whose K was cut into pieces, one share each): delta = their sum in slab order, rounded to T
// as the one product's stored result would have been.
template <typename T>
__global__ void add_slabs_rmsnorm_kernel(float* __restrict__ h, const float* __restrict__ slabs, int n_slabs,
                                         size_t slab_stride, const float* __restrict__ w, float eps,
                                         T* __restrict__ out, const int* __restrict__ rows, int H) {
    __shared__ float scratch[16];
    const int m = blockIdx.x;
    const size_t r = rows ? (size_t)rows[m] : (size_t)m;
    float* hr = h + r * H;
    const float* sr = slabs + r * H;
    const bool write_back = rows == nullptr;
    auto delta_at = [&](int c) {
        float d = 0.f;
        for (int s = 0; s < n_slabs; ++s) d += sr[(size_t)s * slab_stride + c];
        return round_to<T>(d);
    };
    float ss = 0.f;
    for (int c = threadIdx.x; c < H; c += blockDim.x) {
        const float v = hr[c] + delta_at(c);
        if (write_back) hr[c] = v;
        ss += v * v;
    }
    ss = block_sum(ss, scratch);
    const float rstd = 1.0f / sqrtf(ss / (float)H + eps);
    T* o = out + (size_t)m * H;
    for (int c = threadIdx.x; c < H; c += blockDim.x) {
        float v = hr[c];                       // same thread wrote it above
        if (!write_back) v += delta_at(c);
        o[c] = from_f<T>(v * rstd * w[c]);
    }
}

// The same for H % 4 == 0, H <= 4096 C4 and S shares known at compile time: 16-byte accesses, every load
// of a thread asked for at once, the row kept in registers between the two phases. 1024 threads a row,
// C4 pieces of four columns a thread (piece i of thread c: columns 4 (c + 1024 i) ..).
template <typename T, int S, int C4>
__global__ __launch_bounds__(1024) void add_slabs_rmsnorm_vec_kernel(
    float* __restrict__ h, const float* __restrict__ slabs, size_t slab_stride, const float* __restrict__ w, float eps,
    T* __restrict__ out, const int* __restrict__ rows, int H) {
    __shared__ float scratch[16];
    const int m = blockIdx.x;
    const size_t r = rows ? (size_t)rows[m] : (size_t)m;
    bool in[C4];
    int cc[C4];
    float4 v[C4], ww[C4], sh[C4][S];
#pragma unroll
    for (int i = 0; i < C4; ++i) {
        const int c = threadIdx.x + 1024 * i;
        in[i] = c < (H >> 2);
        cc[i] = in[i] ? c : 0;
        v[i] = reinterpret_cast<const float4*>(h + r * H)[cc[i]];
#pragma unroll
        for (int s = 0; s < S; ++s) sh[i][s] = reinterpret_cast<const float4*>(slabs + (size_t)s * slab_stride + r * H)[cc[i]];
        ww[i] = reinterpret_cast<const float4*>(w)[cc[i]];
    }
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < C4; ++i) {
        float4 d = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
        for (int s = 0; s < S; ++s) { d.x += sh[i][s].x; d.y += sh[i][s].y; d.z += sh[i][s].z; d.w += sh[i][s].w; }
        v[i].x += round_to<T>(d.x); v[i].y += round_to<T>(d.y); v[i].z += round_to<T>(d.z); v[i].w += round_to<T>(d.w);
        if (in[i] && rows == nullptr) reinterpret_cast<float4*>(h + r * H)[cc[i]] = v[i];
        ss += in[i] ? v[i].x * v[i].x + v[i].y * v[i].y + v[i].z * v[i].z + v[i].w * v[i].w : 0.f;
    }
    ss = block_sum(ss, scratch);
    const float rstd = 1.0f / sqrtf(ss / (float)H + eps);
#pragma unroll
    for (int i = 0; i < C4; ++i) {
        if (!in[i]) continue;
        T* o = out + (size_t)m * H + 4 * cc[i];
        const float a = v[i].x * rstd * ww[i].x, b = v[i].y * rstd * ww[i].y, e = v[i].z * rstd * ww[i].z,
                    f = v[i].w * rstd * ww[i].w;
        if constexpr (sizeof(T) == 2) {
            uint2 p;
            p.x = (uint32_t)f2bf_bits(a) | ((uint32_t)f2bf_bits(b) << 16);
            p.y = (uint32_t)f2bf_bits(e) | ((uint32_t)f2bf_bits(f) << 16);
            *reinterpret_cast<uint2*>(o) = p;
        } else {
            *reinterpret_cast<float4*>(o) = make_float4(a, b, e, f);
        }
    }
}

template <typename T, int C4>
static bool launch_slabs_vec(int n_slabs, dim3 grid, hipStream_t st, float* h, const float* slabs, size_t stride,
                             const float* w, float eps, T* out, const int* rows, int H) {
    switch (n_slabs) {
        case 2: hipLaunchKernelGGL((add_slabs_rmsnorm_vec_kernel<T, 2, C4>), grid, dim3(1024), 0, st, h, slabs, stride, w, eps, out, rows, H); return true;
        case 4: hipLaunchKernelGGL((add_slabs_rmsnorm_vec_kernel<T, 4, C4>), grid, dim3(1024), 0, st, h, slabs, stride, w, eps, out, rows, H); return true;
        case 8: hipLaunchKernelGGL((add_slabs_rmsnorm_vec_kernel<T, 8, C4>), grid, dim3(1024), 0, st, h, slabs, stride, w, eps, out, rows, H); return true;
        default: return false;
    }
}

// slabs: fp32 [n_slabs, R, H] with R rows as h has them (slab_rows = R).
extern "C" int ra_add_slabs_rmsnorm(float* h, const float* slabs, int n_slabs, long long slab_rows, const float* w,
                                    float eps, void* out, const int* rows, int M, int H, int dtype, void* stream) {
    if (M <= 0) return RA_OK;
    if (n_slabs <= 0 || slab_rows <= 0 || H <= 0) return RA_ERR_ARG;
    hipStream_t st = (hipStream_t)stream;
    const size_t stride = (size_t)slab_rows * H;
    dim3 grid(M);
    if (H % 4 == 0 && H <= 4096) {
        const bool done = dtype == RA_DTYPE_F32
            ? launch_slabs_vec<float, 1>(n_slabs, grid, st, h, slabs, stride, w, eps, (float*)out, rows, H)
            : launch_slabs_vec<bf16, 1>(n_slabs, grid, st, h, slabs, stride, w, eps, (bf16*)out, rows, H);
        if (done) return ra_launch_status();
    } else if (H % 4 == 0 && H <= 8192) {
        const bool done = dtype == RA_DTYPE_F32
            ? launch_slabs_vec<float, 2>(n_slabs, grid, st, h, slabs, stride, w, eps, (float*)out, rows, H)
            : launch_slabs_vec<bf16, 2>(n_slabs, grid, st, h, slabs, stride, w, eps, (bf16*)out, rows, H);
        if (done) return ra_launch_status();
    }
    dim3 block(H >= 2048 ? 1024 : 256);
    if (dtype == RA_DTYPE_F32)
        hipLaunchKernelGGL(add_slabs_rmsnorm_kernel<float>, grid, block, 0, st, h, slabs, n_slabs, stride, w, eps,
                           (float*)out, rows, H);
    else
        hipLaunchKernelGGL(add_slabs_rmsnorm_kernel<bf16>, grid, block, 0, st, h, slabs, n_slabs, stride, w, eps,
                           (bf16*)out, rows, H);
    return ra_launch_status();
}

// ------------------------------------------------------------------ residual add alone
template <typename T>
__global__ void residual_add_kernel(float* __restrict__ h, const T* __restrict__ delta, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) h[i] += to_f(delta[i]);
}

extern "C" int ra_residual_add(float* h, const void* delta, long long n, int dtype, void* stream) {
    if (n <= 0) return RA_OK;
    dim3 block(256), grid((unsigned)((n + 255) / 256));
    if (dtype == RA_DTYPE_F32)
        hipLaunchKernelGGL(residual_add_kernel<float>, grid, block, 0, (hipStream_t)stream, h,
                           (const float*)delta, (size_t)n);
    else
        hipLaunchKernelGGL(residual_add_kernel<bf16>, grid, block, 0, (hipStream_t)stream, h,
                           (const bf16*)delta, (size_t)n);
    return ra_launch_status();
}

// ------------------------------------------------------------------ per-head RMSNorm, in place
// x: [T, heads, D], one wave per (token, head).
template <typename T>
__global__ void head_rmsnorm_kernel(T* __restrict__ x, const float* __restrict__ w, float eps,
                                    long long n_rows, int D) {
    const long long row = (long long)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (row >= n_rows) return;
    const int lane = threadIdx.x & 63;
    T* p = x + row * D;
    float ss = 0.f;
    for (int c = lane; c < D; c += 64) {
        float v = to_f(p[c]);
        ss += v * v;
    }
    ss = wave_sum(ss);
    const float rstd = 1.0f / sqrtf(ss / (float)D + eps);
    for (int c = lane; c < D; c += 64) p[c] = from_f<T>(to_f(p[c]) * rstd * w[c]);
}

extern "C" int ra_head_rmsnorm(void* x, const float* w, float eps, long long n_rows, int D,
                               int dtype, void* stream) {
    if (n_rows <= 0) return RA_OK;
    dim3 block(256), grid((unsigned)((n_rows + 3) / 4));
    if (dtype == RA_DTYPE_F32)
        hipLaunchKernelGGL(head_rmsnorm_kernel<float>, grid, block, 0, (hipStream_t)stream,
                           (float*)x, w, eps, n_rows, D);
    else
        hipLaunchKernelGGL(head_rmsnorm_kernel<bf16>, grid, block, 0, (hipStream_t)stream,
                           (bf16*)x, w, eps, n_rows, D);
    return ra_launch_status();
}

// ------------------------------------------------------------------ rotary rotation, in place
// x: [T, heads, D]; pairs (j, j + R/2) for j < R/2; cos/sin: [max_pos, R/2] fp32.
template <typename T>
__global__ void rope_kernel(T* __restrict__ x, const int* __restrict__ positions,
                            const float* __restrict__ cos_t, const float* __restrict__ sin_t,
                            int T_tokens, int heads, int D, int R) {
    const int half = R >> 1;
    const long long total = (long long)T_tokens * heads * half;
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const int j = (int)(i % half);
    const long long th = i / half;               // token * heads + head
    const int t = (int)(th / heads);
    const int pos = positions[t];
    const float c = cos_t[(size_t)pos * half + j], s = sin_t[(size_t)pos * half + j];
    T* p = x + th * D;
    const float x1 = to_f(p[j]), x2 = to_f(p[j + half]);
    p[j] = from_f<T>(x1 * c - x2 * s);
    p[j + half] = from_f<T>(x2 * c + x1 * s);
}

extern "C" int ra_rope(void* x, const int* positions, const float* cos_t, const float* sin_t,
                       int T_tokens, int heads, int D, int R, int dtype, void* stream) {
    const long long total = (long long)T_tokens * heads * (R / 2);
    if (total <= 0) return RA_OK;
    dim3 block(256), grid((unsigned)((total + 255) / 256));
    if (dtype == RA_DTYPE_F32)
        hipLaunchKernelGGL(rope_kernel<float>, grid, block, 0, (hipStream_t)stream, (float*)x,
                           positions, cos_t, sin_t, T_tokens, heads, D, R);
    else
        hipLaunchKernelGGL(rope_kernel<bf16>, grid, block, 0, (hipStream_t)stream, (bf16*)x,
                           positions, cos_t, sin_t, T_tokens, heads, D, R);
    return ra_launch_status();
}

// ------------------------------------------------------------------ split fused qkv rows into q, k, v
template <typename T>
__global__ void split_heads_kernel(const T* __restrict__ qkv, T* __restrict__ q, T* __restrict__ k,
                                   T* __restrict__ v, int qw, int kw) {
    const int t = blockIdx.x;
    const int W = qw + 2 * kw;
    const T* src = qkv + (size_t)t * W;
    for (int c = threadIdx.x; c < W; c += blockDim.x) {
        if (c < qw) q[(size_t)t * qw + c] = src[c];
        else if (c < qw + kw) k[(size_t)t * kw + (c - qw)] = src[c];
        else v[(size_t)t * kw + (c - qw - kw)] = src[c];
    }
}

extern "C" int ra_split_heads(const void* qkv, void* q, void* k, void* v, int T_tokens, int qw,
                              int kw, int dtype, void* stream) {
    if (T_tokens <= 0) return RA_OK;
    dim3 grid(T_tokens), block(256);
    if (dtype == RA_DTYPE_F32)
        hipLaunchKernelGGL(split_heads_kernel<float>, grid, block, 0, (hipStream_t)stream,
                           (const float*)qkv, (float*)q, (float*)k, (float*)v, qw, kw);
    else
        hipLaunchKernelGGL(split_heads_kernel<bf16>, grid, block, 0, (hipStream_t)stream,
                           (const bf16*)qkv, (bf16*)q, (bf16*)k, (bf16*)v, qw, kw);
    return ra_launch_status();
}

// ------------------------------------------------------------------ cache write
// k, v: [T, Hkv*D] rows; pools: [pages, Hkv, P, D]; slot[t] = page*P + row in the page.
template <typename T>
__global__ void kv_write_kernel(const T* __restrict__ k, const T* __restrict__ v,
                                T* __restrict__ k_pool, T* __restrict__ v_pool,
                                const int* __restrict__ slots, int Hkv, int D, int P, long long pool_rows) {
    const int t = blockIdx.x;
    const long long s = slots[t];
    if (s < 0 || s >= pool_rows) return;        // tables are built on the host; never write outside the pool
    const int W = Hkv * D;
    for (int c = threadIdx.x; c < W; c += blockDim.x) {
        const int kvh = c / D;
        const size_t at = ra_cache_offset(s, kvh, Hkv, P, D) + (c - kvh * D);
        k_pool[at] = k[(size_t)t * W + c];
        v_pool[at] = v[(size_t)t * W + c];
    }
}

extern "C" int ra_kv_write(const void* k, const void* v, void* k_pool, void* v_pool,
                           const int* slots, int T_tokens, int Hkv, int D, int P, long long pool_rows, int dtype,
                           void* stream) {
    if (T_tokens <= 0) return RA_OK;
    if (Hkv <= 0 || D <= 0 || P <= 0) return RA_ERR_ARG;
    dim3 grid(T_tokens), block(256);
    if (dtype == RA_DTYPE_F32)
        hipLaunchKernelGGL(kv_write_kernel<float>, grid, block, 0, (hipStream_t)stream,
                           (const float*)k, (const float*)v, (float*)k_pool, (float*)v_pool, slots,
                           Hkv, D, P, pool_rows);
    else
        hipLaunchKernelGGL(kv_write_kernel<bf16>, grid, block, 0, (hipStream_t)stream,
                           (const bf16*)k, (const bf16*)v, (bf16*)k_pool, (bf16*)v_pool, slots, Hkv, D, P,
                           pool_rows);
    return ra_launch_status();
}

// ------------------------------------------------------------------ fused q/k/v preparation
// One wave per (token, head) over the fused projection row [q heads | k heads | v heads]:
//   q, k heads: optional RMSNorm over D with one weight for all heads, then optional rotation
//   by the token's position; q goes to q_out [T, Hq, D], k and v go to their cache rows.
// D <= 512 (each lane keeps at most 4 rotary pairs and 4 pass-through values).
#define QKV_MAX_PER_LANE 4
template <typename T>
__global__ void qkv_prepare_kernel(const T* __restrict__ qkv, int Hq, int Hkv, int D,
                                   const float* __restrict__ wq, const float* __restrict__ wk,
                                   float eps, const int* __restrict__ positions,
                                   const float* __restrict__ cos_t, const float* __restrict__ sin_t,
                                   int R, T* __restrict__ q_out, T* __restrict__ k_pool,
                                   T* __restrict__ v_pool, const int* __restrict__ slots, int P,
                                   long long pool_rows, long long n_rows) {
    const long long row = (long long)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (row >= n_rows) return;
    const int lane = threadIdx.x & 63;
    const int heads = Hq + 2 * Hkv;
    const int t = (int)(row / heads);
    const int head = (int)(row % heads);
    const T* src = qkv + row * D;

    T* dst;
    const float* w = nullptr;
    bool rotate = false;
    if (head < Hq) {
        dst = q_out + ((size_t)t * Hq + head) * D;
        w = wq;
        rotate = R > 0;
    } else {
        const int kvh = (head - Hq) % Hkv;
        const bool is_k = head < Hq + Hkv;
        T* pool = is_k ? k_pool : v_pool;
        if (pool == nullptr) return;
        const long long s = slots[t];
        if (s < 0 || s >= pool_rows) return;
        dst = pool + ra_cache_offset(s, kvh, Hkv, P, D);
        if (is_k) {
            w = wk;
            rotate = R > 0;
        }
    }

    const int half = R >> 1;
    float a[QKV_MAX_PER_LANE], b[QKV_MAX_PER_LANE], p[QKV_MAX_PER_LANE];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < QKV_MAX_PER_LANE; ++i) {
        const int j = lane + 64 * i;
        a[i] = b[i] = p[i] = 0.f;
        if (j < half) {
            a[i] = to_f(src[j]);
            b[i] = to_f(src[j + half]);
        }
        const int c = R + lane + 64 * i;
        if (c < D) p[i] = to_f(src[c]);
        ss += a[i] * a[i] + b[i] * b[i] + p[i] * p[i];
    }
    float rstd = 1.f;
    if (w != nullptr) {
        ss = wave_sum(ss);
        rstd = 1.0f / sqrtf(ss / (float)D + eps);
    }
    float cs[QKV_MAX_PER_LANE], sn[QKV_MAX_PER_LANE];
    const int pos = rotate ? positions[t] : 0;
#pragma unroll
    for (int i = 0; i < QKV_MAX_PER_LANE; ++i) {
        const int j = lane + 64 * i;
        cs[i] = 1.f;
        sn[i] = 0.f;
        if (rotate && j < half) {
            cs[i] = cos_t[(size_t)pos * half + j];
            sn[i] = sin_t[(size_t)pos * half + j];
        }
    }
#pragma unroll
    for (int i = 0; i < QKV_MAX_PER_LANE; ++i) {
        const int j = lane + 64 * i;
        if (j < half) {
            float x1 = a[i], x2 = b[i];
            if (w != nullptr) {
                x1 = x1 * rstd * w[j];
                x2 = x2 * rstd * w[j + half];
            }
            dst[j] = from_f<T>(x1 * cs[i] - x2 * sn[i]);
            dst[j + half] = from_f<T>(x2 * cs[i] + x1 * sn[i]);
        }
        const int c = R + lane + 64 * i;
        if (c < D) {
            float x = p[i];
            if (w != nullptr) x = x * rstd * w[c];
            dst[c] = from_f<T>(x);
        }
    }
}

// The same for bfloat16 with 16-byte accesses, when the whole head rotates (R == D) or nothing
// does (R == 0) and D % 16 == 0: a group of GP lanes (a power of two >= D/16) takes one
// (token, head); a lane holds eight elements of the first half and their eight partners of the
// second half, so a rotary pair never leaves its lane.
typedef uint32_t qkv_u4 __attribute__((ext_vector_type(4)));
typedef float qkv_f4 __attribute__((ext_vector_type(4)));
template <int GP>
__global__ __launch_bounds__(256) void qkv_prepare_bf16x8_kernel(
    const bf16* __restrict__ qkv, int Hq, int Hkv, int D, const float* __restrict__ wq,
    const float* __restrict__ wk, float eps, const int* __restrict__ positions,
    const float* __restrict__ cos_t, const float* __restrict__ sin_t, int R, bf16* __restrict__ q_out,
    bf16* __restrict__ k_pool, bf16* __restrict__ v_pool, const int* __restrict__ slots, int P,
    long long pool_rows, long long n_rows) {
    const long long row = ((long long)blockIdx.x * 256 + threadIdx.x) / GP;      // (token, head)
    const int sub = threadIdx.x % GP;
    const int half = D >> 1;
    const int j0 = sub * 8;
    const int heads = Hq + 2 * Hkv;
    const bool in = row < n_rows && j0 < half;
    const int t = in ? (int)(row / heads) : 0;
    const int head = in ? (int)(row % heads) : 0;
    const bf16* src = qkv + (in ? row : 0) * D;

    bf16* dst = nullptr;
    const float* w = nullptr;
    bool rotate = false;
    if (in) {
        if (head < Hq) {
            dst = q_out + ((size_t)t * Hq + head) * D;
            w = wq;
            rotate = R > 0;
        } else {
            const int kvh = (head - Hq) % Hkv;
            const bool is_k = head < Hq + Hkv;
            bf16* pool = is_k ? k_pool : v_pool;
            const long long s = slots[t];
            if (pool != nullptr && s >= 0 && s < pool_rows) dst = pool + ra_cache_offset(s, kvh, Hkv, P, D);
            if (is_k) {
                w = wk;
                rotate = R > 0;
            }
        }
    }
    float a[8], b[8];
    if (in) {
        const qkv_u4 a4 = *reinterpret_cast<const qkv_u4*>(src + j0);
        const qkv_u4 b4 = *reinterpret_cast<const qkv_u4*>(src + half + j0);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            a[2 * i] = __uint_as_float(a4[i] << 16);
            a[2 * i + 1] = __uint_as_float(a4[i] & 0xffff0000u);
            b[2 * i] = __uint_as_float(b4[i] << 16);
            b[2 * i + 1] = __uint_as_float(b4[i] & 0xffff0000u);
        }
    } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) a[i] = b[i] = 0.f;
    }
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) ss += a[i] * a[i] + b[i] * b[i];
#pragma unroll
    for (int o = GP / 2; o > 0; o >>= 1) ss += __shfl_xor(ss, o, 64);      // every lane of the wave takes part
    if (dst == nullptr) return;
    if (w != nullptr) {
        const float rstd = 1.0f / sqrtf(ss / (float)D + eps);
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const qkv_f4 w1 = *reinterpret_cast<const qkv_f4*>(w + j0 + 4 * i);
            const qkv_f4 w2 = *reinterpret_cast<const qkv_f4*>(w + half + j0 + 4 * i);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                a[4 * i + e] = a[4 * i + e] * rstd * w1[e];
                b[4 * i + e] = b[4 * i + e] * rstd * w2[e];
            }
        }
    }
    if (rotate) {
        const size_t at = (size_t)positions[t] * half + j0;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const qkv_f4 c4 = *reinterpret_cast<const qkv_f4*>(cos_t + at + 4 * i);
            const qkv_f4 s4 = *reinterpret_cast<const qkv_f4*>(sin_t + at + 4 * i);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float x1 = a[4 * i + e], x2 = b[4 * i + e];
                a[4 * i + e] = x1 * c4[e] - x2 * s4[e];
                b[4 * i + e] = x2 * c4[e] + x1 * s4[e];
            }
        }
    }
    qkv_u4 oa, ob;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        oa[i] = (uint32_t)f2bf_bits(a[2 * i]) | ((uint32_t)f2bf_bits(a[2 * i + 1]) << 16);
        ob[i] = (uint32_t)f2bf_bits(b[2 * i]) | ((uint32_t)f2bf_bits(b[2 * i + 1]) << 16);
    }
    *reinterpret_cast<qkv_u4*>(dst + j0) = oa;
    *reinterpret_cast<qkv_u4*>(dst + half + j0) = ob;
}

template <int GP>
static void launch_qkv_prepare_x8(long long n_rows, hipStream_t st, const bf16* qkv, int Hq, int Hkv, int D,
                                  const float* wq, const float* wk, float eps, const int* positions,
                                  const float* cos_t, const float* sin_t, int R, bf16* q_out, bf16* k_pool,
                                  bf16* v_pool, const int* slots, int P, long long pool_rows) {
    const long long threads = n_rows * GP;
    hipLaunchKernelGGL(qkv_prepare_bf16x8_kernel<GP>, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0,
                       st, qkv, Hq, Hkv, D, wq, wk, eps, positions, cos_t, sin_t, R, q_out, k_pool, v_pool,
                       slots, P, pool_rows, n_rows);
}

extern "C" int ra_qkv_prepare(const void* qkv, int T_tokens, int Hq, int Hkv, int D, const float* wq,
                              const float* wk, float eps, const int* positions, const float* cos_t,
                              const float* sin_t, int R, void* q_out, void* k_pool, void* v_pool,
                              const int* slots, int P, long long pool_rows, int dtype, void* stream) {
    if (T_tokens <= 0) return RA_OK;
    if ((k_pool != nullptr || v_pool != nullptr) && P <= 0) return RA_ERR_ARG;
    if (D > 64 * QKV_MAX_PER_LANE * 2 || R > D || (R & 1)) return RA_ERR_ARG;
    // pairs: R/2 <= 256; pass-through: D-R <= 256
    if ((R >> 1) > 64 * QKV_MAX_PER_LANE || (D - R) > 64 * QKV_MAX_PER_LANE) return RA_ERR_ARG;
    const long long n_rows = (long long)T_tokens * (Hq + 2 * Hkv);
    if (dtype == RA_DTYPE_BF16 && D % 16 == 0 && (R == D || R == 0) && n_rows * 32 < (1ll << 31) * 256) {
        const int lanes = D / 16;                 // lanes that a head needs
#define QKV_X8(GP)                                                                                    \
    launch_qkv_prepare_x8<GP>(n_rows, (hipStream_t)stream, (const bf16*)qkv, Hq, Hkv, D, wq, wk, eps,  \
                              positions, cos_t, sin_t, R, (bf16*)q_out, (bf16*)k_pool, (bf16*)v_pool,  \
                              slots, P, pool_rows)
        if (lanes <= 1) QKV_X8(1);
        else if (lanes <= 2) QKV_X8(2);
        else if (lanes <= 4) QKV_X8(4);
        else if (lanes <= 8) QKV_X8(8);
        else if (lanes <= 16) QKV_X8(16);
        else QKV_X8(32);
#undef QKV_X8
        return ra_launch_status();
    }
    dim3 block(256), grid((unsigned)((n_rows + 3) / 4));
    if (dtype == RA_DTYPE_F32)
        hipLaunchKernelGGL(qkv_prepare_kernel<float>, grid, block, 0, (hipStream_t)stream,
                           (const float*)qkv, Hq, Hkv, D, wq, wk, eps, positions, cos_t, sin_t, R,
                           (float*)q_out, (float*)k_pool, (float*)v_pool, slots, P, pool_rows, n_rows);
    else
        hipLaunchKernelGGL(qkv_prepare_kernel<bf16>, grid, block, 0, (hipStream_t)stream,
                           (const bf16*)qkv, Hq, Hkv, D, wq, wk, eps, positions, cos_t, sin_t, R,
                           (bf16*)q_out, (bf16*)k_pool, (bf16*)v_pool, slots, P, pool_rows, n_rows);
    return ra_launch_status();
}

// ------------------------------------------------------------------ SiLU-mul
// gu: [T, 2I] with the gate in the first half; out: [T, I] = silu(g) * u.
template <typename T>
__global__ void silu_mul_kernel(const T* __restrict__ gu, T* __restrict__ out, int I, long long total) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const long long t = i / I;
    const int c = (int)(i % I);
    const float g = to_f(gu[t * 2 * I + c]);
    const float u = to_f(gu[t * 2 * I + I + c]);
    out[i] = from_f<T>(g / (1.0f + expf(-g)) * u);
}

// eight columns per thread with 16-byte accesses (bf16, I % 8 == 0)
__global__ void silu_mul_bf16x8_kernel(const bf16* __restrict__ gu, bf16* __restrict__ out, int I8,
                                       long long total8) {
    const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total8) return;
    const long long t = i / I8;
    const int c = (int)(i % I8) * 8;
    const int I = I8 * 8;
    const uint4 g4 = *reinterpret_cast<const uint4*>(gu + t * 2 * I + c);
    const uint4 u4 = *reinterpret_cast<const uint4*>(gu + t * 2 * I + I + c);
    const uint32_t gw[4] = {g4.x, g4.y, g4.z, g4.w}, uw[4] = {u4.x, u4.y, u4.z, u4.w};
    uint32_t o[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const float g0 = __uint_as_float(gw[k] << 16), g1 = __uint_as_float(gw[k] & 0xffff0000u);
        const float u0 = __uint_as_float(uw[k] << 16), u1 = __uint_as_float(uw[k] & 0xffff0000u);
        const float y0 = g0 / (1.0f + expf(-g0)) * u0, y1 = g1 / (1.0f + expf(-g1)) * u1;
        o[k] = (uint32_t)f2bf_bits(y0) | ((uint32_t)f2bf_bits(y1) << 16);
    }
    *reinterpret_cast<uint4*>(out + t * I + c) = make_uint4(o[0], o[1], o[2], o[3]);
}

extern "C" int ra_silu_mul(const void* gu, void* out, int T_tokens, int I, int dtype, void* stream) {
    const long long total = (long long)T_tokens * I;
    if (total <= 0) return RA_OK;
    if (dtype == RA_DTYPE_BF16 && I % 8 == 0) {
        const long long total8 = total / 8;
        hipLaunchKernelGGL(silu_mul_bf16x8_kernel, dim3((unsigned)((total8 + 255) / 256)), dim3(256), 0,
                           (hipStream_t)stream, (const bf16*)gu, (bf16*)out, I / 8, total8);
        return ra_launch_status();
    }
    dim3 block(256), grid((unsigned)((total + 255) / 256));
    if (dtype == RA_DTYPE_F32)
        hipLaunchKernelGGL(silu_mul_kernel<float>, grid, block, 0, (hipStream_t)stream,
                           (const float*)gu, (float*)out, I, total);
    else
        hipLaunchKernelGGL(silu_mul_kernel<bf16>, grid, block, 0, (hipStream_t)stream,
                           (const bf16*)gu, (bf16*)out, I, total);
    return ra_launch_status();
}
