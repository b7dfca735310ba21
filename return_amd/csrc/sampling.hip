// Token choice from fp32 logits: greedy, temperature, top-k, top-p; and the chosen token's
// log-probability under the raw logits. One block per row.
//
// What the reference samples with (rollout/model.py:15-61): temperature <= 0 is argmax;
// otherwise logits / temperature; keep the top_k largest; over the kept values in descending
// order drop every token before which more than top_p of the (top-k renormalised) mass
// already lies (the crossing token stays, the first always stays); draw from what is left.
// Logprob is log_softmax(raw logits)[token] (rollout/model.py:64-67).
//
// The draw uses a uniform number u in [0,1) that the host supplies per row: the token is the
// first, in vocabulary order, at which the running sum of kept probabilities exceeds u.
// Tokens that tie with the k-th value, or with the top-p boundary value, are all kept.
#include "common.h"

#define SAMPLE_THREADS 1024
#define SAMPLE_BUCKETS 32

__device__ __forceinline__ uint32_t order_key(float f) {
    const uint32_t b = __float_as_uint(f);
    return (b & 0x80000000u) ? ~b : (b | 0x80000000u);      // ascending float order -> ascending uint
}

// f(i, v) for every element of the row, four at a time where the row allows 16-byte loads
template <typename F>
__device__ __forceinline__ void for_each_logit(const float* __restrict__ x, int V, int tid, F f) {
    if ((V & 3) == 0 && (reinterpret_cast<uintptr_t>(x) & 15) == 0) {
        const float4* x4 = reinterpret_cast<const float4*>(x);
        const int n4 = V >> 2;
        int i = tid;
        for (; i + 7 * SAMPLE_THREADS < n4; i += 8 * SAMPLE_THREADS) {   // eight loads on their way per thread
            float4 a[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) a[j] = x4[i + j * SAMPLE_THREADS];
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int k = 4 * (i + j * SAMPLE_THREADS);
                f(k, a[j].x); f(k + 1, a[j].y); f(k + 2, a[j].z); f(k + 3, a[j].w);
            }
        }
        for (; i < n4; i += SAMPLE_THREADS) {
            const float4 a = x4[i];
            f(4 * i, a.x); f(4 * i + 1, a.y); f(4 * i + 2, a.z); f(4 * i + 3, a.w);
        }
    } else {
        for (int i = tid; i < V; i += SAMPLE_THREADS) f(i, x[i]);
    }
}

// The smallest key t in [lo, hi] with measure{key > t} <= limit, where the measure of a token is 1
// (MASS false: counts, exact in 32-bit floats below 2^24) or exp((x - gmax) * inv_t) (MASS true), and
// measure{key > hi} = above_hi <= limit. Every pass over the row cuts [lo, hi] into up to 32 runs of
// equal width and finds the run that holds t, so that a range of 2^32 keys takes seven passes. A thread
// adds what its tokens weigh into bins of its own in LDS ([run][thread]); the bins are then added over
// the threads in a fixed order, so that the result is the same in every run of the program.
template <bool MASS>
__device__ uint32_t find_threshold(const float* __restrict__ x, int V, int tid, uint32_t lo, uint32_t hi,
                                   float above_hi, float limit, float gmax, float inv_t, float* bins, float* part2,
                                   float* tot, uint32_t* sh_range, float* sh_above) {
    while (lo < hi) {
        const uint32_t width = hi - lo;
        const int bits = 32 - __builtin_clz(width);
        const int sh = bits > 5 ? bits - 5 : 0;                  // (width >> sh) < 32
        const int nb = (int)(width >> sh) + 1;
#pragma unroll
        for (int b = 0; b < SAMPLE_BUCKETS; ++b) bins[b * SAMPLE_THREADS + tid] = 0.f;
        for_each_logit(x, V, tid, [&](int, float v) {
            const uint32_t key = order_key(v);
            if (key > lo && key <= hi) {
                const float w = MASS ? expf((v - gmax) * inv_t) : 1.0f;
                bins[((key - lo) >> sh) * SAMPLE_THREADS + tid] += w;
            }
        });
        __syncthreads();
        {                                                       // thread (b, j) adds bins[b][j], [j + 32], ...
            const int b = tid >> 5, j = tid & 31;
            float t = 0.f;
#pragma unroll 8
            for (int i = 0; i < SAMPLE_THREADS / 32; ++i) t += bins[b * SAMPLE_THREADS + j + 32 * i];
            part2[tid] = t;
        }
        __syncthreads();
        if (tid < SAMPLE_BUCKETS) {
            float t = 0.f;
#pragma unroll 8
            for (int j = 0; j < 32; ++j) t += part2[tid * 32 + j];
            tot[tid] = t;
        }
        __syncthreads();
        if (tid == 0) {
            // run b ends at key T_b = lo + ((b + 1) << sh) - 1; the measure above T_b is above_hi plus the
            // runs above b. t lies in the lowest run whose end has at most `limit` above it.
            float above = above_hi;
            int b = nb - 1;
            while (b > 0 && above + tot[b] <= limit) {
                above += tot[b];
                --b;
            }
            const unsigned long long end = (unsigned long long)lo + (((unsigned long long)b + 1ull) << sh) - 1ull;
            sh_range[1] = end < (unsigned long long)hi ? (uint32_t)end : hi;
            sh_range[0] = b == 0 ? lo : lo + ((uint32_t)b << sh);   // the run below ends with more than `limit` above it
            sh_above[0] = above;
        }
        __syncthreads();
        lo = sh_range[0];
        hi = sh_range[1];
        above_hi = sh_above[0];
        __syncthreads();
    }
    return lo;
}

__global__ __launch_bounds__(SAMPLE_THREADS) void sample_kernel(
    const float* __restrict__ logits, int V, const float* __restrict__ temperature,
    const int* __restrict__ top_k, const float* __restrict__ top_p, const float* __restrict__ u,
    int* __restrict__ out) {
    extern __shared__ __attribute__((aligned(16))) float bins[];          // [SAMPLE_BUCKETS][SAMPLE_THREADS]
    __shared__ float scratch[16];
    __shared__ float part[SAMPLE_THREADS];
    __shared__ float tot[SAMPLE_BUCKETS];
    __shared__ uint32_t sh_range[2];
    __shared__ int sh_int[4];
    __shared__ float sh_f[2];
    const int row = blockIdx.x, tid = threadIdx.x;
    const float* x = logits + (size_t)row * V;

    // ---- one pass: running maximum, first index that holds it, sum of exp(x - maximum)
    float mx = -INFINITY, se = 0.f;
    int arg = 0x7fffffff;
    for_each_logit(x, V, tid, [&](int i, float v) {
        if (v > mx) {
            se = se * __expf(mx - v) + 1.0f;          // mx = -inf: se is 0 and stays finite
            mx = v;
            arg = i;
        } else {
            se += __expf(v - mx);
        }
    });
    // merge (mx, se, arg) over the wave, then over the waves in wave order
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const float m2 = __shfl_xor(mx, o, 64), s2 = __shfl_xor(se, o, 64);
        const int a2 = __shfl_xor(arg, o, 64);
        const float m = fmaxf(mx, m2);
        const float s1 = (mx == -INFINITY) ? 0.f : se * __expf(mx - m);
        const float s3 = (m2 == -INFINITY) ? 0.f : s2 * __expf(m2 - m);
        arg = (m2 > mx) ? a2 : ((m2 == mx) ? min(arg, a2) : arg);
        se = s1 + s3;                                 // the same two numbers in both lanes of a pair
        mx = m;
    }
    __shared__ float wm[16], ws[16];
    __shared__ int wa[16];
    if ((tid & 63) == 0) { wm[tid >> 6] = mx; ws[tid >> 6] = se; wa[tid >> 6] = arg; }
    __syncthreads();
    float gmax = wm[0];
    int argmax = wa[0];
    for (int w = 1; w < SAMPLE_THREADS / 64; ++w) {
        if (wm[w] > gmax) { gmax = wm[w]; argmax = wa[w]; }
        else if (wm[w] == gmax) argmax = min(argmax, wa[w]);
    }
    float total_e = 0.f;
    for (int w = 0; w < SAMPLE_THREADS / 64; ++w)
        total_e += (wm[w] == -INFINITY) ? 0.f : ws[w] * __expf(wm[w] - gmax);
    const float lse = gmax + logf(total_e);

    const float temp = temperature[row];
    if (!(temp > 0.f)) {
        if (tid == 0) {
            out[2 * row] = argmax;
            out[2 * row + 1] = __float_as_int(x[argmax] - lse);
        }
        return;
    }
    const float inv_t = 1.0f / temp;
    const uint32_t top_key = order_key(gmax);

    // ---- top-k: the key of the k-th largest value is the smallest key with at most k - 1 tokens above it
    uint32_t keep_key = 0u;                   // keep tokens whose key >= keep_key
    const int k = top_k[row];
    if (k > 0 && k < V)
        keep_key = find_threshold<false>(x, V, tid, 0u, top_key, 0.f, (float)(k - 1), gmax, inv_t, bins, part, tot,
                                         sh_range, sh_f);

    // ---- top-p: the smallest key with at most p of the kept mass above it
    const float p = top_p[row];
    if (p < 1.0f) {
        float z = 0.f;
        for_each_logit(x, V, tid, [&](int, float v) {
            if (order_key(v) >= keep_key) z += expf((v - gmax) * inv_t);
        });
        z = block_sum(z, scratch);
        keep_key = find_threshold<true>(x, V, tid, keep_key, top_key, 0.f, p * z, gmax, inv_t, bins, part, tot,
                                        sh_range, sh_f);
    }

    // ---- inverse CDF in vocabulary order: contiguous chunk per thread
    const int chunk = (V + SAMPLE_THREADS - 1) / SAMPLE_THREADS;
    const int i0 = min(V, tid * chunk), i1 = min(V, i0 + chunk);
    float mine = 0.f;
    for (int i = i0; i < i1; ++i)
        if (order_key(x[i]) >= keep_key) mine += expf((x[i] - gmax) * inv_t);
    __syncthreads();
    part[tid] = mine;
    __syncthreads();
    if (tid == 0) {
        float total = 0.f;
        for (int i = 0; i < SAMPLE_THREADS; ++i) total += part[i];
        const float target = u[row] * total;
        float run = 0.f, before = 0.f;
        int owner = -1;
        for (int i = 0; i < SAMPLE_THREADS; ++i) {
            if (part[i] > 0.f) {
                owner = i;                           // the last chunk with kept mass if the target is never passed
                before = run;
                if (run + part[i] > target) break;
                run += part[i];
            }
        }
        sh_int[3] = owner < 0 ? 0 : owner;
        sh_f[0] = before;
        sh_f[1] = target;
    }
    __syncthreads();
    if (tid == sh_int[3]) {
        float run = sh_f[0];
        const float target = sh_f[1];
        int tok = -1;
        for (int i = i0; i < i1; ++i) {
            if (order_key(x[i]) >= keep_key) {
                tok = i;                             // last kept token of the chunk if never passed
                run += expf((x[i] - gmax) * inv_t);
                if (run > target) break;
            }
        }
        if (tok < 0) tok = argmax;
        out[2 * row] = tok;
        out[2 * row + 1] = __float_as_int(x[tok] - lse);
    }
}

extern "C" int ra_sample(const float* logits, int M, int V, const float* temperature,
                         const int* top_k, const float* top_p, const float* u, int* out,
                         void* stream) {
    if (M <= 0) return RA_OK;
    if (V <= 0) return RA_ERR_ARG;
    const size_t lds = (size_t)SAMPLE_BUCKETS * SAMPLE_THREADS * sizeof(float);   // 128 KB: each thread's bins
    static bool allowed = false;
    if (!allowed) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(sample_kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)lds) != hipSuccess)
            return RA_ERR_ARG;
        allowed = true;
    }
    hipLaunchKernelGGL(sample_kernel, dim3(M), dim3(SAMPLE_THREADS), lds, (hipStream_t)stream, logits,
                       V, temperature, top_k, top_p, u, out);
    return ra_launch_status();
}
