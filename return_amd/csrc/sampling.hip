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

__device__ __forceinline__ uint32_t order_key(float f) {
    const uint32_t b = __float_as_uint(f);
    return (b & 0x80000000u) ? ~b : (b | 0x80000000u);      // ascending float order -> ascending uint
}

__global__ __launch_bounds__(SAMPLE_THREADS) void sample_kernel(
    const float* __restrict__ logits, int V, const float* __restrict__ temperature,
    const int* __restrict__ top_k, const float* __restrict__ top_p, const float* __restrict__ u,
    int* __restrict__ out) {
    __shared__ float scratch[16];
    __shared__ float part[SAMPLE_THREADS];
    __shared__ int hist[256];
    __shared__ int sh_int[4];
    __shared__ float sh_f[2];
    const int row = blockIdx.x, tid = threadIdx.x;
    const float* x = logits + (size_t)row * V;

    // ---- one pass: running maximum, first index that holds it, sum of exp(x - maximum)
    float mx = -INFINITY, se = 0.f;
    int arg = 0x7fffffff;
    auto take = [&](float v, int i) {
        if (v > mx) {
            se = se * __expf(mx - v) + 1.0f;          // mx = -inf: se is 0 and stays finite
            mx = v;
            arg = i;
        } else {
            se += __expf(v - mx);
        }
    };
    if ((V & 3) == 0) {
        const float4* x4 = reinterpret_cast<const float4*>(x);
        for (int i = tid; i < (V >> 2); i += SAMPLE_THREADS) {
            const float4 v = x4[i];
            take(v.x, 4 * i); take(v.y, 4 * i + 1); take(v.z, 4 * i + 2); take(v.w, 4 * i + 3);
        }
    } else {
        for (int i = tid; i < V; i += SAMPLE_THREADS) take(x[i], i);
    }
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
    float tot = 0.f;
    for (int w = 0; w < SAMPLE_THREADS / 64; ++w)
        tot += (wm[w] == -INFINITY) ? 0.f : ws[w] * __expf(wm[w] - gmax);
    const float lse = gmax + logf(tot);

    const float temp = temperature[row];
    if (!(temp > 0.f)) {
        if (tid == 0) {
            out[2 * row] = argmax;
            out[2 * row + 1] = __float_as_int(x[argmax] - lse);
        }
        return;
    }
    const float inv_t = 1.0f / temp;

    // ---- top-k: key of the k-th largest value (radix select, 4 passes of 8 bits)
    uint32_t keep_key = 0u;                   // keep tokens whose key >= keep_key
    const int k = top_k[row];
    if (k > 0 && k < V) {
        uint32_t prefix = 0u, mask = 0u;
        int remaining = k;
        for (int shift = 24; shift >= 0; shift -= 8) {
            if (tid < 256) hist[tid] = 0;
            __syncthreads();
            for (int i = tid; i < V; i += SAMPLE_THREADS) {
                const uint32_t key = order_key(x[i]);
                if ((key & mask) == prefix) atomicAdd(&hist[(key >> shift) & 255u], 1);
            }
            __syncthreads();
            if (tid == 0) {
                int b = 255, r = remaining;
                for (; b > 0; --b) {
                    if (hist[b] >= r) break;
                    r -= hist[b];
                }
                sh_int[1] = b;
                sh_int[2] = r;
            }
            __syncthreads();
            prefix |= ((uint32_t)sh_int[1]) << shift;
            mask |= 255u << shift;
            remaining = sh_int[2];
            __syncthreads();
        }
        keep_key = prefix;
    }

    // ---- mass of the kept tokens after top-k
    float z = 0.f;
    for (int i = tid; i < V; i += SAMPLE_THREADS)
        if (order_key(x[i]) >= keep_key) z += expf((x[i] - gmax) * inv_t);
    z = block_sum(z, scratch);

    // ---- top-p: smallest key t such that the kept mass above t is <= p * z
    const float p = top_p[row];
    if (p < 1.0f) {
        const float limit = p * z;
        uint32_t lo = keep_key, hi = order_key(gmax);      // f(hi) holds: nothing lies above the maximum
        while (lo < hi) {
            const uint32_t mid = lo + ((hi - lo) >> 1);
            float above = 0.f;
            for (int i = tid; i < V; i += SAMPLE_THREADS) {
                const uint32_t key = order_key(x[i]);
                if (key > mid && key >= keep_key) above += expf((x[i] - gmax) * inv_t);
            }
            above = block_sum(above, scratch);
            if (above <= limit) hi = mid; else lo = mid + 1;
        }
        keep_key = lo;
        z = 0.f;
        for (int i = tid; i < V; i += SAMPLE_THREADS)
            if (order_key(x[i]) >= keep_key) z += expf((x[i] - gmax) * inv_t);
        z = block_sum(z, scratch);
    }

    // ---- inverse CDF in vocabulary order: contiguous chunk per thread
    const int chunk = (V + SAMPLE_THREADS - 1) / SAMPLE_THREADS;
    const int i0 = min(V, tid * chunk), i1 = min(V, i0 + chunk);
    float mine = 0.f;
    for (int i = i0; i < i1; ++i)
        if (order_key(x[i]) >= keep_key) mine += expf((x[i] - gmax) * inv_t);
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
    hipLaunchKernelGGL(sample_kernel, dim3(M), dim3(SAMPLE_THREADS), 0, (hipStream_t)stream, logits,
                       V, temperature, top_k, top_p, u, out);
    return ra_launch_status();
}
