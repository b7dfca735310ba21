// Attention of new queries over the paged cache, the plain kernel: one wave per
// (query token, query head), any head size up to 512, any page size, optional window.
// It is the kernel of the float32 path (every product and sum a 32-bit FMA) and the
// fallback of the bfloat16 path for head sizes the MFMA kernels do not take.
//
// Formulas: scores q.k * scale over keys at positions <= the query's, online softmax with
// running maximum, sum(p*v) / sum(p): rollout/attention.py:126-139; query head h reads kv
// head h / (Hq/Hkv): rollout/attention.py:65. Keys are already rotated in the cache.
// Tables: page_table[cu_pages[s] + i] is the i-th listed page of request s, whose first row
// holds position kv_start[s]; new tokens of s are rows cu_q[s]..cu_q[s+1]-1 of q and sit at
// positions q_start[s], q_start[s]+1, ... (rollout/cache.py:282-328 has the same tables
// with per-page valid counts instead of kv_start). tok_ids, if given, lists the T_tokens rows
// of q to work on (the others belong to another kernel).
#include "common.h"

#define PLAIN_MAX_ACC 8     // D <= 64 * 8

template <typename T>
__global__ __launch_bounds__(64) void attn_plain_kernel(
    const T* __restrict__ q, T* __restrict__ out, const T* __restrict__ k_pool,
    const T* __restrict__ v_pool, const int* __restrict__ page_table,
    const int* __restrict__ cu_pages, const int* __restrict__ kv_start,
    const int* __restrict__ cu_q, const int* __restrict__ q_start,
    const int* __restrict__ tok_ids, int n_seqs, int Hq, int Hkv, int D, int P, float scale,
    int window) {
    extern __shared__ float smem[];
    float* q_s = smem;                       // [D]
    float* p_s = smem + D;                   // [64]
    int* row_s = (int*)(smem + D + 64);      // [64]

    const int t = tok_ids ? tok_ids[blockIdx.x] : (int)blockIdx.x;
    const int head = blockIdx.y, lane = threadIdx.x;
    int lo = 0, hi = n_seqs - 1;
    while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (cu_q[mid] <= t) lo = mid; else hi = mid - 1;
    }
    const int s = lo;
    const int pos_q = q_start[s] + (t - cu_q[s]);
    const int kvh = head / (Hq / Hkv);
    const int start = kv_start[s];
    int first = start;
    if (window > 0 && pos_q - window + 1 > first) first = pos_q - window + 1;
    const int* pt = page_table + cu_pages[s];
    const int n_listed = cu_pages[s + 1] - cu_pages[s];

    const T* qr = q + ((size_t)t * Hq + head) * D;
    for (int c = lane; c < D; c += 64) q_s[c] = to_f(qr[c]);
    __syncthreads();

    float m = -INFINITY, l = 0.f;
    float acc[PLAIN_MAX_ACC];
#pragma unroll
    for (int i = 0; i < PLAIN_MAX_ACC; ++i) acc[i] = 0.f;

    for (int base = first; base <= pos_q; base += 64) {
        const int p = base + lane;
        bool valid = p <= pos_q;
        float score = -INFINITY;
        int row = -1;
        if (valid) {
            const int idx = p - start;
            const int pi = idx / P;
            if (pi < n_listed) {
                row = pt[pi] * P + idx % P;
                const T* kr = k_pool + ((size_t)row * Hkv + kvh) * D;
                float dot = 0.f;
                for (int c = 0; c < D; ++c) dot = fmaf(q_s[c], to_f(kr[c]), dot);
                score = dot * scale;
            } else {
                valid = false;               // table shorter than the positions claim: ignore the key
            }
        }
        const float m_new = fmaxf(m, wave_max(score));
        const float pr = valid ? expf(score - m_new) : 0.f;
        const float alpha = (m == -INFINITY) ? 0.f : expf(m - m_new);
        l = l * alpha + wave_sum(pr);
        p_s[lane] = pr;
        row_s[lane] = row;
        __syncthreads();
#pragma unroll
        for (int i = 0; i < PLAIN_MAX_ACC; ++i) acc[i] *= alpha;
        const int nk = min(64, pos_q - base + 1);
        for (int kk = 0; kk < nk; ++kk) {
            const int r = row_s[kk];
            if (r < 0) continue;
            const float pv = p_s[kk];
            const T* vr = v_pool + ((size_t)r * Hkv + kvh) * D;
#pragma unroll
            for (int i = 0; i < PLAIN_MAX_ACC; ++i) {
                const int c = lane + 64 * i;
                if (c < D) acc[i] = fmaf(pv, to_f(vr[c]), acc[i]);
            }
        }
        __syncthreads();
        m = m_new;
    }
    T* o = out + ((size_t)t * Hq + head) * D;
    const float inv = l > 0.f ? 1.0f / l : 0.f;
#pragma unroll
    for (int i = 0; i < PLAIN_MAX_ACC; ++i) {
        const int c = lane + 64 * i;
        if (c < D) o[c] = from_f<T>(acc[i] * inv);
    }
}

extern "C" int ra_attention_plain(const void* q, void* out, const void* k_pool, const void* v_pool,
                                  const int* page_table, const int* cu_pages, const int* kv_start,
                                  const int* cu_q, const int* q_start, const int* tok_ids,
                                  int n_seqs, int T_tokens, int Hq, int Hkv, int D, int P, float scale, int window, int dtype,
                                  void* stream) {
    if (T_tokens <= 0 || n_seqs <= 0) return RA_OK;
    if (D > 64 * PLAIN_MAX_ACC || D <= 0 || Hkv <= 0 || Hq % Hkv != 0 || P <= 0) return RA_ERR_ARG;
    dim3 grid(T_tokens, Hq), block(64);
    const size_t shmem = (size_t)(D + 128) * sizeof(float);
    hipStream_t st = (hipStream_t)stream;
    if (dtype == RA_DTYPE_F32)
        hipLaunchKernelGGL(attn_plain_kernel<float>, grid, block, shmem, st, (const float*)q,
                           (float*)out, (const float*)k_pool, (const float*)v_pool, page_table,
                           cu_pages, kv_start, cu_q, q_start, tok_ids, n_seqs, Hq, Hkv, D, P, scale,
                           window);
    else
        hipLaunchKernelGGL(attn_plain_kernel<bf16>, grid, block, shmem, st, (const bf16*)q,
                           (bf16*)out, (const bf16*)k_pool, (const bf16*)v_pool, page_table,
                           cu_pages, kv_start, cu_q, q_start, tok_ids, n_seqs, Hq, Hkv, D, P, scale,
                           window);
    return ra_launch_status();
}
