// Attention of new queries over the paged cache, the plain kernel: every product and sum a
// 32-bit FMA, any head size up to 512, any page size, any number of heads, optional window.
// It is the kernel of the float32 path and the fallback of the bfloat16 path for head sizes
// the MFMA kernels do not take.
//
// Formulas: scores q.k * scale over keys at positions <= the query's, online softmax with
// running maximum, sum(p*v) / sum(p): rollout/attention.py:126-139; query head h reads kv
// head h / (Hq/Hkv): rollout/attention.py:65. Keys are already rotated in the cache.
// Tables: page_table[cu_pages[s] + i] is the i-th listed page of request s, whose first row
// holds position kv_start[s]; new tokens of s are rows cu_q[s]..cu_q[s+1]-1 of q and sit at
// positions q_start[s], q_start[s]+1, ... (rollout/cache.py:282-328 has the same tables
// with per-page valid counts instead of kv_start). tok_ids, if given, lists the T_tokens rows
// of q to work on (the others belong to another kernel).
//
// A workgroup takes QR consecutive query rows of one head; rows of the same request are worked
// on together (one pass over the keys for all of them), rows of other requests in further
// passes. Its waves take the chunks of 64 key positions in turn (chunk c, counted from
// position 0, is wave c % WAVES's), so a row's sums are formed in an order that depends on
// nothing but its own positions; at the end the waves' running maxima, sums and rows are merged
// through LDS in wave order. Within a chunk four lanes share a key (each a quarter of the
// head's elements, 16 bytes at a time), 16 keys at once; for the values the lanes run along the
// head's elements, one key after the other.
#include "common.h"

#define PLAIN_MAX_ACC 8     // D <= 64 * 8
#define PLAIN_CHUNK 64

// four consecutive elements as floats; p is aligned to four elements
__device__ __forceinline__ void plain_load4(const float* p, float (&v)[4]) {
    const float4 t = *reinterpret_cast<const float4*>(p);
    v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
}
__device__ __forceinline__ void plain_load4(const bf16* p, float (&v)[4]) {
    const uint2 t = *reinterpret_cast<const uint2*>(p);
    v[0] = __uint_as_float(t.x << 16); v[1] = __uint_as_float(t.x & 0xffff0000u);
    v[2] = __uint_as_float(t.y << 16); v[3] = __uint_as_float(t.y & 0xffff0000u);
}

template <typename T, int QR, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void attn_plain_kernel(
    const T* __restrict__ q, T* __restrict__ out, const T* __restrict__ k_pool,
    const T* __restrict__ v_pool, const int* __restrict__ page_table,
    const int* __restrict__ cu_pages, const int* __restrict__ kv_start,
    const int* __restrict__ cu_q, const int* __restrict__ q_start,
    const int* __restrict__ tok_ids, int n_seqs, int T_tokens, int Hq, int Hkv, int D, int P, float scale,
    int window) {
    extern __shared__ __attribute__((aligned(16))) float smem[];
    float* q_s = smem;                                   // [QR][D]
    float* p_s = q_s + QR * D;                           // [WAVES][QR][64]
    int* row_s = (int*)(p_s + WAVES * QR * 64);          // [WAVES][64]
    float* ml_s = (float*)(row_s + WAVES * 64);          // [WAVES][QR][2]
    float* acc_s = ml_s + WAVES * QR * 2;                // [WAVES][QR][D]

    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, part = lane & 3, sub = lane >> 2;
    const int head = blockIdx.y, kvh = head / (Hq / Hkv);
    const bool vec = (D & 3) == 0;

    // the rows of this workgroup: token row, request, position; bit r of todo: row r is still to do
    int t_of[QR], seg_of[QR], pos_of[QR];
    unsigned todo = 0;
#pragma unroll
    for (int r = 0; r < QR; ++r) {
        const int qi = blockIdx.x * QR + r;
        t_of[r] = seg_of[r] = pos_of[r] = 0;
        if (qi < T_tokens) {
            const int t = tok_ids ? tok_ids[qi] : qi;
            int lo = 0, hi = n_seqs - 1;
            while (lo < hi) {
                const int mid = (lo + hi + 1) >> 1;
                if (cu_q[mid] <= t) lo = mid; else hi = mid - 1;
            }
            todo |= 1u << r;
            t_of[r] = t;
            seg_of[r] = lo;
            pos_of[r] = q_start[lo] + (t - cu_q[lo]);
        }
    }

    while (todo) {                                       // one pass per request among the rows; the same in every thread
        int s = 0;
#pragma unroll
        for (int r = QR - 1; r >= 0; --r)
            if ((todo >> r) & 1u) s = seg_of[r];         // the request of the first row still to do
        bool active[QR];
        int first_of[QR];
        const int start = kv_start[s];
        int lo_pos = 0x7fffffff, hi_pos = -1;
#pragma unroll
        for (int r = 0; r < QR; ++r) {
            active[r] = ((todo >> r) & 1u) && seg_of[r] == s;
            if (active[r]) todo &= ~(1u << r);
            first_of[r] = start;
            if (window > 0 && pos_of[r] - window + 1 > start) first_of[r] = pos_of[r] - window + 1;
            if (active[r]) {
                lo_pos = min(lo_pos, first_of[r]);
                hi_pos = max(hi_pos, pos_of[r]);
            }
        }
        const int* pt = page_table + cu_pages[s];
        const int n_listed = cu_pages[s + 1] - cu_pages[s];

#pragma unroll
        for (int r = 0; r < QR; ++r) {
            const T* qr = q + ((size_t)t_of[r] * Hq + head) * D;
            for (int c = tid; c < D; c += WAVES * 64) q_s[r * D + c] = active[r] ? to_f(qr[c]) : 0.f;
        }
        __syncthreads();

        float m[QR], l[QR], acc[QR][PLAIN_MAX_ACC];
#pragma unroll
        for (int r = 0; r < QR; ++r) {
            m[r] = -INFINITY;
            l[r] = 0.f;
#pragma unroll
            for (int i = 0; i < PLAIN_MAX_ACC; ++i) acc[r][i] = 0.f;
        }
        float* my_p = p_s + wave * QR * 64;
        int* my_row = row_s + wave * 64;

        const int c_first = lo_pos / PLAIN_CHUNK;
        int c = c_first + ((wave - c_first) % WAVES + WAVES) % WAVES;      // first chunk >= c_first of this wave
        for (; c * PLAIN_CHUNK <= hi_pos; c += WAVES) {
            const int base = c * PLAIN_CHUNK;
            // ---- scores: 16 keys at once, four lanes to a key
            float sc[4][QR];
#pragma unroll
            for (int sp = 0; sp < 4; ++sp) {
                const int kk = 16 * sp + sub;
                const int p = base + kk;
                const int idx = p - start;
                const int pi = idx >= 0 ? idx / P : 0;
                const bool there = p >= lo_pos && p <= hi_pos && pi < n_listed;   // else: not a key of this pass
                const int row = there ? (pt[pi] * Hkv + kvh) * P + (idx - pi * P) : -1;   // [page][kv head][row in page]
                float dot[QR];
#pragma unroll
                for (int r = 0; r < QR; ++r) dot[r] = 0.f;
                if (there) {
                    const T* kr = k_pool + (size_t)row * D;
                    if (vec) {
                        for (int j = part; 4 * j < D; j += 4) {
                            float kv[4];
                            plain_load4(kr + 4 * j, kv);
#pragma unroll
                            for (int r = 0; r < QR; ++r) {
                                const float4 qv = *reinterpret_cast<const float4*>(q_s + r * D + 4 * j);
                                dot[r] = fmaf(qv.x, kv[0], dot[r]);
                                dot[r] = fmaf(qv.y, kv[1], dot[r]);
                                dot[r] = fmaf(qv.z, kv[2], dot[r]);
                                dot[r] = fmaf(qv.w, kv[3], dot[r]);
                            }
                        }
                    } else {
                        for (int e = part; e < D; e += 4) {
                            const float kv = to_f(kr[e]);
#pragma unroll
                            for (int r = 0; r < QR; ++r) dot[r] = fmaf(q_s[r * D + e], kv, dot[r]);
                        }
                    }
                }
#pragma unroll
                for (int r = 0; r < QR; ++r) {
                    float d = dot[r];
                    d += __shfl_xor(d, 1, 64);
                    d += __shfl_xor(d, 2, 64);
                    const bool ok = there && active[r] && p <= pos_of[r] && p >= first_of[r];
                    sc[sp][r] = ok ? d * scale : -INFINITY;
                }
                if (part == 0) my_row[kk] = row;
            }
            // ---- running maximum and sum of every row; the chunk's probabilities into LDS
#pragma unroll
            for (int r = 0; r < QR; ++r) {
                const float mx = wave_max(fmaxf(fmaxf(sc[0][r], sc[1][r]), fmaxf(sc[2][r], sc[3][r])));
                const float m_new = fmaxf(m[r], mx);
                const float alpha = (m[r] == -INFINITY) ? 0.f : expf(m[r] - m_new);
                float mine = 0.f;
#pragma unroll
                for (int sp = 0; sp < 4; ++sp) {
                    const float pr = (sc[sp][r] == -INFINITY) ? 0.f : expf(sc[sp][r] - m_new);
                    if (part == 0) {
                        my_p[r * 64 + 16 * sp + sub] = pr;
                        mine += pr;
                    }
                }
                l[r] = l[r] * alpha + wave_sum(mine);
                m[r] = m_new;
#pragma unroll
                for (int i = 0; i < PLAIN_MAX_ACC; ++i) acc[r][i] *= alpha;
            }
            __builtin_amdgcn_wave_barrier();             // LDS serves a wave's accesses in order
            // ---- values: the lanes run along the head's elements
            const int nk = min(PLAIN_CHUNK, hi_pos - base + 1);
#pragma unroll 4
            for (int kk = 0; kk < nk; ++kk) {
                const int row = max(my_row[kk], 0);      // a key that is not there has probability 0
                const T* vr = v_pool + (size_t)row * D;
                float pv[QR];
#pragma unroll
                for (int r = 0; r < QR; ++r) pv[r] = my_p[r * 64 + kk];
#pragma unroll
                for (int i = 0; i < PLAIN_MAX_ACC; ++i) {
                    const int e = lane + 64 * i;
                    if (e < D) {
                        const float v = to_f(vr[e]);
#pragma unroll
                        for (int r = 0; r < QR; ++r) acc[r][i] = fmaf(pv[r], v, acc[r][i]);
                    }
                }
            }
            __builtin_amdgcn_wave_barrier();
        }

        // ---- merge of the waves, in wave order
#pragma unroll
        for (int r = 0; r < QR; ++r) {
            if (lane == 0) {
                ml_s[(wave * QR + r) * 2] = m[r];
                ml_s[(wave * QR + r) * 2 + 1] = l[r];
            }
#pragma unroll
            for (int i = 0; i < PLAIN_MAX_ACC; ++i) {
                const int e = lane + 64 * i;
                if (e < D) acc_s[(wave * QR + r) * D + e] = acc[r][i];
            }
        }
        __syncthreads();
        for (int idx = tid; idx < QR * D; idx += WAVES * 64) {
            const int r = idx / D, e = idx - r * D;
            bool act = false;
            int t_row = 0;
#pragma unroll
            for (int rr = 0; rr < QR; ++rr)
                if (rr == r) { act = active[rr]; t_row = t_of[rr]; }
            if (!act) continue;
            float mm = -INFINITY;
            for (int w = 0; w < WAVES; ++w) mm = fmaxf(mm, ml_s[(w * QR + r) * 2]);
            float num = 0.f, den = 0.f;
            for (int w = 0; w < WAVES; ++w) {
                const float mw = ml_s[(w * QR + r) * 2];
                const float ew = (mw == -INFINITY) ? 0.f : expf(mw - mm);
                num = fmaf(acc_s[(w * QR + r) * D + e], ew, num);
                den = fmaf(ml_s[(w * QR + r) * 2 + 1], ew, den);
            }
            out[((size_t)t_row * Hq + head) * D + e] = from_f<T>(den > 0.f ? num / den : 0.f);
        }
        __syncthreads();                                 // before the next pass writes q_s and the merge buffers
    }
}

template <typename T, int QR, int WAVES>
static void plain_launch(hipStream_t st, const void* q, void* out, const void* k_pool, const void* v_pool,
                         const int* page_table, const int* cu_pages, const int* kv_start, const int* cu_q,
                         const int* q_start, const int* tok_ids, int n_seqs, int T_tokens, int Hq, int Hkv,
                         int D, int P, float scale, int window) {
    const size_t floats = (size_t)QR * D + (size_t)WAVES * QR * 64 + WAVES * 64 + WAVES * QR * 2 +
                          (size_t)WAVES * QR * D;
    dim3 grid((T_tokens + QR - 1) / QR, Hq), block(WAVES * 64);
    hipLaunchKernelGGL((attn_plain_kernel<T, QR, WAVES>), grid, block, floats * sizeof(float), st, (const T*)q,
                       (T*)out, (const T*)k_pool, (const T*)v_pool, page_table, cu_pages, kv_start, cu_q,
                       q_start, tok_ids, n_seqs, T_tokens, Hq, Hkv, D, P, scale, window);
}

extern "C" int ra_attention_plain(const void* q, void* out, const void* k_pool, const void* v_pool,
                                  const int* page_table, const int* cu_pages, const int* kv_start,
                                  const int* cu_q, const int* q_start, const int* tok_ids,
                                  int n_seqs, int T_tokens, int Hq, int Hkv, int D, int P, float scale, int window, int dtype,
                                  void* stream) {
    if (T_tokens <= 0 || n_seqs <= 0) return RA_OK;
    if (D > 64 * PLAIN_MAX_ACC || D <= 0 || Hkv <= 0 || Hq % Hkv != 0 || P <= 0 || Hq > 65535) return RA_ERR_ARG;
    if (dtype != RA_DTYPE_F32 && dtype != RA_DTYPE_BF16) return RA_ERR_ARG;
    hipStream_t st = (hipStream_t)stream;
    // one row per request (decoding): a workgroup per row, eight waves over its keys; else four rows
    // a workgroup, which share the keys they read when they belong to one request
    const bool single = tok_ids == nullptr && T_tokens == n_seqs;
#define PLAIN_GO(T_, QR_, W_)                                                                              \
    plain_launch<T_, QR_, W_>(st, q, out, k_pool, v_pool, page_table, cu_pages, kv_start, cu_q, q_start,   \
                              tok_ids, n_seqs, T_tokens, Hq, Hkv, D, P, scale, window)
    if (dtype == RA_DTYPE_F32) {
        if (single) PLAIN_GO(float, 1, 8); else PLAIN_GO(float, 4, 4);
    } else {
        if (single) PLAIN_GO(bf16, 1, 8); else PLAIN_GO(bf16, 4, 4);
    }
#undef PLAIN_GO
    return ra_launch_status();
}
