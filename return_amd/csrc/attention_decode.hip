// Decode attention for bfloat16: one query token per request over its paged keys and values,
// split along the keys so that a single request still fills the chip.
//
// What it restates of the reference: rollout/attention.py:430-514 (_decode_split_kernel: one
// program per (request, kv head, split) handles the whole GQA group, block of 16 query rows,
// writes un-normalised partial sums with their running maximum m and sum l) and
// rollout/attention.py:517-540 (_decode_combine: log-sum-exp merge of the splits).
// Different here: keys are already rotated in the cache; splits are fixed runs of
// `split_tokens` positions (not a share of the pages that depends on batch size as in
// rollout/attention.py:543-546), so a request's result does not depend on the batch.
//
// One wave per (request, kv head, split). Scores S^T = K Q^T come from MFMA 16x16x16 bf16
// with the key tile as the A operand, read straight from the cache: lane (m, g) holds
// key m's elements d = g*D/4 + 4j .. +3 for MFMA j, and the query operand is laid out the
// same way, so each lane reads one contiguous quarter of its key row. The result leaves
// lane (n, g) with the scores of query head n for keys 4g..4g+3 of each 16-key tile.
// P.V runs on the vector unit: a lane owns a few columns d and walks the 64 keys.
#include "common.h"

typedef short short4_t __attribute__((ext_vector_type(4)));
typedef float float4_t __attribute__((ext_vector_type(4)));

#define DEC_CHUNK 64          // keys per pass of a wave
#define DEC_MAX_GROUP 16      // query heads per kv head (rows of the MFMA tile)

struct DecodeRange {
    int lo, hi;               // key positions of this split, inclusive; lo > hi: empty
    int n_splits;             // splits that hold keys for this request
};

__device__ __forceinline__ DecodeRange decode_range(int pos_q, int start, int window,
                                                    int split_tokens, int sp) {
    int first = start;
    if (window > 0 && pos_q - window + 1 > first) first = pos_q - window + 1;
    const int split0 = first / split_tokens;
    const int s_abs = split0 + sp;
    DecodeRange r;
    r.lo = max(first, s_abs * split_tokens);
    r.hi = min(pos_q, (s_abs + 1) * split_tokens - 1);
    r.n_splits = pos_q / split_tokens - split0 + 1;
    return r;
}

template <int D16>
__global__ __launch_bounds__(64) void attn_decode_kernel(
    const bf16* __restrict__ q, float* __restrict__ part_acc, float* __restrict__ part_ml,
    const bf16* __restrict__ k_pool, const bf16* __restrict__ v_pool,
    const int* __restrict__ page_table, const int* __restrict__ cu_pages,
    const int* __restrict__ kv_start, const int* __restrict__ cu_q,
    const int* __restrict__ q_start, const int* __restrict__ seg_ids, int Hq, int Hkv, int P,
    float scale, int window, int split_tokens, int max_splits) {
    constexpr int D = 16 * D16;
    constexpr int VEC = (D % 128 == 0) ? 2 : 1;                 // columns per lane per V load
    constexpr int NE = (D + 64 * VEC - 1) / (64 * VEC);        // V loads per key per lane
    constexpr bool PRELOAD_V = (D <= 128);

    __shared__ float p_s[DEC_CHUNK * DEC_MAX_GROUP];           // [key][query head]
    __shared__ float alpha_s[DEC_MAX_GROUP];

    const int di = blockIdx.x, kvh = blockIdx.y, sp = blockIdx.z;
    const int seg = seg_ids ? seg_ids[di] : di;
    const int lane = threadIdx.x, n = lane & 15, g = lane >> 4;
    const int G = Hq / Hkv;
    const int t = cu_q[seg];
    const int pos_q = q_start[seg];
    const int start = kv_start[seg];
    const DecodeRange rg = decode_range(pos_q, start, window, split_tokens, sp);
    if (rg.lo > rg.hi) return;
    const int* pt = page_table + cu_pages[seg];

    // query operand: lane (n, g) holds head kvh*G+n, elements g*D/4 + 4j..+3
    short4_t bq[D16];
    {
        const bf16* qp = q + ((size_t)t * Hq + (size_t)kvh * G + (n < G ? n : 0)) * D + g * (D / 4);
#pragma unroll
        for (int j = 0; j < D16; ++j) {
            short4_t v = *reinterpret_cast<const short4_t*>(qp + 4 * j);
            if (n >= G) v = short4_t{0, 0, 0, 0};
            bq[j] = v;
        }
    }

    float m_run = -INFINITY, l_run = 0.f;
    float acc[DEC_MAX_GROUP][NE * VEC];
#pragma unroll
    for (int h = 0; h < DEC_MAX_GROUP; ++h)
#pragma unroll
        for (int e = 0; e < NE * VEC; ++e) acc[h][e] = 0.f;

    const int c_begin = (rg.lo / DEC_CHUNK) * DEC_CHUNK;
    for (int c0 = c_begin; c0 <= rg.hi; c0 += DEC_CHUNK) {
        // row of this lane's key (clamped into the split so that every address is valid)
        int kpos = c0 + lane;
        kpos = min(max(kpos, rg.lo), rg.hi);
        const int idx = kpos - start;
        const int row = pt[idx / P] * P + idx % P;

        // ---- K tiles straight into MFMA A operands
        short4_t ak[4][D16];
#pragma unroll
        for (int st = 0; st < 4; ++st) {
            const int r = __shfl(row, st * 16 + n, 64);
            const bf16* kp = k_pool + ((size_t)r * Hkv + kvh) * D + g * (D / 4);
#pragma unroll
            for (int j = 0; j < D16; ++j) ak[st][j] = *reinterpret_cast<const short4_t*>(kp + 4 * j);
        }
        // ---- V rows for the vector stage
        uint32_t vreg[PRELOAD_V ? DEC_CHUNK : 1][NE];
        if constexpr (PRELOAD_V) {
#pragma unroll
            for (int k = 0; k < DEC_CHUNK; ++k) {
                const int r = __builtin_amdgcn_readlane(row, k);
                const bf16* vp = v_pool + ((size_t)r * Hkv + kvh) * D;
#pragma unroll
                for (int e = 0; e < NE; ++e) {
                    const int d = e * 64 * VEC + lane * VEC;
                    if (VEC == 2) vreg[k][e] = *reinterpret_cast<const uint32_t*>(vp + d);
                    else vreg[k][e] = (d < D) ? (uint32_t)vp[d].x : 0u;
                }
            }
        }

        // ---- scores
        float s[4][4];
        float mx = -INFINITY;
#pragma unroll
        for (int st = 0; st < 4; ++st) {
            float4_t c = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int j = 0; j < D16; ++j)
                c = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(ak[st][j], bq[j], c, 0, 0, 0);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int kp_abs = c0 + st * 16 + 4 * g + i;
                const bool ok = kp_abs >= rg.lo && kp_abs <= rg.hi;
                s[st][i] = ok ? c[i] * scale : -INFINITY;
                mx = fmaxf(mx, s[st][i]);
            }
        }
        mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        const float m_new = fmaxf(m_run, mx);            // finite: the chunk holds a valid key
        float lsum = 0.f;
#pragma unroll
        for (int st = 0; st < 4; ++st)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float p = (s[st][i] == -INFINITY) ? 0.f : __expf(s[st][i] - m_new);
                lsum += p;
                p_s[(st * 16 + 4 * g + i) * DEC_MAX_GROUP + n] = p;
            }
        lsum += __shfl_xor(lsum, 16, 64);
        lsum += __shfl_xor(lsum, 32, 64);
        const float alpha = (m_run == -INFINITY) ? 0.f : __expf(m_run - m_new);
        if (g == 0) alpha_s[n] = alpha;
        l_run = l_run * alpha + lsum;
        m_run = m_new;
        __syncthreads();

        // ---- P.V on the vector unit
#pragma unroll
        for (int h = 0; h < DEC_MAX_GROUP; ++h) {
            if (h >= G) break;
            const float a = alpha_s[h];
#pragma unroll
            for (int e = 0; e < NE * VEC; ++e) acc[h][e] *= a;
        }
#pragma unroll
        for (int k = 0; k < DEC_CHUNK; ++k) {
            float vf[NE * VEC];
            if constexpr (PRELOAD_V) {
#pragma unroll
                for (int e = 0; e < NE; ++e) {
                    if (VEC == 2) {
                        vf[2 * e] = __uint_as_float(vreg[k][e] << 16);
                        vf[2 * e + 1] = __uint_as_float(vreg[k][e] & 0xffff0000u);
                    } else {
                        vf[e] = __uint_as_float(vreg[k][e] << 16);
                    }
                }
            } else {
                const int r = __builtin_amdgcn_readlane(row, k);
                const bf16* vp = v_pool + ((size_t)r * Hkv + kvh) * D;
#pragma unroll
                for (int e = 0; e < NE; ++e) {
                    const int d = e * 64 * VEC + lane * VEC;
                    if (VEC == 2) {
                        const uint32_t u = *reinterpret_cast<const uint32_t*>(vp + d);
                        vf[2 * e] = __uint_as_float(u << 16);
                        vf[2 * e + 1] = __uint_as_float(u & 0xffff0000u);
                    } else {
                        vf[e] = (d < D) ? to_f(vp[d]) : 0.f;
                    }
                }
            }
#pragma unroll
            for (int h = 0; h < DEC_MAX_GROUP; ++h) {
                if (h >= G) break;
                const float p = p_s[k * DEC_MAX_GROUP + h];
#pragma unroll
                for (int e = 0; e < NE * VEC; ++e) acc[h][e] = fmaf(p, vf[e], acc[h][e]);
            }
        }
        __syncthreads();
    }

    // ---- partial results of this split
#pragma unroll
    for (int h = 0; h < DEC_MAX_GROUP; ++h) {
        if (h >= G) break;
        float* pa = part_acc + (((size_t)di * Hq + (size_t)kvh * G + h) * max_splits + sp) * D;
#pragma unroll
        for (int e = 0; e < NE; ++e) {
            const int d = e * 64 * VEC + lane * VEC;
            if (VEC == 2) {
                pa[d] = acc[h][2 * e];
                pa[d + 1] = acc[h][2 * e + 1];
            } else if (d < D) {
                pa[d] = acc[h][e];
            }
        }
    }
    if (g == 0 && n < G) {
        float* pm = part_ml + (((size_t)di * Hq + (size_t)kvh * G + n) * max_splits + sp) * 2;
        pm[0] = m_run;
        pm[1] = l_run;
    }
}

// Merge of the splits, in split order: out = sum_s acc_s * exp(m_s - m) / sum_s l_s * exp(m_s - m).
__global__ __launch_bounds__(64) void attn_decode_combine_kernel(
    const float* __restrict__ part_acc, const float* __restrict__ part_ml, bf16* __restrict__ out,
    const int* __restrict__ kv_start, const int* __restrict__ cu_q, const int* __restrict__ q_start,
    const int* __restrict__ seg_ids, int Hq, int D, int window, int split_tokens, int max_splits) {
    const int di = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
    const int seg = seg_ids ? seg_ids[di] : di;
    const int t = cu_q[seg];
    const DecodeRange rg = decode_range(q_start[seg], kv_start[seg], window, split_tokens, 0);
    const int ns = min(rg.n_splits, max_splits);
    const float* pm = part_ml + ((size_t)di * Hq + head) * max_splits * 2;
    const float* pa = part_acc + ((size_t)di * Hq + head) * max_splits * D;
    float m = -INFINITY;
    for (int s = 0; s < ns; ++s) m = fmaxf(m, pm[2 * s]);
    float l = 0.f;
    for (int s = 0; s < ns; ++s) l += pm[2 * s + 1] * __expf(pm[2 * s] - m);
    const float inv = l > 0.f ? 1.0f / l : 0.f;
    for (int d = lane; d < D; d += 64) {
        float o = 0.f;
        for (int s = 0; s < ns; ++s) o += pa[(size_t)s * D + d] * __expf(pm[2 * s] - m);
        out[((size_t)t * Hq + head) * D + d] = from_f<bf16>(o * inv);
    }
}

template <int D16>
static void launch_decode(dim3 grid, hipStream_t st, const bf16* q, float* pa, float* pm,
                          const bf16* kp, const bf16* vp, const int* pt, const int* cup,
                          const int* kvs, const int* cuq, const int* qs, const int* segs, int Hq,
                          int Hkv, int P, float scale, int window, int split_tokens, int max_splits) {
    hipLaunchKernelGGL(attn_decode_kernel<D16>, grid, dim3(64), 0, st, q, pa, pm, kp, vp, pt, cup,
                       kvs, cuq, qs, segs, Hq, Hkv, P, scale, window, split_tokens, max_splits);
}

// part_acc: fp32 [n_dec, Hq, max_splits, D]; part_ml: fp32 [n_dec, Hq, max_splits, 2].
// max_splits must cover ceil((longest sequence)/split_tokens) + 1 splits... the host passes
// the number of splits of the longest request; requests with fewer leave the rest untouched.
extern "C" int ra_attention_decode_bf16(const void* q, void* out, void* part_acc, void* part_ml,
                                        const void* k_pool, const void* v_pool,
                                        const int* page_table, const int* cu_pages,
                                        const int* kv_start, const int* cu_q, const int* q_start,
                                        const int* seg_ids, int n_dec, int Hq, int Hkv, int D, int P,
                                        float scale, int window, int split_tokens, int max_splits,
                                        void* stream) {
    if (n_dec <= 0) return RA_OK;
    if (D % 16 != 0 || D < 16 || D > 256 || Hkv <= 0 || Hq % Hkv != 0 || Hq / Hkv > DEC_MAX_GROUP ||
        split_tokens <= 0 || split_tokens % DEC_CHUNK != 0 || max_splits <= 0 || max_splits > 65535 ||
        Hkv > 65535 || P <= 0)
        return RA_ERR_ARG;
    hipStream_t st = (hipStream_t)stream;
    dim3 grid(n_dec, Hkv, max_splits);
    const bf16* qq = (const bf16*)q;
    const bf16* kp = (const bf16*)k_pool;
    const bf16* vp = (const bf16*)v_pool;
    float* pa = (float*)part_acc;
    float* pm = (float*)part_ml;
#define DEC_CASE(N)                                                                              \
    case N:                                                                                      \
        launch_decode<N>(grid, st, qq, pa, pm, kp, vp, page_table, cu_pages, kv_start, cu_q,     \
                         q_start, seg_ids, Hq, Hkv, P, scale, window, split_tokens, max_splits); \
        break;
    switch (D / 16) {
        DEC_CASE(1) DEC_CASE(2) DEC_CASE(3) DEC_CASE(4) DEC_CASE(5) DEC_CASE(6) DEC_CASE(7) DEC_CASE(8)
        DEC_CASE(9) DEC_CASE(10) DEC_CASE(11) DEC_CASE(12) DEC_CASE(13) DEC_CASE(14) DEC_CASE(15)
        DEC_CASE(16)
        default: return RA_ERR_ARG;
    }
#undef DEC_CASE
    if (hipGetLastError() != hipSuccess) return RA_ERR_LAUNCH;
    hipLaunchKernelGGL(attn_decode_combine_kernel, dim3(n_dec, Hq), dim3(64), 0, st, pa, pm,
                       (bf16*)out, kv_start, cu_q, q_start, seg_ids, Hq, D, window, split_tokens,
                       max_splits);
    return ra_launch_status();
}
