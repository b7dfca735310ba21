// Decode attention for bfloat16: one query token per request over its paged keys and values,
// split along the keys so that a single request still fills the chip.
//
// What it restates of the reference: rollout/attention.py:430-514 (_decode_split_kernel: one
// program per (request, kv head, split) handles the whole GQA group as a block of 16 query
// rows and writes un-normalised partial sums with their running maximum m and sum l) and
// rollout/attention.py:517-540 (_decode_combine: log-sum-exp merge of the splits).
// Different here: keys are already rotated in the cache; splits are fixed runs of
// `split_tokens` positions counted from position 0 (the reference gives every split a share
// of the pages, rollout/attention.py:458-461).
//
// One wave per (request, kv head, split), 64 keys per pass.
//  scores  S^T = K Q^T by MFMA 16x16x32 bf16, the key tile as A operand read straight from
//          the cache: lane (n, g) loads the 16 bytes d = 32j + 8g .. +7 of key n, so the four
//          lane groups of a key read 64 contiguous bytes per load; the B operand holds the
//          group's query heads (up to 16) the same way. A trailing 16 of D is one more step of
//          the same MFMA with the upper half of k zero (an accumulation chain that mixed
//          16x16x32 and 16x16x16 lost the last 16x16x32 term on gfx950, so one shape is used
//          throughout). Lane (n, g) ends up with query head n, keys 4g..4g+3 of each tile.
//  P.V     O^T += V^T P^T by the same MFMA: the value rows go through LDS (16-byte pieces in,
//          transposing reads ds_read_b64_tr_b16 out: within 16 lanes, lane l receives element
//          l%4 of the 8 bytes addressed by lanes l/4, l/4+4, l/4+8, l/4+12), and P goes from
//          the softmax registers straight into the B operand because the contraction runs over
//          keys in the order the lanes already hold them (k-slot (g, e) of a 32-key block is
//          key 16*(e/4) + 4g + e%4). The cost does not depend on how many heads share a kv head,
//          up to 16; a larger group takes one wave per 16 heads, which read the same keys.
// BUILD-VARIANTS: DEC_PART=0 DEC_PART=1 DEC_PART=2 DEC_PART=3 DEC_API=1
// (each DEC_PART instantiates four head sizes; DEC_API holds the entry point and the merge)
#include "common.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef short short4_t __attribute__((ext_vector_type(4)));
typedef short short8_t __attribute__((ext_vector_type(8)));
typedef float float2_t __attribute__((ext_vector_type(2)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef uint32_t uint4_t __attribute__((ext_vector_type(4)));
typedef short4_t __attribute__((address_space(3))) * lds_short4_ptr;

#define DEC_CHUNK 64          // keys per pass of a wave
#define DEC_MAX_GROUP 16      // query heads a wave takes (columns of the MFMA tile); larger groups take several waves

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

#ifdef DEC_PART
// two floats to two bf16 in one word, round to nearest even (v_cvt_pk_bf16_f32)
__device__ __forceinline__ uint32_t pack2(float a, float b) {
    const float2_t v = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}

template <int D16>
__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(D16 <= 8 ? 2 : 1))) void attn_decode_kernel(
    const bf16* __restrict__ q, float* __restrict__ part_acc, float* __restrict__ part_ml,
    const bf16* __restrict__ k_pool, const bf16* __restrict__ v_pool,
    const int* __restrict__ page_table, const int* __restrict__ cu_pages,
    const int* __restrict__ kv_start, const int* __restrict__ cu_q,
    const int* __restrict__ q_start, const int* __restrict__ seg_ids, int Hq, int Hkv, int P,
    float scale, int window, int split_tokens, int max_splits) {
    constexpr int D = 16 * D16;
    constexpr int D32 = D / 32;                 // full MFMA x32 steps
    constexpr bool TAIL16 = (D % 32) != 0;      // one more step, upper k half zero
    constexpr int LPR = D / 8;                  // 16-byte pieces in one value row
    constexpr int NVL = (DEC_CHUNK * LPR + 63) / 64;   // pieces of the value tile per lane
    constexpr int VS = D + 16;                  // value tile row stride in LDS (elements): rows shift by 8 banks

    __shared__ __attribute__((aligned(16))) uint16_t v_s[DEC_CHUNK * VS];

    // blockIdx.y: kv head and, when more than 16 query heads share it, which 16 of them
    const int group = Hq / Hkv, blocks = (group + DEC_MAX_GROUP - 1) / DEC_MAX_GROUP;
    const int di = blockIdx.x, kvh = blockIdx.y / blocks, hb = blockIdx.y - kvh * blocks, sp = blockIdx.z;
    const int seg = seg_ids ? seg_ids[di] : di;
    const int lane = threadIdx.x, n = lane & 15, g = lane >> 4;
    const int h0 = kvh * group + hb * DEC_MAX_GROUP;             // first query head of this wave
    const int G = min(DEC_MAX_GROUP, group - hb * DEC_MAX_GROUP);  // and how many it has
    const int t = cu_q[seg];
    const int pos_q = q_start[seg];
    const int start = kv_start[seg];
    const DecodeRange rg = decode_range(pos_q, start, window, split_tokens, sp);
    if (rg.lo > rg.hi) return;
    const int* pt = page_table + cu_pages[seg];
    const int p_shift = (P & (P - 1)) == 0 ? __builtin_ctz(P) : -1;

    // query operand: lane (n, g) holds head h0+n, d = 32j + 8g .. +7 (and D-16+8g.. for the tail)
    const bf16x8_t z8 = {0, 0, 0, 0, 0, 0, 0, 0};
    bf16x8_t bq[D32 > 0 ? D32 : 1];
    bf16x8_t bq_tail = z8;
    {
        const bf16* qp = q + ((size_t)t * Hq + h0 + (n < G ? n : 0)) * D;
#pragma unroll
        for (int j = 0; j < D32; ++j) {
            bf16x8_t v = *reinterpret_cast<const bf16x8_t*>(qp + 32 * j + 8 * g);
            bq[j] = (n < G) ? v : z8;
        }
        if constexpr (TAIL16) {
            if (n < G && g < 2) bq_tail = *reinterpret_cast<const bf16x8_t*>(qp + (D - 16) + 8 * g);
        }
    }

    const float scale2 = scale * 1.44269504088896340736f;      // scores in the base-2 domain
    float m_run = -INFINITY, l_run = 0.f;
    float4_t acc[D16];                           // acc[dt][i] = O^T[d = 16dt + 4g + i][head n]
#pragma unroll
    for (int dt = 0; dt < D16; ++dt) acc[dt] = float4_t{0.f, 0.f, 0.f, 0.f};

    const int c_begin = (rg.lo / DEC_CHUNK) * DEC_CHUNK;
    for (int c0 = c_begin; c0 <= rg.hi; c0 += DEC_CHUNK) {
        // row of this lane's key (clamped into the split so that every address is valid)
        const int kpos = min(max(c0 + lane, rg.lo), rg.hi);
        const int idx = kpos - start;
        const int pi = p_shift >= 0 ? (idx >> p_shift) : (idx / P);
        const int row = pt[pi] * P + (idx - pi * P);

        // ---- K tiles straight into MFMA A operands
        bf16x8_t ak[4][D32 > 0 ? D32 : 1];
        bf16x8_t ak_tail[4];
#pragma unroll
        for (int st = 0; st < 4; ++st) {
            const int r = __shfl(row, st * 16 + n, 64);
            const bf16* kp = k_pool + ((size_t)r * Hkv + kvh) * D;
#pragma unroll
            for (int j = 0; j < D32; ++j)
                ak[st][j] = *reinterpret_cast<const bf16x8_t*>(kp + 32 * j + 8 * g);
            if constexpr (TAIL16) {
                ak_tail[st] = z8;
                if (g < 2) ak_tail[st] = *reinterpret_cast<const bf16x8_t*>(kp + (D - 16) + 8 * g);
            }
        }
        // ---- V rows: 16-byte pieces, all loads of the pass issued now, then into LDS
        uint4_t vv[NVL];
#pragma unroll
        for (int i = 0; i < NVL; ++i) {
            const int e = min(lane + 64 * i, DEC_CHUNK * LPR - 1);
            const int r = __shfl(row, e / LPR, 64);
            vv[i] = *reinterpret_cast<const uint4_t*>(v_pool + ((size_t)r * Hkv + kvh) * D + (e % LPR) * 8);
        }
        __syncthreads();                           // the previous pass has read its value tile
#pragma unroll
        for (int i = 0; i < NVL; ++i) {
            const int e = min(lane + 64 * i, DEC_CHUNK * LPR - 1);
            *reinterpret_cast<uint4_t*>(&v_s[(e / LPR) * VS + (e % LPR) * 8]) = vv[i];
        }

        // ---- scores
        float4_t cs[4];
#pragma unroll
        for (int st = 0; st < 4; ++st) {
            float4_t c = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int j = 0; j < D32; ++j)
                c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ak[st][j], bq[j], c, 0, 0, 0);
            if constexpr (TAIL16)
                c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ak_tail[st], bq_tail, c, 0, 0, 0);
            cs[st] = c;
        }
        MFMA_SETTLE();
        float s[4][4];
        float mx = -INFINITY;
#pragma unroll
        for (int st = 0; st < 4; ++st) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int kp_abs = c0 + st * 16 + 4 * g + i;
                const bool ok = kp_abs >= rg.lo && kp_abs <= rg.hi;
                s[st][i] = ok ? cs[st][i] * scale2 : -INFINITY;
                mx = fmaxf(mx, s[st][i]);
            }
        }
        mx = rows_max(mx);
        const float m_new = fmaxf(m_run, mx);            // finite: the pass holds a valid key
        float lsum = 0.f;
#pragma unroll
        for (int st = 0; st < 4; ++st)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                s[st][i] = __builtin_amdgcn_exp2f(s[st][i] - m_new);   // 2^(-inf) = 0 for masked keys
                lsum += s[st][i];
            }
        lsum = rows_sum(lsum);
        const float alpha = (m_run == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(m_run - m_new);
        l_run = l_run * alpha + lsum;
        if (__any(m_new != m_run)) {
#pragma unroll
            for (int dt = 0; dt < D16; ++dt) {
                acc[dt][0] *= alpha;
                acc[dt][1] *= alpha;
                acc[dt][2] *= alpha;
                acc[dt][3] *= alpha;
            }
        }
        m_run = m_new;
        __syncthreads();                           // the value tile is complete in LDS

        // ---- O^T += V^T P^T, 32 keys per MFMA
#pragma unroll
        for (int b = 0; b < 2; ++b) {
            const uint4_t pw = {pack2(s[2 * b][0], s[2 * b][1]), pack2(s[2 * b][2], s[2 * b][3]),
                                pack2(s[2 * b + 1][0], s[2 * b + 1][1]), pack2(s[2 * b + 1][2], s[2 * b + 1][3])};
            const bf16x8_t pb = __builtin_bit_cast(bf16x8_t, pw);
            // this lane's address as lane l' = n of its group: key 32b + 4g + n/4, columns 4(n%4)..+3
            const uint16_t* vr = &v_s[(32 * b + 4 * g + (n >> 2)) * VS + 4 * (n & 3)];
#pragma unroll
            for (int dt = 0; dt < D16; ++dt) {
                const short4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4_ptr)(vr + dt * 16));
                const short4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4_ptr)(vr + 16 * VS + dt * 16));
                const short8_t both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
                acc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, both), pb, acc[dt], 0, 0, 0);
            }
        }
    }
    MFMA_SETTLE();

    // ---- partial results of this split: lane (n, g) holds head n, columns 16dt + 4g .. +3
    if (n < G) {
        float* pa = part_acc + (((size_t)di * Hq + h0 + n) * max_splits + sp) * D;
#pragma unroll
        for (int dt = 0; dt < D16; ++dt) *reinterpret_cast<float4_t*>(pa + dt * 16 + 4 * g) = acc[dt];
        if (g == 0) {
            float* pm = part_ml + (((size_t)di * Hq + h0 + n) * max_splits + sp) * 2;
            pm[0] = m_run;
            pm[1] = l_run;
        }
    }
}

#define DEC_CAT2(a, b) a##b
#define DEC_CAT(a, b) DEC_CAT2(a, b)
// head sizes 16*(4*DEC_PART+1) .. 16*(4*DEC_PART+4)
extern "C" int DEC_CAT(ra_dec_part_, DEC_PART)(int D16, dim3 grid, hipStream_t st, const bf16* q, float* pa,
                                              float* pm, const bf16* kp, const bf16* vp, const int* pt,
                                              const int* cup, const int* kvs, const int* cuq,
                                              const int* qs, const int* segs, int Hq, int Hkv, int P,
                                              float scale, int window, int split_tokens,
                                              int max_splits) {
#define DEC_CASE(N)                                                                                \
    case N:                                                                                        \
        hipLaunchKernelGGL(attn_decode_kernel<N>, grid, dim3(64), 0, st, q, pa, pm, kp, vp, pt, cup, \
                           kvs, cuq, qs, segs, Hq, Hkv, P, scale, window, split_tokens, max_splits); \
        return RA_OK;
    switch (D16) {
        DEC_CASE(4 * DEC_PART + 1) DEC_CASE(4 * DEC_PART + 2) DEC_CASE(4 * DEC_PART + 3)
        DEC_CASE(4 * DEC_PART + 4)
        default: return RA_ERR_ARG;
    }
#undef DEC_CASE
}
#endif  // DEC_PART

#ifdef DEC_API

#define DEC_PART_ARGS int D16, dim3 grid, hipStream_t st, const bf16* q, float* pa, float* pm,        \
    const bf16* kp, const bf16* vp, const int* pt, const int* cup, const int* kvs, const int* cuq,   \
    const int* qs, const int* segs, int Hq, int Hkv, int P, float scale, int window,                 \
    int split_tokens, int max_splits
extern "C" int ra_dec_part_0(DEC_PART_ARGS);
extern "C" int ra_dec_part_1(DEC_PART_ARGS);
extern "C" int ra_dec_part_2(DEC_PART_ARGS);
extern "C" int ra_dec_part_3(DEC_PART_ARGS);

// Merge of the splits, in split order: out = sum_s acc_s * w_s / sum_s l_s * w_s, w_s = exp(m_s - m).
__global__ __launch_bounds__(128) void attn_decode_combine_kernel(
    const float* __restrict__ part_acc, const float* __restrict__ part_ml, bf16* __restrict__ out,
    const int* __restrict__ kv_start, const int* __restrict__ cu_q, const int* __restrict__ q_start,
    const int* __restrict__ seg_ids, int Hq, int D, int window, int split_tokens, int max_splits) {
    extern __shared__ float w_s[];                     // [ns]
    __shared__ float stat[2];
    const int di = blockIdx.x, head = blockIdx.y, tid = threadIdx.x;
    const int seg = seg_ids ? seg_ids[di] : di;
    const int t = cu_q[seg];
    const DecodeRange rg = decode_range(q_start[seg], kv_start[seg], window, split_tokens, 0);
    const int ns = min(rg.n_splits, max_splits);
    const float* pm = part_ml + ((size_t)di * Hq + head) * max_splits * 2;
    const float* pa = part_acc + ((size_t)di * Hq + head) * max_splits * D;
    if (tid < 64) {                                    // first wave: maximum, weights, sum in split order
        float m = -INFINITY;                           // (the maxima are base-2 exponents)
        for (int s = tid; s < ns; s += 64) m = fmaxf(m, pm[2 * s]);
        m = wave_max(m);
        for (int s = tid; s < ns; s += 64) w_s[s] = __builtin_amdgcn_exp2f(pm[2 * s] - m);
        if (tid == 0) {
            float l = 0.f;
            for (int s = 0; s < ns; ++s) l += pm[2 * s + 1] * __builtin_amdgcn_exp2f(pm[2 * s] - m);
            stat[0] = l > 0.f ? 1.0f / l : 0.f;
        }
    }
    __syncthreads();
    const float inv = stat[0];
    for (int d = tid; d < D; d += 128) {
        float o = 0.f;
#pragma unroll 8
        for (int s = 0; s < ns; ++s) o = fmaf(pa[(size_t)s * D + d], w_s[s], o);
        out[((size_t)t * Hq + head) * D + d] = from_f<bf16>(o * inv);
    }
}

// part_acc: fp32 [n_dec, Hq, max_splits, D]; part_ml: fp32 [n_dec, Hq, max_splits, 2].
// max_splits is the number of splits of the request with the most; requests with fewer leave
// the rest untouched and the merge does not read it.
extern "C" int ra_attention_decode_bf16(const void* q, void* out, void* part_acc, void* part_ml,
                                        const void* k_pool, const void* v_pool,
                                        const int* page_table, const int* cu_pages,
                                        const int* kv_start, const int* cu_q, const int* q_start,
                                        const int* seg_ids, int n_dec, int Hq, int Hkv, int D, int P,
                                        float scale, int window, int split_tokens, int max_splits,
                                        void* stream) {
    if (n_dec <= 0) return RA_OK;
    if (D % 16 != 0 || D < 16 || D > 256 || Hkv <= 0 || Hq % Hkv != 0 ||
        split_tokens <= 0 || split_tokens % DEC_CHUNK != 0 || max_splits <= 0 || max_splits > 65535 || P <= 0)
        return RA_ERR_ARG;
    const int head_blocks = Hkv * ((Hq / Hkv + DEC_MAX_GROUP - 1) / DEC_MAX_GROUP);
    if (head_blocks > 65535) return RA_ERR_ARG;
    hipStream_t st = (hipStream_t)stream;
    dim3 grid(n_dec, head_blocks, max_splits);
    const bf16* qq = (const bf16*)q;
    const bf16* kp = (const bf16*)k_pool;
    const bf16* vp = (const bf16*)v_pool;
    float* pa = (float*)part_acc;
    float* pm = (float*)part_ml;
    int rc;
    const int d16 = D / 16;
    switch ((d16 - 1) / 4) {
        case 0: rc = ra_dec_part_0(d16, grid, st, qq, pa, pm, kp, vp, page_table, cu_pages, kv_start, cu_q, q_start, seg_ids, Hq, Hkv, P, scale, window, split_tokens, max_splits); break;
        case 1: rc = ra_dec_part_1(d16, grid, st, qq, pa, pm, kp, vp, page_table, cu_pages, kv_start, cu_q, q_start, seg_ids, Hq, Hkv, P, scale, window, split_tokens, max_splits); break;
        case 2: rc = ra_dec_part_2(d16, grid, st, qq, pa, pm, kp, vp, page_table, cu_pages, kv_start, cu_q, q_start, seg_ids, Hq, Hkv, P, scale, window, split_tokens, max_splits); break;
        case 3: rc = ra_dec_part_3(d16, grid, st, qq, pa, pm, kp, vp, page_table, cu_pages, kv_start, cu_q, q_start, seg_ids, Hq, Hkv, P, scale, window, split_tokens, max_splits); break;
        default: return RA_ERR_ARG;
    }
    if (rc != RA_OK) return rc;
    if (hipGetLastError() != hipSuccess) return RA_ERR_LAUNCH;
    hipLaunchKernelGGL(attn_decode_combine_kernel, dim3(n_dec, Hq), dim3(128),
                       (size_t)max_splits * sizeof(float), st, pa, pm, (bf16*)out, kv_start, cu_q,
                       q_start, seg_ids, Hq, D, window, split_tokens, max_splits);
    return ra_launch_status();
}
#endif  // DEC_API
