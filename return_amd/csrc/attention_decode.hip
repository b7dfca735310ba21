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
#ifdef DEC_API
#include <mutex>
#include "no_alloc.h"
#endif

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

// What the kernel needs to prepare the new token's q, k and v itself (the work of the q/k/v
// preparation kernel: per-head RMSNorm of q and k, rotation, k and v into the cache;
// rollout/monkey_patch/qwen3.py:29-31, 40-42 and rollout/attention.py:10-25), so that a decode
// step has one kernel less per layer. qkv == nullptr: q is ready and the cache holds the token.
struct DecodeFused {
    const bf16* qkv;                  // [tokens, (Hq + 2 Hkv) D]: q heads, k heads, v heads of each token
    const float* w_q;                 // [D] norm weights; nullptr: no norm
    const float* w_k;
    float eps;
    const float* cos_t;               // [positions, D/2]; nullptr: no rotation
    const float* sin_t;
    bf16* k_out;                      // the pools again, to write the new token's row
    bf16* v_out;
};

#ifdef DEC_PART
// Order between the LDS accesses of one wave (a write by one lane, a read of it by another): LDS
// serves a wave's instructions in order, so only the compiler has to keep them in order.
#define WAVE_SYNC()                                              \
    do {                                                         \
        __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");   \
        __builtin_amdgcn_wave_barrier();                         \
    } while (0)

// two floats to two bf16 in one word, round to nearest even (v_cvt_pk_bf16_f32)
__device__ __forceinline__ uint32_t pack2(float a, float b) {
    const float2_t v = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}

// RMSNorm over the head and rotation of one head held as MFMA operand pieces: this lane has
// d = 32j + 8g .. +7 of it, the four lanes l, l^16, l^32, l^48 together all of it. The rotary
// partner of d is d + D/2, which is piece j + D32/2 of the same lane. Sums and products in
// 32-bit, one rounding to bfloat16 at the end, as in the preparation kernel.
// What a lane needs of the norm weight and of the angles is loaded apart from the arithmetic
// (HeadWeight, HeadAngles), so that a caller can ask for everything at once and for more after it.
template <int D32>
struct HeadWeight {
    float4_t w[D32][2];
    __device__ __forceinline__ void load(const float* __restrict__ src, int g) {      // src == nullptr: no norm
        if (src == nullptr) return;
#pragma unroll
        for (int j = 0; j < D32; ++j)
#pragma unroll
            for (int h = 0; h < 2; ++h) w[j][h] = *reinterpret_cast<const float4_t*>(src + 32 * j + 8 * g + 4 * h);
    }
};

template <int D32>
struct HeadAngles {
    float4_t c[D32 / 2][2], s[D32 / 2][2];
    __device__ __forceinline__ void load(const float* __restrict__ cs, const float* __restrict__ sn, int g) {
        if (cs == nullptr) return;                                                     // no rotation
#pragma unroll
        for (int j = 0; j < D32 / 2; ++j)
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                c[j][h] = *reinterpret_cast<const float4_t*>(cs + 32 * j + 8 * g + 4 * h);
                s[j][h] = *reinterpret_cast<const float4_t*>(sn + 32 * j + 8 * g + 4 * h);
            }
    }
};

template <int D32, bool NORM, bool ROPE>
__device__ __forceinline__ void prepare_head_as(bf16x8_t (&v)[D32], const HeadWeight<D32>& wt, float eps,
                                                const HeadAngles<D32>& an) {
    constexpr int D = 32 * D32;
    float rstd = 1.0f;
    if constexpr (NORM) {
        float ss = 0.f;
#pragma unroll
        for (int j = 0; j < D32; ++j) {
            const uint4_t u = __builtin_bit_cast(uint4_t, v[j]);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float lo = __uint_as_float(u[i] << 16), hi = __uint_as_float(u[i] & 0xffff0000u);
                ss += lo * lo + hi * hi;
            }
        }
        ss = rows_sum(ss);
        rstd = 1.0f / sqrtf(ss / (float)D + eps);
    }
    // a piece and its rotary partner at a time
#pragma unroll
    for (int j = 0; j < D32 / 2; ++j) {
        const int jp = j + D32 / 2;
        const uint4_t ua = __builtin_bit_cast(uint4_t, v[j]), ub = __builtin_bit_cast(uint4_t, v[jp]);
        float a[8], b[8];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            a[2 * i] = __uint_as_float(ua[i] << 16);
            a[2 * i + 1] = __uint_as_float(ua[i] & 0xffff0000u);
            b[2 * i] = __uint_as_float(ub[i] << 16);
            b[2 * i + 1] = __uint_as_float(ub[i] & 0xffff0000u);
        }
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                float x1 = a[4 * h + e], x2 = b[4 * h + e];
                if constexpr (NORM) {
                    x1 = x1 * rstd * wt.w[j][h][e];
                    x2 = x2 * rstd * wt.w[jp][h][e];
                }
                if constexpr (ROPE) {
                    const float y1 = x1 * an.c[j][h][e] - x2 * an.s[j][h][e];
                    x2 = x2 * an.c[j][h][e] + x1 * an.s[j][h][e];
                    x1 = y1;
                }
                a[4 * h + e] = x1;
                b[4 * h + e] = x2;
            }
        const uint4_t oa = {pack2(a[0], a[1]), pack2(a[2], a[3]), pack2(a[4], a[5]), pack2(a[6], a[7])};
        const uint4_t ob = {pack2(b[0], b[1]), pack2(b[2], b[3]), pack2(b[4], b[5]), pack2(b[6], b[7])};
        v[j] = __builtin_bit_cast(bf16x8_t, oa);
        v[jp] = __builtin_bit_cast(bf16x8_t, ob);
    }
}

// norm: the weight was loaded (its pointer was not null); rope: the angles were (the same in every lane)
template <int D32>
__device__ __forceinline__ void prepare_head(bf16x8_t (&v)[D32], const HeadWeight<D32>& wt, bool norm, float eps,
                                             const HeadAngles<D32>& an, bool rope) {
    if (norm && rope) prepare_head_as<D32, true, true>(v, wt, eps, an);
    else if (norm) prepare_head_as<D32, true, false>(v, wt, eps, an);
    else if (rope) prepare_head_as<D32, false, true>(v, wt, eps, an);
}

// LDS of one wave: its value tile, and after its passes its sums for the merge (whichever is larger)
__host__ __device__ constexpr int dec_region_bytes(int D) {
    return (DEC_CHUNK * (D + 16) * 2 > 16 * (D + 2) * 4) ? DEC_CHUNK * (D + 16) * 2 : 16 * (D + 2) * 4;
}

// merge_waves == 1: one wave per workgroup, blockIdx.z is the split, partial sums go to memory
// and attn_decode_combine_kernel merges them. merge_waves > 1: a workgroup of merge_waves waves
// per (request, kv head), wave w takes split w, and the waves' sums are merged through LDS here
// (the same sums in the same order as the merge kernel), so that nothing goes through memory and
// no second kernel runs; for requests whose splits fit one workgroup.
template <int D16, bool FUSED>
__global__ __launch_bounds__(D16 <= 8 ? 512 : 256) __attribute__((amdgpu_waves_per_eu(D16 <= 8 ? 2 : 1)))
void attn_decode_kernel(
    const bf16* __restrict__ q, float* __restrict__ part_acc, float* __restrict__ part_ml,
    const bf16* k_pool, const bf16* v_pool,
    const int* __restrict__ page_table, const int* __restrict__ cu_pages,
    const int* __restrict__ kv_start, const int* __restrict__ cu_q,
    const int* __restrict__ q_start, const int* __restrict__ seg_ids, int Hq, int Hkv, int P,
    float scale, int window, int split_tokens, int max_splits, DecodeFused fz, int merge_waves,
    bf16* __restrict__ out) {
    constexpr int D = 16 * D16;
    constexpr int D32 = D / 32;                 // full MFMA x32 steps
    constexpr bool TAIL16 = (D % 32) != 0;      // one more step, upper k half zero
    constexpr int LPR = D / 8;                  // 16-byte pieces in one value row
    constexpr int NVL = (DEC_CHUNK * LPR + 63) / 64;   // pieces of the value tile per lane
    constexpr int VS = D + 16;                  // value tile row stride in LDS (elements): rows shift by 8 banks

    constexpr int REGION = dec_region_bytes(D);
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    const int wv = threadIdx.x >> 6;             // wave of the workgroup
    uint16_t* v_s = reinterpret_cast<uint16_t*>(lds_raw + (size_t)wv * REGION);
    [[maybe_unused]] uint16_t* new_s =           // FUSED: the new token's k and v, behind the waves' regions
        reinterpret_cast<uint16_t*>(lds_raw + (size_t)merge_waves * REGION + (size_t)wv * 4 * D);

    // blockIdx.y: kv head and, when more than 16 query heads share it, which 16 of them
    const int group = Hq / Hkv, blocks = (group + DEC_MAX_GROUP - 1) / DEC_MAX_GROUP;
    const int di = blockIdx.x, kvh = blockIdx.y / blocks, hb = blockIdx.y - kvh * blocks;
    const int sp = merge_waves > 1 ? wv : (int)blockIdx.z;
    const int seg = seg_ids ? seg_ids[di] : di;
    const int lane = threadIdx.x & 63, n = lane & 15, g = lane >> 4;
    const int h0 = kvh * group + hb * DEC_MAX_GROUP;             // first query head of this wave
    const int G = min(DEC_MAX_GROUP, group - hb * DEC_MAX_GROUP);  // and how many it has
    // (the request's four numbers are asked for together; cu_q == nullptr: every request brings one
    // token, so its row is its number, and the loads of q need not wait for a table)
    const int t = cu_q ? cu_q[seg] : seg;
    const int pos_q = q_start[seg];
    const int start = kv_start[seg];
    const int first_page = cu_pages[seg];
    // A merging workgroup cuts its own request into merge_waves even splits (counted from
    // position 0), whatever the longest request of the step is.
    if (merge_waves > 1) split_tokens = max(1, (pos_q + DEC_CHUNK * merge_waves) / (DEC_CHUNK * merge_waves)) * DEC_CHUNK;
    const DecodeRange rg = decode_range(pos_q, start, window, split_tokens, sp);
    const bool empty = rg.lo > rg.hi;            // a split beyond the request's keys
    if (empty && merge_waves == 1) return;       // (in a merging workgroup the wave stays for the barrier, with no keys)
    const int* pt = page_table + first_page;
    const int p_shift = (P & (P - 1)) == 0 ? __builtin_ctz(P) : -1;

    // query operand: lane (n, g) holds head h0+n, d = 32j + 8g .. +7 (and D-16+8g.. for the tail)
    const bf16x8_t z8 = {0, 0, 0, 0, 0, 0, 0, 0};
    bf16x8_t bq[D32 > 0 ? D32 : 1];
    bf16x8_t bq_tail = z8;
    // FUSED: the new token is not among the keys of the passes; its key and value come from the
    // projection and are added at the end
    [[maybe_unused]] const bool has_new = FUSED && !empty && rg.hi == pos_q;
    const int key_hi = has_new ? pos_q - 1 : rg.hi;          // last key position read from the cache
    const int c_begin = (rg.lo / DEC_CHUNK) * DEC_CHUNK;
    // row in the pools of this lane's key of the pass that starts at c (clamped into the split so
    // that every address is valid); the next pass's rows are looked up while this one's loads run
    auto row_of = [&](int c) {
        const int kpos = max(min(max(c + lane, rg.lo), key_hi), start);
        const int idx = kpos - start;
        const int pi = p_shift >= 0 ? (idx >> p_shift) : (idx / P);
        return (pt[pi] * Hkv + kvh) * P + (idx - pi * P);     // [page][kv head][row in page]: this head's row
    };
    int row_next = 0;
    [[maybe_unused]] int first_row = 0;          // FUSED: the rows of the first pass, whose keys are asked for before the loop
    // the key tiles of a pass, straight into MFMA A operands
    bf16x8_t ak[4][D32 > 0 ? D32 : 1];
    bf16x8_t ak_tail[4];
    auto load_keys = [&](int row) {
#pragma unroll
        for (int st = 0; st < 4; ++st) {
            const int r = __shfl(row, st * 16 + n, 64);
            const bf16* kp = k_pool + (size_t)r * D;
#pragma unroll
            for (int j = 0; j < D32; ++j)
                ak[st][j] = *reinterpret_cast<const bf16x8_t*>(kp + 32 * j + 8 * g);
            if constexpr (TAIL16) {
                ak_tail[st] = z8;
                if (g < 2) ak_tail[st] = *reinterpret_cast<const bf16x8_t*>(kp + (D - 16) + 8 * g);
            }
        }
    };
    const bool any_pass = c_begin <= key_hi && rg.lo <= key_hi;
    // (at head size 256 a tile of keys beside everything the preparation holds no longer fits the registers)
    constexpr bool EARLY_KEYS = FUSED && D16 <= 12;
    if constexpr (FUSED) {
        static_assert(!TAIL16 && D32 % 2 == 0, "the fused preparation needs a head size that is a multiple of 64");
        const size_t width = (size_t)(Hq + 2 * Hkv) * D;
        const bf16* tok = fz.qkv + (size_t)t * width;
        const float* cs = fz.cos_t ? fz.cos_t + (size_t)pos_q * (D / 2) : nullptr;
        const float* sn = fz.cos_t ? fz.sin_t + (size_t)pos_q * (D / 2) : nullptr;
        const bf16* qp = tok + (size_t)(h0 + (n < G ? n : 0)) * D;
        // Everything that waits for no table is asked for at once: q, the norm weights, the angles, and
        // in the split that holds the new token its k and v. Then the first pass's keys, as soon as the
        // page table has said where they are: a wave of two passes would otherwise spend a third of its
        // life on preparing heads before its first key is on its way.
        HeadWeight<D32> wq, wk;
        HeadAngles<D32> an;
#pragma unroll
        for (int j = 0; j < D32; ++j) bq[j] = *reinterpret_cast<const bf16x8_t*>(qp + 32 * j + 8 * g);
        row_next = row_of(c_begin);
        wq.load(fz.w_q, g);
        an.load(cs, sn, g);
        bf16x8_t kn[D32];
        uint4_t vn = {0u, 0u, 0u, 0u};
        if (has_new) {
            const bf16* kp = tok + (size_t)(Hq + kvh) * D;
#pragma unroll
            for (int j = 0; j < D32; ++j) kn[j] = *reinterpret_cast<const bf16x8_t*>(kp + 32 * j + 8 * g);
            if (lane < LPR) vn = *reinterpret_cast<const uint4_t*>(tok + (size_t)(Hq + Hkv + kvh) * D + lane * 8);
            wk.load(fz.w_k, g);
        }
        if (EARLY_KEYS && any_pass) {
            const int row = row_next;
            if (c_begin + DEC_CHUNK <= key_hi) row_next = row_of(c_begin + DEC_CHUNK);
            load_keys(row);
            first_row = row;
        }
        prepare_head<D32>(bq, wq, fz.w_q != nullptr, fz.eps, an, cs != nullptr);
#pragma unroll
        for (int j = 0; j < D32; ++j) bq[j] = (n < G) ? bq[j] : z8;
        if (has_new) {
            // The new token's key (normed, rotated) and value go into the cache for the steps to
            // come, and into LDS for the end of this kernel. When more than 16 heads share the kv
            // head, each of their waves writes the same bits.
            const int idx = pos_q - start;
            const int pi = p_shift >= 0 ? (idx >> p_shift) : (idx / P);
            const size_t row_new = ((size_t)pt[pi] * Hkv + kvh) * P + (idx - pi * P);
            prepare_head<D32>(kn, wk, fz.w_k != nullptr, fz.eps, an, cs != nullptr);
            if (n == 0) {                                   // one lane of each g holds every piece once
#pragma unroll
                for (int j = 0; j < D32; ++j) {
                    *reinterpret_cast<bf16x8_t*>(fz.k_out + row_new * D + 32 * j + 8 * g) = kn[j];
                    *reinterpret_cast<bf16x8_t*>(&new_s[32 * j + 8 * g]) = kn[j];
                }
            }
            if (lane < LPR) {
                *reinterpret_cast<uint4_t*>(fz.v_out + row_new * D + lane * 8) = vn;
                *reinterpret_cast<uint4_t*>(&new_s[D + lane * 8]) = vn;
            }
        }
    } else {
        const bf16* qp = q + ((size_t)t * Hq + h0 + (n < G ? n : 0)) * D;
#pragma unroll
        for (int j = 0; j < D32; ++j) {
            bf16x8_t v = *reinterpret_cast<const bf16x8_t*>(qp + 32 * j + 8 * g);
            bq[j] = (n < G) ? v : z8;
        }
        if constexpr (TAIL16) {
            if (n < G && g < 2) bq_tail = *reinterpret_cast<const bf16x8_t*>(qp + (D - 16) + 8 * g);
        }
        row_next = row_of(c_begin);
    }

    const float scale2 = scale * 1.44269504088896340736f;      // scores in the base-2 domain
    float m_run = -INFINITY, l_run = 0.f;
    float4_t acc[D16];                           // acc[dt][i] = O^T[d = 16dt + 4g + i][head n]
#pragma unroll
    for (int dt = 0; dt < D16; ++dt) acc[dt] = float4_t{0.f, 0.f, 0.f, 0.f};

    for (int c0 = c_begin; c0 <= key_hi && rg.lo <= key_hi; c0 += DEC_CHUNK) {
        int row;
        if (EARLY_KEYS && c0 == c_begin) {
            row = first_row;                       // (its keys are on their way already)
        } else {
            row = row_next;
            if (c0 + DEC_CHUNK <= key_hi) row_next = row_of(c0 + DEC_CHUNK);
            load_keys(row);
        }
        // ---- V rows: 16-byte pieces, all loads of the pass issued now, then into LDS
        uint4_t vv[NVL];
#pragma unroll
        for (int i = 0; i < NVL; ++i) {
            const int e = min(lane + 64 * i, DEC_CHUNK * LPR - 1);
            const int r = __shfl(row, e / LPR, 64);
            vv[i] = *reinterpret_cast<const uint4_t*>(v_pool + (size_t)r * D + (e % LPR) * 8);
        }
        WAVE_SYNC();                               // the previous pass has read its value tile
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
                const bool ok = kp_abs >= rg.lo && kp_abs <= key_hi;
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
        WAVE_SYNC();                               // the value tile is complete in LDS

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

    if constexpr (FUSED) {
        if (has_new) {
            // ---- the new token as one more key: its score by plain 32-bit sums of bf16 products
            // (this lane's 8*D32 elements, then over the four lanes of the head), then the same
            // running maximum and sums as in a pass
            WAVE_SYNC();
            float dot = 0.f;
#pragma unroll
            for (int j = 0; j < D32; ++j) {
                const uint4_t kq = __builtin_bit_cast(uint4_t, bq[j]);
                const uint4_t kk = *reinterpret_cast<const uint4_t*>(&new_s[32 * j + 8 * g]);
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    dot = fmaf(__uint_as_float(kq[i] << 16), __uint_as_float(kk[i] << 16), dot);
                    dot = fmaf(__uint_as_float(kq[i] & 0xffff0000u), __uint_as_float(kk[i] & 0xffff0000u), dot);
                }
            }
            const float sc = rows_sum(dot) * scale2;
            const float m_new = fmaxf(m_run, sc);
            const float alpha = (m_run == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(m_run - m_new);
            const float pr = __builtin_amdgcn_exp2f(sc - m_new);
            l_run = l_run * alpha + pr;
            m_run = m_new;
#pragma unroll
            for (int dt = 0; dt < D16; ++dt) {
                const uint32_t* vp2 = reinterpret_cast<const uint32_t*>(&new_s[D + dt * 16 + 4 * g]);
                const uint32_t v01 = vp2[0], v23 = vp2[1];
                acc[dt][0] = fmaf(pr, __uint_as_float(v01 << 16), acc[dt][0] * alpha);
                acc[dt][1] = fmaf(pr, __uint_as_float(v01 & 0xffff0000u), acc[dt][1] * alpha);
                acc[dt][2] = fmaf(pr, __uint_as_float(v23 << 16), acc[dt][2] * alpha);
                acc[dt][3] = fmaf(pr, __uint_as_float(v23 & 0xffff0000u), acc[dt][3] * alpha);
            }
        }
    }

    if (merge_waves > 1) {
        // ---- this wave's sums into its own region (its value tile is no longer needed), then
        // every thread of the workgroup merges a piece of the result over the waves, in wave order
        WAVE_SYNC();
        float* mine = reinterpret_cast<float*>(lds_raw + (size_t)wv * REGION);      // [16][D] sums, then [16][2] m, l
#pragma unroll
        for (int dt = 0; dt < D16; ++dt) *reinterpret_cast<float4_t*>(mine + n * D + dt * 16 + 4 * g) = acc[dt];
        if (g == 0) {
            mine[16 * D + 2 * n] = m_run;
            mine[16 * D + 2 * n + 1] = l_run;
        }
        __syncthreads();
        const int threads = merge_waves * 64;
        for (int idx = threadIdx.x; idx < G * (D / 4); idx += threads) {
            const int hn = idx / (D / 4), d4 = idx - hn * (D / 4);
            float mx = -INFINITY;
            for (int w = 0; w < merge_waves; ++w)
                mx = fmaxf(mx, reinterpret_cast<const float*>(lds_raw + (size_t)w * REGION)[16 * D + 2 * hn]);
            float4_t o = {0.f, 0.f, 0.f, 0.f};
            float l = 0.f;
            for (int w = 0; w < merge_waves; ++w) {
                const float* other = reinterpret_cast<const float*>(lds_raw + (size_t)w * REGION);
                const float mw = other[16 * D + 2 * hn];
                const float e = (mw == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(mw - mx);
                const float4_t a = *reinterpret_cast<const float4_t*>(other + hn * D + 4 * d4);
                o[0] = fmaf(a[0], e, o[0]); o[1] = fmaf(a[1], e, o[1]);
                o[2] = fmaf(a[2], e, o[2]); o[3] = fmaf(a[3], e, o[3]);
                l += other[16 * D + 2 * hn + 1] * e;
            }
            const float inv = l > 0.f ? 1.0f / l : 0.f;
            const uint2 packed = {pack2(o[0] * inv, o[1] * inv), pack2(o[2] * inv, o[3] * inv)};
            *reinterpret_cast<uint2*>(out + ((size_t)t * Hq + h0 + hn) * D + 4 * d4) = packed;
        }
        return;
    }

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
template <int N, bool FUSED>
static int dec_launch_one(dim3 grid, hipStream_t st, const bf16* q, float* pa, float* pm, const bf16* kp,
                          const bf16* vp, const int* pt, const int* cup, const int* kvs, const int* cuq,
                          const int* qs, const int* segs, int Hq, int Hkv, int P, float scale, int window,
                          int split_tokens, int max_splits, DecodeFused fz, int merge_waves, bf16* out) {
    constexpr int D = 16 * N;
    const size_t lds = (size_t)merge_waves * (dec_region_bytes(D) + (FUSED ? 4 * D : 0));
    auto kern = attn_decode_kernel<N, FUSED>;
    static size_t allowed = 64 * 1024;                        // per instantiation: raised when needed
    if (lds > allowed) {
        if (lds > 160 * 1024 ||
            hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)lds) != hipSuccess)
            return RA_ERR_ARG;
        allowed = lds;
    }
    hipLaunchKernelGGL(kern, grid, dim3(64 * merge_waves), lds, st, q, pa, pm, kp, vp, pt, cup, kvs, cuq, qs,
                       segs, Hq, Hkv, P, scale, window, split_tokens, max_splits, fz, merge_waves, out);
    return RA_OK;
}

extern "C" int DEC_CAT(ra_dec_part_, DEC_PART)(int D16, dim3 grid, hipStream_t st, const bf16* q, float* pa,
                                              float* pm, const bf16* kp, const bf16* vp, const int* pt,
                                              const int* cup, const int* kvs, const int* cuq,
                                              const int* qs, const int* segs, int Hq, int Hkv, int P,
                                              float scale, int window, int split_tokens,
                                              int max_splits, DecodeFused fz, int merge_waves, bf16* out) {
#define DEC_ARGS grid, st, q, pa, pm, kp, vp, pt, cup, kvs, cuq, qs, segs, Hq, Hkv, P, scale, window, \
                 split_tokens, max_splits, fz, merge_waves, out
    if (fz.qkv != nullptr) {                      // head sizes 64, 128, 192, 256: one of them in each part
        if (D16 != 4 * DEC_PART + 4) return RA_ERR_ARG;
        return dec_launch_one<4 * DEC_PART + 4, true>(DEC_ARGS);
    }
    switch (D16) {
        case 4 * DEC_PART + 1: return dec_launch_one<4 * DEC_PART + 1, false>(DEC_ARGS);
        case 4 * DEC_PART + 2: return dec_launch_one<4 * DEC_PART + 2, false>(DEC_ARGS);
        case 4 * DEC_PART + 3: return dec_launch_one<4 * DEC_PART + 3, false>(DEC_ARGS);
        case 4 * DEC_PART + 4: return dec_launch_one<4 * DEC_PART + 4, false>(DEC_ARGS);
        default: return RA_ERR_ARG;
    }
#undef DEC_ARGS
}
#endif  // DEC_PART

#ifdef DEC_API

#define DEC_PART_ARGS int D16, dim3 grid, hipStream_t st, const bf16* q, float* pa, float* pm,        \
    const bf16* kp, const bf16* vp, const int* pt, const int* cup, const int* kvs, const int* cuq,   \
    const int* qs, const int* segs, int Hq, int Hkv, int P, float scale, int window,                 \
    int split_tokens, int max_splits, DecodeFused fz, int merge_waves, bf16* out
extern "C" int ra_dec_part_0(DEC_PART_ARGS);
extern "C" int ra_dec_part_1(DEC_PART_ARGS);
extern "C" int ra_dec_part_2(DEC_PART_ARGS);
extern "C" int ra_dec_part_3(DEC_PART_ARGS);

// Merge of the splits: out = sum_s acc_s * w_s / sum_s l_s * w_s, w_s = exp(m_s - m).
// The kernel is a chain of loads that wait for each other (the request's tables, then the splits'
// maxima, then their sums), and each link costs about a microsecond after a kernel that wrote them.
// So a thread's COMBINE_AHEAD splits' maxima and sums are asked for at once with the tables, before it
// is known how many splits hold keys: what a split beyond them left in memory (never written by this
// call: whatever the allocator, or an earlier call on the library's own buffer, left there) is read,
// at addresses clamped to the request's max_splits places, and not used: every use below is guarded
// by s < ns, and that guard must stay ahead of the arithmetic, since such values may be NaN.
// A request of more than COMBINE_AHEAD splits has GROUPS groups of 128 threads, each for a run of
// at most COMBINE_AHEAD consecutive splits (or more, by a loop, beyond 8 groups' worth), so that all
// loads of a long request are on their way together; the groups' sums are merged through LDS in group
// order. Every thread forms the weights itself (the same numbers in the same order), so that within a
// group no thread waits for another.
#define COMBINE_AHEAD 16
#define COMBINE_MAX_GROUPS 8
template <int GROUPS>
__global__ __launch_bounds__(128 * GROUPS) void attn_decode_combine_kernel(
    const float* __restrict__ part_acc, const float* __restrict__ part_ml, bf16* __restrict__ out,
    const int* __restrict__ kv_start, const int* __restrict__ cu_q, const int* __restrict__ q_start,
    const int* __restrict__ seg_ids, int Hq, int D, int window, int split_tokens, int max_splits) {
    const int di = blockIdx.x, head = blockIdx.y, tid = threadIdx.x & 127, grp = threadIdx.x >> 7;
    // this group's run of splits: [first, first + per)
    const int per = GROUPS == 1 ? max_splits : (max_splits + GROUPS - 1) / GROUPS;
    const int first = grp * per;
    const float* pm = part_ml + (((size_t)di * Hq + head) * max_splits + first) * 2;
    const float* pa = part_acc + (((size_t)di * Hq + head) * max_splits + first) * D;
    const int d0 = min(tid, D - 1), d1 = min(tid + 128, D - 1);       // this thread's columns (D <= 256), clamped for the loads
    float2_t ml[COMBINE_AHEAD];
    float a0[COMBINE_AHEAD], a1[COMBINE_AHEAD];
    const int last_valid = max(max_splits - 1 - first, 0);           // (a group beyond the splits reads the last one and uses nothing)
    const bool any = first < max_splits;
#pragma unroll
    for (int s = 0; s < COMBINE_AHEAD; ++s) {
        const int sc = any ? min(s, last_valid) : 0;
        const float* pms = any ? pm : part_ml + ((size_t)di * Hq + head) * max_splits * 2;
        const float* pas = any ? pa : part_acc + ((size_t)di * Hq + head) * max_splits * D;
        ml[s] = *reinterpret_cast<const float2_t*>(pms + 2 * sc);
        a0[s] = pas[(size_t)sc * D + d0];
        a1[s] = pas[(size_t)sc * D + d1];
    }
    const int seg = seg_ids ? seg_ids[di] : di;
    const int t = cu_q ? cu_q[seg] : seg;
    const DecodeRange rg = decode_range(q_start[seg], kv_start[seg], window, split_tokens, 0);
    const int ns_all = min(rg.n_splits, max_splits);
    const int ns = max(0, min(ns_all - first, per));        // splits of this group that hold keys
    float m = -INFINITY;                                   // (the maxima are base-2 exponents)
#pragma unroll
    for (int s = 0; s < COMBINE_AHEAD; ++s) m = s < ns ? fmaxf(m, ml[s][0]) : m;
#pragma unroll 8
    for (int s = COMBINE_AHEAD; s < ns; ++s) m = fmaxf(m, pm[2 * s]);
    float l = 0.f, o0 = 0.f, o1 = 0.f;
#pragma unroll
    for (int s = 0; s < COMBINE_AHEAD; ++s) {
        if (s < ns) {
            const float w = __builtin_amdgcn_exp2f(ml[s][0] - m);
            l += ml[s][1] * w;
            o0 = fmaf(a0[s], w, o0);
            o1 = fmaf(a1[s], w, o1);
        }
    }
#pragma unroll 8
    for (int s = COMBINE_AHEAD; s < ns; ++s) {
        const float w = __builtin_amdgcn_exp2f(pm[2 * s] - m);
        l += pm[2 * s + 1] * w;
        o0 = fmaf(pa[(size_t)s * D + d0], w, o0);
        o1 = fmaf(pa[(size_t)s * D + d1], w, o1);
    }
    if constexpr (GROUPS > 1) {
        // the groups' (m, l, o0, o1) per thread, merged by group 0 in group order
        __shared__ float4_t sums[GROUPS][128];
        sums[grp][tid] = float4_t{m, l, o0, o1};
        __syncthreads();
        if (grp != 0) return;
        float mx = -INFINITY;
#pragma unroll
        for (int g2 = 0; g2 < GROUPS; ++g2) mx = fmaxf(mx, sums[g2][tid][0]);
        l = 0.f; o0 = 0.f; o1 = 0.f;
#pragma unroll
        for (int g2 = 0; g2 < GROUPS; ++g2) {
            const float4_t v = sums[g2][tid];
            const float w = (v[0] == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(v[0] - mx);
            l = fmaf(v[1], w, l);
            o0 = fmaf(v[2], w, o0);
            o1 = fmaf(v[3], w, o1);
        }
    }
    const float inv = l > 0.f ? 1.0f / l : 0.f;
    bf16* o = out + ((size_t)t * Hq + head) * D;
    if (tid < D) o[tid] = from_f<bf16>(o0 * inv);
    if (tid + 128 < D) o[tid + 128] = from_f<bf16>(o1 * inv);
}

// part_acc: fp32 [n_dec, Hq, max_splits, D]; part_ml: fp32 [n_dec, Hq, max_splits, 2].
// max_splits is the number of splits of the request with the most; requests with fewer leave
// the rest untouched and the merge does not read it.
// merge != 0: the splits of a request are the waves of one workgroup and are merged there (no partial
// sums in memory, no merge kernel); max_splits must not exceed ra_attention_decode_merge_waves(D).
// Most waves (splits) of a merging workgroup for head size D: what the LDS holds and the kernel's
// launch bounds allow.
extern "C" int ra_attention_decode_merge_waves(int D) {
    if (D % 16 != 0 || D < 16 || D > 256) return 0;
    const int region = (DEC_CHUNK * (D + 16) * 2 > 16 * (D + 2) * 4) ? DEC_CHUNK * (D + 16) * 2 : 16 * (D + 2) * 4;
    const int by_lds = (160 * 1024 - 1024) / (region + 4 * D);
    const int by_bounds = D <= 128 ? 8 : 4;
    return by_lds < by_bounds ? by_lds : by_bounds;
}

static int decode_launch(const bf16* qq, void* out, float* pa, float* pm, const bf16* kp, const bf16* vp,
                         const int* page_table, const int* cu_pages, const int* kv_start, const int* cu_q,
                         const int* q_start, const int* seg_ids, int n_dec, int Hq, int Hkv, int D, int P,
                         float scale, int window, int split_tokens, int max_splits, DecodeFused fz,
                         int merge, hipStream_t st) {
    if (n_dec <= 0) return RA_OK;
    if (D % 16 != 0 || D < 16 || D > 256 || Hkv <= 0 || Hq % Hkv != 0 ||
        split_tokens <= 0 || split_tokens % DEC_CHUNK != 0 || max_splits <= 0 || max_splits > 65535 || P <= 0)
        return RA_ERR_ARG;
    const int head_blocks = Hkv * ((Hq / Hkv + DEC_MAX_GROUP - 1) / DEC_MAX_GROUP);
    if (head_blocks > 65535) return RA_ERR_ARG;
    if (merge && (max_splits < 2 || max_splits > ra_attention_decode_merge_waves(D) || window > 0)) return RA_ERR_ARG;
    dim3 grid(n_dec, head_blocks, merge ? 1 : max_splits);
    const int merge_waves = merge ? max_splits : 1;
    int rc;
    const int d16 = D / 16;
#define DEC_GO(N) rc = ra_dec_part_##N(d16, grid, st, qq, pa, pm, kp, vp, page_table, cu_pages, kv_start, cu_q, \
                                       q_start, seg_ids, Hq, Hkv, P, scale, window, split_tokens, max_splits, fz, \
                                       merge_waves, (bf16*)out)
    switch ((d16 - 1) / 4) {
        case 0: DEC_GO(0); break;
        case 1: DEC_GO(1); break;
        case 2: DEC_GO(2); break;
        case 3: DEC_GO(3); break;
        default: return RA_ERR_ARG;
    }
#undef DEC_GO
    if (rc != RA_OK) return rc;
    if (hipGetLastError() != hipSuccess) return RA_ERR_LAUNCH;
    if (merge) return RA_OK;
#define DEC_COMBINE(G) hipLaunchKernelGGL(attn_decode_combine_kernel<G>, dim3(n_dec, Hq), dim3(128 * G), 0, st, pa, pm, \
                                          (bf16*)out, kv_start, cu_q, q_start, seg_ids, Hq, D, window, split_tokens, max_splits)
    const int groups = (max_splits + COMBINE_AHEAD - 1) / COMBINE_AHEAD;
    if (groups <= 1) DEC_COMBINE(1);
    else if (groups <= 2) DEC_COMBINE(2);
    else if (groups <= 4) DEC_COMBINE(4);
    else DEC_COMBINE(COMBINE_MAX_GROUPS);
#undef DEC_COMBINE
    return ra_launch_status();
}

extern "C" int ra_attention_decode_bf16(const void* q, void* out, void* part_acc, void* part_ml,
                                        const void* k_pool, const void* v_pool,
                                        const int* page_table, const int* cu_pages,
                                        const int* kv_start, const int* cu_q, const int* q_start,
                                        const int* seg_ids, int n_dec, int Hq, int Hkv, int D, int P,
                                        float scale, int window, int split_tokens, int max_splits,
                                        int merge, void* stream) {
    DecodeFused none = {};
    return decode_launch((const bf16*)q, out, (float*)part_acc, (float*)part_ml, (const bf16*)k_pool,
                         (const bf16*)v_pool, page_table, cu_pages, kv_start, cu_q, q_start, seg_ids, n_dec, Hq,
                         Hkv, D, P, scale, window, split_tokens, max_splits, none, merge, (hipStream_t)stream);
}

// The same for requests whose new token has not been prepared: qkv [tokens, (Hq + 2 Hkv) D] as the
// projection left it. The kernel norms (w_q, w_k [D]; nullptr: no norm) and rotates (cos, sin
// [positions, D/2] at the request's position; nullptr: no rotation) q and k itself and writes k and
// v of the new token into the pools. Head sizes 64, 128, 192, 256. cu_q == nullptr: every request brings
// exactly one token and row i of qkv and of out is request i (no seg_ids then).
extern "C" int ra_attention_decode_fused_bf16(const void* qkv, void* out, void* part_acc, void* part_ml,
                                              void* k_pool, void* v_pool, const int* page_table,
                                              const int* cu_pages, const int* kv_start, const int* cu_q,
                                              const int* q_start, const int* seg_ids, int n_dec, int Hq,
                                              int Hkv, int D, int P, float scale, int window,
                                              int split_tokens, int max_splits, const float* w_q,
                                              const float* w_k, float eps, const float* cos_t,
                                              const float* sin_t, int merge, void* stream) {
    if (qkv == nullptr || D % 64 != 0 || (w_q == nullptr) != (w_k == nullptr) ||
        (cos_t == nullptr) != (sin_t == nullptr) || (cu_q == nullptr && seg_ids != nullptr))
        return RA_ERR_ARG;
    DecodeFused fz = {(const bf16*)qkv, w_q, w_k, eps, cos_t, sin_t, (bf16*)k_pool, (bf16*)v_pool};
    return decode_launch(nullptr, out, (float*)part_acc, (float*)part_ml, (const bf16*)k_pool,
                         (const bf16*)v_pool, page_table, cu_pages, kv_start, cu_q, q_start, seg_ids, n_dec, Hq,
                         Hkv, D, P, scale, window, split_tokens, max_splits, fz, merge, (hipStream_t)stream);
}

// ---- the entry point that allocates nothing (declared in no_alloc.h) ----
// The partial sums live in a file-scope device array. In host code that name is a stand-in of the
// host side, not a device address: the address on each GPU (every GPU has its own copy) is asked
// for once per device with hipGetSymbolAddress and kept; only that pointer goes to kernels.
static __device__ __align__(256) float ra_decode_scratch[RA_DECODE_STATIC_FLOATS];

#define RA_MAX_DEVICES 64
static std::mutex ra_scratch_lock;
static float* ra_scratch_on_device[RA_MAX_DEVICES] = {};

// The device array's address on the current device, or nullptr. Asked for at the first call on a device.
static float* decode_scratch_here() {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= RA_MAX_DEVICES) return nullptr;
    std::lock_guard<std::mutex> hold(ra_scratch_lock);
    if (ra_scratch_on_device[dev] == nullptr) {
        void* p = nullptr;
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(ra_decode_scratch)) != hipSuccess) {
            (void)hipGetLastError();
            return nullptr;
        }
        ra_scratch_on_device[dev] = (float*)p;
    }
    return ra_scratch_on_device[dev];
}

extern "C" int ra_attention_decode_static_bf16(const void* q, void* out, const void* k_pool, const void* v_pool,
                                               const int* page_table, const int* cu_pages,
                                               const int* kv_start, const int* cu_q, const int* q_start,
                                               const int* seg_ids, int n_dec, int Hq, int Hkv, int D, int P,
                                               float scale, int window, int split_tokens, int max_splits,
                                               int merge, void* stream) {
    if (n_dec < 0 || Hq <= 0 || D <= 0 || max_splits <= 0) return RA_ERR_ARG;
    float* pa = nullptr;
    float* pm = nullptr;
    if (!merge && n_dec > 0) {
        const unsigned long long acc = (unsigned long long)n_dec * Hq * max_splits * D;
        const unsigned long long ml = (unsigned long long)n_dec * Hq * max_splits * 2;
        if (acc + ml > (unsigned long long)RA_DECODE_STATIC_FLOATS) return RA_ERR_SCRATCH;
        float* base = decode_scratch_here();
        if (base == nullptr) return RA_ERR_SETUP;
        pa = base;                 // [n_dec, Hq, max_splits, D]
        pm = base + acc;           // [n_dec, Hq, max_splits, 2]
    }
    DecodeFused none = {};
    return decode_launch((const bf16*)q, out, pa, pm, (const bf16*)k_pool, (const bf16*)v_pool, page_table,
                         cu_pages, kv_start, cu_q, q_start, seg_ids, n_dec, Hq, Hkv, D, P, scale, window,
                         split_tokens, max_splits, none, merge, (hipStream_t)stream);
}
#endif  // DEC_API
