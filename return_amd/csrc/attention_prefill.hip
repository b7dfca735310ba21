// Prefill attention for bfloat16: portions of prompts (two or more new tokens of a request)
// over everything the paged cache holds for it, causal by position, optional window.
//
// What it restates of the reference: rollout/attention.py:45-142 (_prefill_kernel: packed
// varlen causal GQA attention over paged K/V with online softmax; programs are (q tile,
// segment, head); pages above the tile's last position are skipped, 103-106; mask
// pos_q >= pos_k, 126-127). Different here: keys are already rotated in the cache; the grid
// is a flat list of (request, q tile) made on the host instead of ceil(S/128) programs per
// segment that mostly exit early (attention.py:168-174).
//
// BUILD-VARIANTS: PRE_PART=0 PRE_PART=1 PRE_PART=2 PRE_PART=3 PRE_API=1
//
// One workgroup of four waves per (q tile of 64*QG rows, query head); wave w owns QG groups of
// 16 rows, 16*QG*w .. 16*QG*(w+1)-1. QG is 2 up to head size 128 and 1 beyond: with two groups
// every operand that comes out of LDS (a K row piece, a V^T piece) feeds two MFMAs, which
// halves the LDS traffic per flop; beyond 128 the accumulators of two groups no longer fit.
// Per pass a tile of BN keys sits in LDS, K and V both row-major with padded rows; the next
// tile's rows are already on their way from the cache into registers while this one is used.
//  scores  S^T = K Q^T by MFMA 16x16x32 bf16: A = K tile rows from LDS, B = 16 query rows
//          held in registers. Lane (n, g) gets query n of each group, keys 4g..4g+3 of each
//          16-key tile.
//  P.V     O^T += V^T P^T by the same MFMA. The contraction runs over keys in the order the
//          lanes already hold them: k-slot (g, e) of a 32-key block is key 16*(e/4) + 4g + e%4,
//          so P goes from the softmax registers straight into the B operand. The A operand,
//          V^T, comes from the row-major V tile through the transposing LDS read of gfx950
//          (ds_read_b64_tr_b16): within 16 lanes, lane l receives element l%4 of the 8 bytes
//          addressed by lanes l/4, l/4+4, l/4+8, l/4+12. Lane l' therefore points at key
//          4g + l'/4 (and 16 more for the second half), columns 16dt + 4(l'%4)..+3, and lane n
//          ends up with column 16dt + n of keys 4g..4g+3.
// A trailing 16 of D is a 16x16x32 step with the upper k half zero (one MFMA shape per chain).
#include "common.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef short short4_t __attribute__((ext_vector_type(4)));
typedef float float4_t __attribute__((ext_vector_type(4)));

// head sizes up to 16 * PRE_WIDE_D16 run two groups of query rows per wave (tiles of 128 rows)
#define PRE_WIDE_D16 8

#ifdef PRE_PART

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float float2_t __attribute__((ext_vector_type(2)));
// two floats to two bf16 in one word, round to nearest even (v_cvt_pk_bf16_f32)
__device__ __forceinline__ uint32_t pack2(float a, float b) {
    const float2_t v = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}

typedef short short8_t __attribute__((ext_vector_type(8)));
typedef uint32_t uint4_t __attribute__((ext_vector_type(4)));

typedef short4_t __attribute__((address_space(3))) * lds_short4_ptr;

template <int D16, int QG, int KSPLIT>
__global__ __launch_bounds__(256 * KSPLIT) __attribute__((amdgpu_waves_per_eu(2))) void attn_prefill_kernel(
    const bf16* __restrict__ q, bf16* __restrict__ out, const bf16* __restrict__ k_pool,
    const bf16* __restrict__ v_pool, const int* __restrict__ page_table,
    const int* __restrict__ cu_pages, const int* __restrict__ kv_start,
    const int* __restrict__ cu_q, const int* __restrict__ q_start,
    const int* __restrict__ tiles,       // [n_tiles][2]: request number, first row of the tile within it
    int n_tiles, int Hq, int Hkv, int P, float scale, int window) {
    constexpr int D = 16 * D16;
    constexpr int D32 = D / 32;
    constexpr bool TAIL16 = (D % 32) != 0;
    constexpr int BM = 64 * QG;                         // query rows per workgroup
    constexpr int BN = (D <= 128) ? 64 : 32;            // keys per pass
    constexpr int KS = D + 8;                           // K tile row stride (elements): rows shift by 4 banks
    constexpr int VS = D + 16;                          // V tile row stride: rows shift by 8 banks (transposing reads)
    constexpr int LPR = D / 8;                          // 16-byte pieces in one row
    constexpr int TPK = 256 / BN;                       // threads that share the loading of one key row
    constexpr int NLD = (LPR + TPK - 1) / TPK;          // pieces of K (and of V) per thread per tile

    // Per group of four waves two tiles of K and of V: one is used while the next is written. With
    // KSPLIT == 2 a second group of four waves works on the same query rows and takes every other
    // key tile; at the end its sums are merged into the first group's through the same memory.
    constexpr int TILE = BN * KS + BN * VS;             // elements of one K tile and one V tile
    constexpr int MERGE_SLOTS = 4 * D16 + 2;            // per lane and query group: the accumulators, m and l
    constexpr size_t TILE_BYTES = (size_t)KSPLIT * 2 * TILE * 2;
    constexpr size_t MERGE_BYTES = KSPLIT > 1 ? (size_t)4 * QG * MERGE_SLOTS * 64 * 4 : 0;
    __shared__ __attribute__((aligned(16))) unsigned char lds_raw[TILE_BYTES > MERGE_BYTES ? TILE_BYTES : MERGE_BYTES];
    const int grp = threadIdx.x >> 8;                   // which group of four waves
    uint16_t* const tiles_s = reinterpret_cast<uint16_t*>(lds_raw) + (size_t)grp * 2 * TILE;
#define K_S(buf_) (tiles_s + (buf_) * TILE)
#define V_S(buf_) (tiles_s + (buf_) * TILE + BN * KS)

    // Workgroups go to the 8 XCDs round-robin by their number, and each XCD has an L2 of its own:
    // all workgroups of one kv head are sent to the same XCD, so that its keys and values are
    // fetched into one L2 only (when the kv heads divide evenly among the XCDs).
    int tile, head;
    {
        const int wg = blockIdx.x, per_head = n_tiles;
        if (Hkv % 8 == 0) {
            const int xcd = wg & 7, slot = wg >> 3;              // slot-th workgroup of this XCD
            const int G_ = Hq / Hkv;
            const int heads_here = Hq >> 3;
            const int hh = slot % heads_here;                    // which of this XCD's query heads
            const int kv_local = hh / G_;                        // kv heads xcd, xcd+8, ... belong here
            head = (kv_local * 8 + xcd) * G_ + hh % G_;
            tile = slot / heads_here;                            // tiles come longest first: all heads' long ones start early
        } else {
            head = wg % Hq;
            tile = wg / Hq;
        }
    }
    const int seg = tiles[2 * tile], q_off = tiles[2 * tile + 1];
    const int tid = threadIdx.x & 255, wave = tid >> 6, lane = tid & 63, n = lane & 15, g = lane >> 4;
    const int kvh = head / (Hq / Hkv);
    const int q_len = cu_q[seg + 1] - cu_q[seg];
    const int pos0 = q_start[seg];                       // position of the request's first new token
    const int start = kv_start[seg];
    const int* pt = page_table + cu_pages[seg];

    // this lane's query rows (for the B operands and for the mask): row n of each of the wave's groups
    int pos_q[QG];
    bool q_ok[QG];
    const bf16x8_t z8 = {0, 0, 0, 0, 0, 0, 0, 0};
    bf16x8_t bq[QG][D32 > 0 ? D32 : 1];
    bf16x8_t bq_tail[QG];
#pragma unroll
    for (int qg = 0; qg < QG; ++qg) {
        const int q_local = q_off + (wave * QG + qg) * 16 + n;
        q_ok[qg] = q_local < q_len;
        pos_q[qg] = pos0 + q_local;
        const bf16* qp = q + ((size_t)(cu_q[seg] + (q_ok[qg] ? q_local : 0)) * Hq + head) * D;
#pragma unroll
        for (int j = 0; j < D32; ++j) {
            bf16x8_t v = *reinterpret_cast<const bf16x8_t*>(qp + 32 * j + 8 * g);
            bq[qg][j] = q_ok[qg] ? v : z8;
        }
        bq_tail[qg] = z8;
        if constexpr (TAIL16) {
            if (q_ok[qg] && g < 2) bq_tail[qg] = *reinterpret_cast<const bf16x8_t*>(qp + (D - 16) + 8 * g);
        }
    }

    // keys this tile needs: from the earliest key any of its rows may read to its last row's position
    const int tile_first_pos = pos0 + q_off;
    const int tile_last_pos = pos0 + min(q_off + BM, q_len) - 1;
    int first_key = start;
    if (window > 0 && tile_first_pos - window + 1 > first_key) first_key = tile_first_pos - window + 1;

    const float scale2 = scale * 1.44269504088896340736f;
    // positions of the first and last row of this wave (wave-uniform, for skipping the mask)
    const int wave_first_pos = pos0 + q_off + wave * QG * 16;
    const int wave_last_pos = wave_first_pos + QG * 16 - 1;
    float m_run[QG], l_run[QG];                          // (the running maxima are raw scores, before the scale)
    float4_t acc[QG][D16];
#pragma unroll
    for (int qg = 0; qg < QG; ++qg) {
        m_run[qg] = -INFINITY;
        l_run[qg] = 0.f;
#pragma unroll
        for (int dt = 0; dt < D16; ++dt) acc[qg][dt] = float4_t{0.f, 0.f, 0.f, 0.f};
    }

    // what each thread moves per tile: its key row's pieces my_sub, my_sub + TPK, ... of K and of V
    uint4_t kreg[NLD], vreg[NLD];                        // native vectors: they stay in registers
    const int my_key = tid / TPK, my_sub = tid % TPK;
    // cache row of key position kp (clamped into what this tile may read, so every address is valid)
    const int p_shift = (P & (P - 1)) == 0 ? __builtin_ctz(P) : -1;
#define ROW_OF(kp)                                                                  \
    ([&]() {                                                                        \
        const int idx_ = min(max((kp), first_key), tile_last_pos) - start;          \
        const int pi_ = p_shift >= 0 ? (idx_ >> p_shift) : (idx_ / P);              \
        return (pt[pi_] * Hkv + kvh) * P + (idx_ - pi_ * P);                        \
    }())
#define FETCH_ROW(row_)                                                             \
    {                                                                               \
        const size_t base_ = (size_t)(row_) * D;                                    \
        _Pragma("unroll") for (int i = 0; i < NLD; ++i) {                           \
            const int p_ = my_sub + TPK * i;                                        \
            if (p_ < LPR) {                                                         \
                kreg[i] = *reinterpret_cast<const uint4_t*>(k_pool + base_ + 8 * p_); \
                vreg[i] = *reinterpret_cast<const uint4_t*>(v_pool + base_ + 8 * p_); \
            }                                                                       \
        }                                                                           \
    }
#define STAGE_TO(buf_)                                                              \
    _Pragma("unroll") for (int i = 0; i < NLD; ++i) {                               \
        const int p_ = my_sub + TPK * i;                                            \
        if (p_ < LPR) {                                                             \
            *reinterpret_cast<uint4_t*>(K_S(buf_) + my_key * KS + 8 * p_) = kreg[i]; \
            *reinterpret_cast<uint4_t*>(V_S(buf_) + my_key * VS + 8 * p_) = vreg[i]; \
        }                                                                           \
    }
    // group grp takes the key tiles grp, grp + KSPLIT, grp + 2 KSPLIT, ... counted from c_first
    const int c_first = (first_key / BN) * BN;
    constexpr int STEP = KSPLIT * BN;                    // from one tile of a group to its next
    int row_next;                                        // row of this thread's key in the tile fetched next
    {
        const int c_mine = c_first + grp * BN;
        const int r0 = ROW_OF(c_mine + my_key);
        row_next = ROW_OF(c_mine + STEP + my_key);
        FETCH_ROW(r0)
        STAGE_TO(0)
        FETCH_ROW(row_next)                              // the group's second tile (or a repeat of valid rows if there is none)
        row_next = ROW_OF(c_mine + 2 * STEP + my_key);
    }
    __syncthreads();

    int it = 0;
    for (int c_it = c_first; c_it <= tile_last_pos; c_it += STEP, ++it) {
        const int c0 = c_it + grp * BN;                  // beyond tile_last_pos: this group sits the pass out
        const int cur = it & 1;
        const uint16_t* k_cur = K_S(cur);
        const uint16_t* v_cur = V_S(cur);
        if (c0 + STEP <= tile_last_pos) {
            // the next tile, asked for one pass ago, goes into the other buffer (which every wave left
            // at the last barrier); then the tile after it is asked for
            STAGE_TO(cur ^ 1)
            if (c0 + 2 * STEP <= tile_last_pos) {
                FETCH_ROW(row_next)
                row_next = ROW_OF(c0 + 3 * STEP + my_key);
            }
        }

        // a tile that lies wholly above every row of the wave has nothing for it
        if (c0 <= wave_last_pos && c0 <= tile_last_pos) {
        // ---- scores of the wave's rows against the BN keys; a K piece from LDS serves every group
        float4_t cs[QG][BN / 16];
#pragma unroll
        for (int st = 0; st < BN / 16; ++st) {
#pragma unroll
            for (int qg = 0; qg < QG; ++qg) cs[qg][st] = float4_t{0.f, 0.f, 0.f, 0.f};
            const uint16_t* kr = &k_cur[(st * 16 + n) * KS];
#pragma unroll
            for (int j = 0; j < D32; ++j) {
                const bf16x8_t a = *reinterpret_cast<const bf16x8_t*>(kr + 32 * j + 8 * g);
#pragma unroll
                for (int qg = 0; qg < QG; ++qg)
                    cs[qg][st] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, bq[qg][j], cs[qg][st], 0, 0, 0);
            }
            if constexpr (TAIL16) {
                bf16x8_t a = z8;
                if (g < 2) a = *reinterpret_cast<const bf16x8_t*>(kr + (D - 16) + 8 * g);
#pragma unroll
                for (int qg = 0; qg < QG; ++qg)
                    cs[qg][st] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, bq_tail[qg], cs[qg][st], 0, 0, 0);
            }
        }
        MFMA_SETTLE();
        // p = 2^((s - m) * scale * log2(e)) with s the raw score and m the raw maximum of the row: one fused
        // multiply-add and one exponential a score (the scale is positive, so the maximum may be taken first).
        // a tile that lies wholly below every row of the wave and inside every window needs no mask
        const bool need_mask = (c0 + BN - 1 > wave_first_pos) || (c0 < first_key) ||
                               (window > 0 && c0 <= wave_last_pos - window);
        uint4_t pw[QG][BN / 32];                         // P as bf16, in the order the B operand wants
#pragma unroll
        for (int qg = 0; qg < QG; ++qg) {
            float s[BN / 16][4];
            float mx = -INFINITY;
            if (need_mask) {
#pragma unroll
                for (int st = 0; st < BN / 16; ++st) {
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int kpos = c0 + st * 16 + 4 * g + i;
                        bool ok = kpos >= first_key && kpos <= pos_q[qg];
                        if (window > 0) ok = ok && kpos > pos_q[qg] - window;
                        s[st][i] = ok ? cs[qg][st][i] : -INFINITY;
                        mx = fmaxf(mx, s[st][i]);
                    }
                }
            } else {
#pragma unroll
                for (int st = 0; st < BN / 16; ++st) {
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        s[st][i] = cs[qg][st][i];
                        mx = fmaxf(mx, s[st][i]);
                    }
                }
            }
            mx = rows_max(mx);
            const float m_new = fmaxf(m_run[qg], mx);
            // a row that sees no key yet (all of this pass lies above it or outside its window) keeps m = -inf
            const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
            const float off = -m_use * scale2;
            float lsum = 0.f;
#pragma unroll
            for (int st = 0; st < BN / 16; ++st)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    s[st][i] = __builtin_amdgcn_exp2f(fmaf(s[st][i], scale2, off));      // 2^(-inf) = 0 for masked keys
                    lsum += s[st][i];
                }
            lsum = rows_sum(lsum);
            const float alpha = (m_run[qg] == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f((m_run[qg] - m_use) * scale2);
            l_run[qg] = l_run[qg] * alpha + lsum;
            if (__any(m_new != m_run[qg])) {             // some row's maximum moved: rescale what is summed so far
#pragma unroll
                for (int dt = 0; dt < D16; ++dt) {
                    acc[qg][dt][0] *= alpha;
                    acc[qg][dt][1] *= alpha;
                    acc[qg][dt][2] *= alpha;
                    acc[qg][dt][3] *= alpha;
                }
            }
            m_run[qg] = m_new;
#pragma unroll
            for (int b = 0; b < BN / 32; ++b)
                pw[qg][b] = uint4_t{pack2(s[2 * b][0], s[2 * b][1]), pack2(s[2 * b][2], s[2 * b][3]),
                                    pack2(s[2 * b + 1][0], s[2 * b + 1][1]), pack2(s[2 * b + 1][2], s[2 * b + 1][3])};
        }

        // ---- O^T += V^T P^T, 32 keys per MFMA; V^T through the transposing LDS read, once for every group
#pragma unroll
        for (int b = 0; b < BN / 32; ++b) {
            // this lane's address as lane l' = n of its group: key 32b + 4g + n/4, columns 4(n%4)..+3
            const uint16_t* vr = &v_cur[(32 * b + 4 * g + (n >> 2)) * VS + 4 * (n & 3)];
#pragma unroll
            for (int dt = 0; dt < D16; ++dt) {
                const short4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4_ptr)(vr + dt * 16));
                const short4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4_ptr)(vr + 16 * VS + dt * 16));
                const short8_t both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
#pragma unroll
                for (int qg = 0; qg < QG; ++qg)
                    acc[qg][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                        __builtin_bit_cast(bf16x8_t, both), __builtin_bit_cast(bf16x8_t, pw[qg][b]), acc[qg][dt], 0, 0, 0);
            }
        }
        }
        __syncthreads();                                 // every wave is done with this tile; the next one is complete
    }

#undef FETCH_ROW
#undef STAGE_TO
#undef ROW_OF
#undef K_S
#undef V_S
    MFMA_SETTLE();
    if constexpr (KSPLIT > 1) {
        // the second group hands over what it has summed: per lane m, l and the accumulators, lane fastest
        float* ms = reinterpret_cast<float*>(lds_raw) + (size_t)wave * QG * MERGE_SLOTS * 64 + lane;
        if (grp == 1) {
#pragma unroll
            for (int qg = 0; qg < QG; ++qg) {
                float* mq = ms + qg * MERGE_SLOTS * 64;
                mq[0] = m_run[qg];
                mq[64] = l_run[qg];
#pragma unroll
                for (int dt = 0; dt < D16; ++dt)
#pragma unroll
                    for (int i = 0; i < 4; ++i) mq[(2 + 4 * dt + i) * 64] = acc[qg][dt][i];
            }
        }
        __syncthreads();
        if (grp == 1) return;
#pragma unroll
        for (int qg = 0; qg < QG; ++qg) {
            const float* mq = ms + qg * MERGE_SLOTS * 64;
            const float m1 = mq[0], l1 = mq[64];
            const float m = fmaxf(m_run[qg], m1);        // (raw scores: the scale comes in with the exponent)
            const float a0 = (m_run[qg] == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f((m_run[qg] - m) * scale2);
            const float a1 = (m1 == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f((m1 - m) * scale2);
            l_run[qg] = l_run[qg] * a0 + l1 * a1;
#pragma unroll
            for (int dt = 0; dt < D16; ++dt)
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    acc[qg][dt][i] = acc[qg][dt][i] * a0 + mq[(2 + 4 * dt + i) * 64] * a1;
        }
    }
    // ---- acc[qg][dt][i] = O^T[d = 16dt + 4g + i][query n of group qg]
#pragma unroll
    for (int qg = 0; qg < QG; ++qg) {
        if (!q_ok[qg]) continue;
        const float inv = l_run[qg] > 0.f ? 1.0f / l_run[qg] : 0.f;
        bf16* op = out + ((size_t)(cu_q[seg] + pos_q[qg] - pos0) * Hq + head) * D;
#pragma unroll
        for (int dt = 0; dt < D16; ++dt) {
            uint2 w;
            w.x = pack2(acc[qg][dt][0] * inv, acc[qg][dt][1] * inv);
            w.y = pack2(acc[qg][dt][2] * inv, acc[qg][dt][3] * inv);
            *reinterpret_cast<uint2*>(op + dt * 16 + 4 * g) = w;
        }
    }
}

#define PRE_CAT2(a, b) a##b
#define PRE_CAT(a, b) PRE_CAT2(a, b)
// head sizes 16*(4*PRE_PART+1) .. 16*(4*PRE_PART+4)
extern "C" int PRE_CAT(ra_pre_part_, PRE_PART)(int D16, int tile_rows, int key_split, dim3 grid, hipStream_t st, const bf16* q, bf16* out,
                                              const bf16* kp, const bf16* vp, const int* pt,
                                              const int* cup, const int* kvs, const int* cuq,
                                              const int* qs, const int* tiles, int n_tiles, int Hq,
                                              int Hkv, int P, float scale, int window) {
#define PRE_LAUNCH(N, QG_, KS_)                                                                    \
    hipLaunchKernelGGL((attn_prefill_kernel<N, QG_, KS_>), grid, dim3(256 * KS_), 0, st, q, out, kp, vp, pt, \
                       cup, kvs, cuq, qs, tiles, n_tiles, Hq, Hkv, P, scale, window)
#define PRE_CASE(N)                                                                               \
    case N:                                                                                       \
        if (N <= PRE_WIDE_D16 && tile_rows == 128) {                                              \
            if (key_split == 2) PRE_LAUNCH(N, (N <= PRE_WIDE_D16 ? 2 : 1), (N <= PRE_WIDE_D16 ? 2 : 1)); \
            else PRE_LAUNCH(N, (N <= PRE_WIDE_D16 ? 2 : 1), 1);                                   \
        } else {                                                                                  \
            if (key_split == 2 && N <= PRE_WIDE_D16) PRE_LAUNCH(N, 1, (N <= PRE_WIDE_D16 ? 2 : 1)); \
            else PRE_LAUNCH(N, 1, 1);                                                             \
        }                                                                                         \
        return RA_OK;
    switch (D16) {
        PRE_CASE(4 * PRE_PART + 1) PRE_CASE(4 * PRE_PART + 2) PRE_CASE(4 * PRE_PART + 3)
        PRE_CASE(4 * PRE_PART + 4)
        default: return RA_ERR_ARG;
    }
#undef PRE_CASE
#undef PRE_LAUNCH
}
#endif  // PRE_PART

#ifdef PRE_API
#define PRE_PART_ARGS int D16, int tile_rows, int key_split, dim3 grid, hipStream_t st, const bf16* q, bf16* out, const bf16* kp,    \
    const bf16* vp, const int* pt, const int* cup, const int* kvs, const int* cuq, const int* qs,    \
    const int* tiles, int n_tiles, int Hq, int Hkv, int P, float scale, int window
extern "C" int ra_pre_part_0(PRE_PART_ARGS);
extern "C" int ra_pre_part_1(PRE_PART_ARGS);
extern "C" int ra_pre_part_2(PRE_PART_ARGS);
extern "C" int ra_pre_part_3(PRE_PART_ARGS);

// Rows of a q tile for head size D: 128 up to head size 128, 64 beyond. Up to head size 128 tiles of 64
// rows are taken too (one group of rows per wave: more LDS traffic per flop, twice the workgroups).
extern "C" int ra_attention_prefill_tile_rows(int D) { return D <= 16 * PRE_WIDE_D16 ? 128 : 64; }

// tiles: int32 [n_tiles][2] = (request number, first row of the tile within the request's new
// tokens); every request with more than one new token is covered in tiles of tile_rows rows,
// which must be what ra_attention_prefill_tile_rows(D) says.
extern "C" int ra_attention_prefill_bf16(const void* q, void* out, const void* k_pool,
                                         const void* v_pool, const int* page_table,
                                         const int* cu_pages, const int* kv_start, const int* cu_q,
                                         const int* q_start, const int* tiles, int n_tiles,
                                         int tile_rows, int key_split, int Hq, int Hkv, int D, int P,
                                         float scale, int window, void* stream) {
    if (n_tiles <= 0) return RA_OK;
    if (D % 16 != 0 || D < 16 || D > 256 || Hkv <= 0 || Hq % Hkv != 0 || P <= 0 ||
        (long long)n_tiles * Hq > 0x7fffffffLL || (tile_rows != ra_attention_prefill_tile_rows(D) && tile_rows != 64))
        return RA_ERR_ARG;
    hipStream_t st = (hipStream_t)stream;
    dim3 grid(n_tiles * Hq);
    const int d16 = D / 16;
    // key_split 2: a second group of waves takes every other key tile of each workgroup (head
    // sizes up to 128; it pays when the workgroups are few and the longest tile decides the time).
    // 0 decides here by the number of workgroups alone.
    if (key_split <= 0) key_split = (long long)n_tiles * Hq <= 256 ? 2 : 1;
    if (key_split > 2) return RA_ERR_ARG;
    int rc;
#define GO(k)                                                                                      \
    rc = ra_pre_part_##k(d16, tile_rows, key_split, grid, st, (const bf16*)q, (bf16*)out, (const bf16*)k_pool,           \
                         (const bf16*)v_pool, page_table, cu_pages, kv_start, cu_q, q_start, tiles, \
                         n_tiles, Hq, Hkv, P, scale, window)
    switch ((d16 - 1) / 4) {
        case 0: GO(0); break;
        case 1: GO(1); break;
        case 2: GO(2); break;
        case 3: GO(3); break;
        default: return RA_ERR_ARG;
    }
#undef GO
    if (rc != RA_OK) return rc;
    return ra_launch_status();
}
#endif  // PRE_API
