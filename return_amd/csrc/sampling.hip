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
// Among tokens that tie at a boundary the earlier ones in the vocabulary stay, as a stable sort
// puts them first: exactly top_k tokens are kept (rollout/model.py:45-50 keeps topk(k)), and of the
// tokens that tie with the top-p boundary value those before which at most top_p of the mass lies.
//
// top-k and top-p need a threshold among the largest logits. The row's tokens within CAND_SPAN of
// the largest logit (in units of the temperature: every other token weighs less than e^-16 of the
// largest) are first collected into a list in LDS, in vocabulary order; if they fit, and if the
// thresholds lie among them (k is at most their number; their mass is more than top_p of the whole),
// the thresholds are searched and the token is drawn from the list alone, which takes microseconds.
// Otherwise (a flat row, a large k, top_p near 1) the searches go over the whole row, pass by pass.
// Which way a row goes depends on that row alone.
#include "common.h"

#define SAMPLE_THREADS 1024
#define CAND_WAVES (SAMPLE_THREADS / 64)
#define CAND_PER_WAVE 512                                        // list entries of one wave's run of the row
#define CAND_OWN (CAND_WAVES * CAND_PER_WAVE / SAMPLE_THREADS)   // entries a thread looks after in a search: 8
#define CAND_SPAN 16.0f
#define SAMPLE_BLOCKS 64                                         // blocks of 256 tokens in a wave's run whose masses are kept

__device__ __forceinline__ uint32_t order_key(float f) {
    const uint32_t b = __float_as_uint(f);
    return (b & 0x80000000u) ? ~b : (b | 0x80000000u);      // ascending float order -> ascending uint
}

__device__ __forceinline__ float key_value(uint32_t k) {      // the float whose order_key is k
    return __uint_as_float((k & 0x80000000u) ? (k & 0x7fffffffu) : ~k);
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

// Measures are whole numbers: a token counts 2^40 (top-k), or weighs exp((x - gmax) / T) as a multiple of
// 2^-40 (top-p; what weighs less than 2^-41 of the largest token weighs nothing). Sums of whole numbers do
// not depend on the order in which they are formed, so they may be formed by atomics, by any number of
// threads, and come out the same in every run of the program.
typedef unsigned long long fixed_t;
#define FIXED_ONE_F 1099511627776.0f               // 2^40
__device__ __forceinline__ fixed_t to_fixed(float w) {          // 0 <= w <= 1
    const float t = w * 256.0f;
    const float hi = floorf(t);
    return ((fixed_t)(uint32_t)hi << 32) + (fixed_t)(uint32_t)((t - hi) * 4294967296.0f);
}

// Sum of whole numbers over the block; every thread gets it. wsum: CAND_WAVES words of LDS.
__device__ __forceinline__ fixed_t block_sum_fixed(fixed_t v, fixed_t* wsum) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) wsum[threadIdx.x >> 6] = v;
    __syncthreads();
    fixed_t t = 0ull;
    for (int w = 0; w < CAND_WAVES; ++w) t += wsum[w];
    __syncthreads();
    return t;
}

// The smallest key t in [lo, hi] with measure{key > t} <= limit, given measure{key > hi} = 0. visit(lo, hi, f)
// calls f(key, measure) for every token with lo < key <= hi that this thread looks after (all threads
// together: every such token once).
// A pass cuts (lo, hi] into up to SEARCH_BUCKETS runs of equal width, adds the tokens' measures into the
// runs (fx, LDS atomics) and finds the highest run b with more than `limit` at and above it: t lies in it.
// A range of 2^32 keys takes three passes. wsum: CAND_WAVES words, sh_b, sh_above: one word each, all LDS.
#define SEARCH_BITS 11
#define SEARCH_BUCKETS (1 << SEARCH_BITS)
// above (may be nullptr) is told measure{key > t}; at (may be nullptr) measure{key == t} where the last pass has
// it (its run of the key range was the one key t), else FIXED_UNKNOWN (t is the lo it was given, whose tokens no
// pass visits).
#define FIXED_UNKNOWN (~0ull)
template <typename Visit>
__device__ uint32_t search_threshold(Visit visit, int tid, uint32_t lo, uint32_t hi, fixed_t limit, fixed_t* fx,
                                     fixed_t* wsum, int* sh_b, fixed_t* sh_above, fixed_t* above = nullptr,
                                     fixed_t* at = nullptr) {
    fixed_t at_t = FIXED_UNKNOWN;
    static_assert(SEARCH_BUCKETS == 2 * SAMPLE_THREADS, "a thread looks after two runs");
    const int wave = tid >> 6, lane = tid & 63;
    fixed_t above_hi = 0ull;
    while (lo < hi) {
        const uint32_t width = hi - lo;
        const int bits = 32 - __builtin_clz(width);
        const int sh = bits > SEARCH_BITS ? bits - SEARCH_BITS : 0;       // (width >> sh) < SEARCH_BUCKETS
        fx[2 * tid] = 0ull;
        fx[2 * tid + 1] = 0ull;
        if (tid == 0) *sh_b = 0;
        __syncthreads();
        visit(lo, hi, [&](uint32_t key, fixed_t m) { atomicAdd(&fx[(key - lo) >> sh], m); });
        __syncthreads();
        // at_and_above(b) = the measure of runs b and higher; this thread has runs 2 tid and 2 tid + 1
        const fixed_t f0 = fx[2 * tid], f1 = fx[2 * tid + 1];
        fixed_t from_here = f0 + f1;                                      // then: over this and the higher threads
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) {
            const fixed_t t = __shfl_down(from_here, o, 64);
            if (lane + o < 64) from_here += t;
        }
        if (lane == 0) wsum[wave] = from_here;
        __syncthreads();
        for (int w = wave + 1; w < CAND_WAVES; ++w) from_here += wsum[w];
        const fixed_t s0 = from_here, s1 = from_here - f0;               // at_and_above(2 tid), (2 tid + 1)
        // the highest run with more than `limit` at and above it (run 0 if there is none)
        const int mine = above_hi + s1 > limit ? 2 * tid + 1 : (above_hi + s0 > limit ? 2 * tid : 0);
        if (mine > 0) atomicMax(sh_b, mine);
        __syncthreads();
        const int b = *sh_b;
        // what lies above run b: at_and_above(b + 1)
        if (b + 1 == 2 * tid) *sh_above = above_hi + s0;
        if (b + 1 == 2 * tid + 1) *sh_above = above_hi + s1;
        if (b + 1 == SEARCH_BUCKETS && tid == 0) *sh_above = above_hi;
        __syncthreads();
        above_hi = *sh_above;
        // run b ends at key lo + ((b + 1) << sh) - 1
        const unsigned long long end = (unsigned long long)lo + (((unsigned long long)b + 1ull) << sh) - 1ull;
        const uint32_t new_hi = end < (unsigned long long)hi ? (uint32_t)end : hi;
        lo = b == 0 ? lo : lo + ((uint32_t)b << sh);
        hi = new_hi;
        if (lo == hi && b > 0) at_t = fx[b];           // the run was that one key: what was added into it is the key's
        __syncthreads();
    }
    if (above) *above = above_hi;
    if (at) *at = at_t;
    return lo;
}

// Of the tokens that tie at a boundary, the first `stay` in vocabulary order stay: returns the index of the
// last of them (`upto` if all of them stay). count_ties(f) calls f(index) for every tying token of this thread
// with index <= upto. One pass counts them; only if they are more than may stay, the index is searched.
// (A function of its own, not inlined: it runs four times in the kernel, and inlined the kernel no longer
// fits the 128 registers that a block of 1,024 threads leaves a lane.)
// known: their number if the search has it already (then nothing is counted), else FIXED_UNKNOWN.
template <typename Ties>
__device__ __noinline__ int tie_cut(Ties ties, int tid, int V, unsigned long long stay, int upto, fixed_t known,
                       fixed_t* fx, fixed_t* wsum, int* sh_b, fixed_t* sh_above) {
    fixed_t n = known;
    if (known == FIXED_UNKNOWN) {
        fixed_t mine = 0ull;
        ties([&](int) { mine += 1ull; });
        n = block_sum_fixed(mine, wsum);
    }
    if (stay >= n) return upto;
    if (stay == 0ull) return -1;
    // the stay-th tie from the front: the smallest t with at most stay - 1 ties at keys V - 1 - index above it
    const uint32_t t = search_threshold(
        [&](uint32_t lo, uint32_t hi, auto add) {
            ties([&](int i) {
                const uint32_t key = (uint32_t)(V - 1 - i);
                if (key > lo && key <= hi) add(key, 1ull << 40);
            });
        },
        tid, 0u, (uint32_t)(V - 1), (fixed_t)(stay - 1ull) << 40, fx, wsum, sh_b, sh_above);
    return V - 1 - (int)t;
}

// The draw's first step: wmass[w] is the kept mass of wave w's run of tokens (runs in vocabulary order).
// Gives the wave in whose run the running sum passes u times the total (the last run with kept mass if it
// never does), the sum before that run and the target. Every thread computes the same.
__device__ __forceinline__ void pick_wave(const float* wmass, float u, int& owner, float& before, float& target) {
    float total = 0.f;
    for (int w = 0; w < CAND_WAVES; ++w) total += wmass[w];
    target = u * total;
    float run = 0.f;
    owner = -1;
    before = 0.f;
    for (int w = 0; w < CAND_WAVES; ++w) {
        if (wmass[w] > 0.f) {
            owner = w;
            before = run;
            if (run + wmass[w] > target) break;
            run += wmass[w];
        }
    }
}

// Running sums over the lanes of a wave, lane by lane in lane order (inclusive).
__device__ __forceinline__ float wave_running_sum(float v, int lane) {
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
        const float t = __shfl_up(v, o, 64);
        if (lane >= o) v += t;
    }
    return v;
}

__global__ __launch_bounds__(SAMPLE_THREADS) void sample_kernel(
    const float* __restrict__ logits, int V, const float* __restrict__ temperature,
    const int* __restrict__ top_k, const float* __restrict__ top_p, const float* __restrict__ u,
    int* __restrict__ out, int* __restrict__ path) {
    extern __shared__ __attribute__((aligned(16))) float dyn[];           // the list (64 KB), then the search's runs (16 KB)
    __shared__ float scratch[16];
    __shared__ float wmass[CAND_WAVES];
    __shared__ fixed_t wsum[CAND_WAVES];
    __shared__ fixed_t sh_above;
    __shared__ int sh_b;
    fixed_t* fx = reinterpret_cast<fixed_t*>(dyn + 2 * CAND_WAVES * CAND_PER_WAVE);
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
    // a row with no value above -inf (all -inf, or NaN after an overflow upstream) never set an index:
    // token 0 then, so that nothing below reads beyond the row
    if ((unsigned)argmax >= (unsigned)V) argmax = 0;
    float total_e = 0.f;
    for (int w = 0; w < SAMPLE_THREADS / 64; ++w)
        total_e += (wm[w] == -INFINITY) ? 0.f : ws[w] * __expf(wm[w] - gmax);
    const float lse = gmax + logf(total_e);

    const float temp = temperature[row];
    if (!(temp > 0.f)) {
        if (tid == 0) {
            out[2 * row] = argmax;
            out[2 * row + 1] = __float_as_int(x[argmax] - lse);
            if (path) path[row] = 0;
        }
        return;
    }
    const float inv_t = 1.0f / temp;
    const uint32_t top_key = order_key(gmax);

    // Wave w's run of the row (a multiple of 256 tokens): a lane reads four consecutive tokens of every 256,
    // so that what a wave meets, load by load, lane by lane, is in vocabulary order.
    const int wave = tid >> 6, lane = tid & 63;
    const int seg = ((V + CAND_WAVES - 1) / CAND_WAVES + 255) / 256 * 256;
    const int beg = min(V, wave * seg), end = min(V, beg + seg);
    const bool vec = (V & 3) == 0 && (reinterpret_cast<uintptr_t>(x) & 15) == 0;
    auto load4 = [&](int i, float (&a)[4]) {           // tokens i .. i+3 of the run, -inf beyond its end
        if (vec) {
            if (i < end) {
                const float4 t = *reinterpret_cast<const float4*>(x + i);
                a[0] = t.x; a[1] = t.y; a[2] = t.z; a[3] = t.w;
            } else {
                a[0] = a[1] = a[2] = a[3] = -INFINITY;
            }
        } else {
#pragma unroll
            for (int c = 0; c < 4; ++c) a[c] = i + c < end ? x[i + c] : -INFINITY;
        }
    };

    const int k = top_k[row];
    const float p = top_p[row];
    const bool want_k = k > 0 && k < V, want_p = p < 1.0f;
    // what stays: tokens whose key is above keep_key, and of those whose key is keep_key the ones up to tie_limit
    uint32_t keep_key = 0u;
    int tie_limit = 0x7fffffff;
    auto kept = [&](uint32_t key, int i) { return key > keep_key || (key == keep_key && i <= tie_limit); };

    if (want_k || want_p) {
        // ---- the list: wave w goes through its run of the row, 64 tokens a load, and appends the tokens
        // within CAND_SPAN of the largest to its part of the list, in their order
        float* cv = dyn;                                                   // [CAND_WAVES][CAND_PER_WAVE] logits
        int* ci = reinterpret_cast<int*>(dyn + CAND_WAVES * CAND_PER_WAVE);    // and their token numbers
        __shared__ int cnt[CAND_WAVES];
        __shared__ int sh_over;
        const float cut = gmax - CAND_SPAN * temp;
        const uint32_t cut_key = order_key(cut);
        const bool sum_rest = want_p && !want_k;       // top-p alone is over the mass of the whole row
        if (tid == 0) sh_over = 0;
        __syncthreads();
        {
            int have = 0;
            float rest = 0.f;
            const unsigned long long below = (1ull << lane) - 1ull;        // the lanes before this one
            for (int i0 = beg + 4 * lane; i0 - 4 * lane < end; i0 += 4 * 256) {      // four loads on their way
                if (have > CAND_PER_WAVE) break;          // (a flat row: this run alone is too much for the list)
                float v[4][4];
#pragma unroll
                for (int j = 0; j < 4; ++j) load4(i0 + 256 * j, v[j]);
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    int before = 0, all = 0;
                    bool in[4];
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        in[c] = v[j][c] >= cut;
                        const unsigned long long m = __ballot(in[c]);
                        before += __popcll(m & below);
                        all += __popcll(m);
                    }
                    if (all != 0) {
                        int at = have + before;
#pragma unroll
                        for (int c = 0; c < 4; ++c) {
                            if (in[c]) {
                                if (at < CAND_PER_WAVE) {
                                    cv[wave * CAND_PER_WAVE + at] = v[j][c];
                                    ci[wave * CAND_PER_WAVE + at] = i0 + 256 * j + c;
                                }
                                ++at;
                            }
                        }
                        have += all;
                    }
                    if (sum_rest) {
#pragma unroll
                        for (int c = 0; c < 4; ++c) rest += in[c] ? 0.f : __expf((v[j][c] - gmax) * inv_t);
                    }
                }
            }
            if (lane == 0) {
                cnt[wave] = min(have, CAND_PER_WAVE);
                if (have > CAND_PER_WAVE) sh_over = 1;
            }
            const float z_rest = sum_rest ? block_sum(rest, scratch) : 0.f;     // (with barriers of its own, or:)
            __syncthreads();
            int total = 0;
            for (int w = 0; w < CAND_WAVES; ++w) total += cnt[w];
            bool listed = sh_over == 0 && cut_key > 0u && (!want_k || k <= total);

            // a thread's entries for the searches: place (tid % CAND_PER_WAVE) of every other wave's part
            if (listed) {
                uint32_t key[CAND_OWN];
                float weight[CAND_OWN];                    // exp((x - max) / T), made a whole number where it is added
                int idx[CAND_OWN];                         // the entry's token; -1: no entry
                const int half = tid / CAND_PER_WAVE, off = tid - half * CAND_PER_WAVE;
#pragma unroll
                for (int e = 0; e < CAND_OWN; ++e) {
                    const int w = half + (SAMPLE_THREADS / CAND_PER_WAVE) * e;
                    const bool there = off < cnt[w];
                    const float v = there ? cv[w * CAND_PER_WAVE + off] : 0.f;
                    key[e] = there ? order_key(v) : 0u;
                    weight[e] = there ? __expf((v - gmax) * inv_t) : 0.f;
                    idx[e] = there ? ci[w * CAND_PER_WAVE + off] : -1;
                }
                // the entries that tie at key t, up to token `upto`
                auto ties_at = [&](uint32_t t, int upto) {
                    return [&key, &idx, t, upto](auto f) {
#pragma unroll
                        for (int e = 0; e < CAND_OWN; ++e)
                            if (idx[e] >= 0 && key[e] == t && idx[e] <= upto) f(idx[e]);
                    };
                };
                // top-k: the k-th largest is on the list; below cut_key - 1 nothing of it lies
                if (want_k) {
                    fixed_t above = 0ull, at = FIXED_UNKNOWN;
                    keep_key = search_threshold(
                        [&](uint32_t lo, uint32_t hi, auto add) {
#pragma unroll
                            for (int e = 0; e < CAND_OWN; ++e)
                                if (key[e] > lo && key[e] <= hi) add(key[e], 1ull << 40);
                        },
                        tid, cut_key - 1u, top_key, (fixed_t)(k - 1) << 40, fx, wsum, &sh_b, &sh_above, &above, &at);
                    // of the tokens that tie with the k-th value, as many stay as make k with those above them
                    tie_limit = tie_cut(ties_at(keep_key, 0x7fffffff), tid, V, (unsigned long long)k - (above >> 40),
                                        0x7fffffff, at == FIXED_UNKNOWN ? at : at >> 40, fx, wsum, &sh_b, &sh_above);
                }
                if (want_p) {
                    fixed_t zc = 0ull;
#pragma unroll
                    for (int e = 0; e < CAND_OWN; ++e) zc += idx[e] >= 0 && kept(key[e], idx[e]) ? to_fixed(weight[e]) : 0ull;
                    zc = block_sum_fixed(zc, wsum);
                    const fixed_t z = zc + (fixed_t)((double)z_rest * (double)FIXED_ONE_F);
                    const fixed_t limit = (fixed_t)((double)p * (double)z);
                    // the boundary is on the list if the list's mass is more than p of the whole (always, after top-k)
                    if (want_k || zc > limit) {
                        const uint32_t k_key = keep_key;     // what top-k left: the search goes over that
                        const int k_limit = tie_limit;
                        fixed_t above = 0ull, at = FIXED_UNKNOWN;
                        keep_key = search_threshold(
                            [&](uint32_t lo, uint32_t hi, auto add) {
#pragma unroll
                                for (int e = 0; e < CAND_OWN; ++e)
                                    if (idx[e] >= 0 && key[e] > lo && key[e] <= hi &&
                                        (key[e] > k_key || idx[e] <= k_limit)) add(key[e], to_fixed(weight[e]));
                            },
                            tid, want_k ? k_key : cut_key - 1u, top_key, limit, fx, wsum, &sh_b, &sh_above, &above, &at);
                        // of the tokens that tie with the boundary value, the i-th in vocabulary order stays while
                        // what lies before it, the mass above them and i of their own, is at most top_p of the whole
                        const fixed_t each = to_fixed(__expf((key_value(keep_key) - gmax) * inv_t));
                        const unsigned long long stay = each ? (limit - above) / each + 1ull : ~0ull;
                        const int upto = keep_key == k_key ? k_limit : 0x7fffffff;
                        // (a boundary above top-k's: every token of that value was in the search, their mass is their number)
                        const fixed_t known = (at != FIXED_UNKNOWN && each && (!want_k || keep_key != k_key)) ? at / each : FIXED_UNKNOWN;
                        tie_limit = tie_cut(ties_at(keep_key, upto), tid, V, stay, upto, known, fx, wsum, &sh_b, &sh_above);
                    } else {
                        listed = false;
                    }
                }
            }
            if (listed) {
                // ---- the draw over the list, which is in vocabulary order: wave w has its own part,
                // a lane CAND_PER_WAVE / 64 consecutive entries of it
                constexpr int RUN = CAND_PER_WAVE / 64;
                const int o0 = min(cnt[wave], RUN * lane), o1 = min(cnt[wave], o0 + RUN);
                float mine = 0.f;
                for (int o = o0; o < o1; ++o) {
                    const float v = cv[wave * CAND_PER_WAVE + o];
                    if (kept(order_key(v), ci[wave * CAND_PER_WAVE + o])) mine += __expf((v - gmax) * inv_t);
                }
                const float upto = wave_running_sum(mine, lane);
                __syncthreads();
                if (lane == 63) wmass[wave] = upto;
                __syncthreads();
                int owner;
                float before, target;
                pick_wave(wmass, u[row], owner, before, target);
                if (owner < 0) {                       // (nothing is kept: cannot be, the largest always is)
                    if (tid == 0) {
                        out[2 * row] = argmax;
                        out[2 * row + 1] = __float_as_int(x[argmax] - lse);
                        if (path) path[row] = 1;
                    }
                    return;
                }
                if (wave != owner) return;
                // the lane in whose entries the running sum passes the target, else the last one with kept mass
                const unsigned long long passed = __ballot(mine > 0.f && before + upto > target);
                const unsigned long long any = __ballot(mine > 0.f);
                const int who = passed ? __ffsll((long long)passed) - 1 : 63 - __builtin_clzll(any);
                if (lane == who) {
                    float run = before + (upto - mine);
                    int tok = argmax;
                    for (int o = o0; o < o1; ++o) {
                        const float v = cv[wave * CAND_PER_WAVE + o];
                        if (kept(order_key(v), ci[wave * CAND_PER_WAVE + o])) {
                            tok = ci[wave * CAND_PER_WAVE + o];      // the last kept entry if the target is never passed
                            run += __expf((v - gmax) * inv_t);
                            if (run > target) break;
                        }
                    }
                    out[2 * row] = tok;
                    out[2 * row + 1] = __float_as_int(x[tok] - lse);
                    if (path) path[row] = 1;
                }
                return;
            }
        }
        __syncthreads();
        keep_key = 0u;
        tie_limit = 0x7fffffff;
        // the row's tokens that tie at key t, up to token `upto`
        auto ties_at = [&](uint32_t t, int upto) {
            return [x, V, tid, t, upto](auto f) {
                for_each_logit(x, V, tid, [&](int i, float v) {
                    if (order_key(v) == t && i <= upto) f(i);
                });
            };
        };

        // ---- over the whole row. top-k: the key of the k-th largest value is the smallest key with at most
        // k - 1 tokens above it
        if (want_k) {
            fixed_t above = 0ull, at = FIXED_UNKNOWN;
            keep_key = search_threshold(
                [&](uint32_t lo, uint32_t hi, auto add) {
                    for_each_logit(x, V, tid, [&](int, float v) {
                        const uint32_t key = order_key(v);
                        if (key > lo && key <= hi) add(key, 1ull << 40);
                    });
                },
                tid, 0u, top_key, (fixed_t)(k - 1) << 40, fx, wsum, &sh_b, &sh_above, &above, &at);
            tie_limit = tie_cut(ties_at(keep_key, 0x7fffffff), tid, V, (unsigned long long)k - (above >> 40),
                                0x7fffffff, at == FIXED_UNKNOWN ? at : at >> 40, fx, wsum, &sh_b, &sh_above);
        }
        // top-p: the smallest key with at most p of the kept mass above it
        if (want_p) {
            fixed_t z = 0ull;
            for_each_logit(x, V, tid, [&](int i, float v) {
                if (kept(order_key(v), i)) z += to_fixed(__expf((v - gmax) * inv_t));
            });
            z = block_sum_fixed(z, wsum);
            const fixed_t limit = (fixed_t)((double)p * (double)z);
            const uint32_t k_key = keep_key;             // what top-k left: the search goes over that
            const int k_limit = tie_limit;
            fixed_t above = 0ull, at = FIXED_UNKNOWN;
            keep_key = search_threshold(
                [&](uint32_t lo, uint32_t hi, auto add) {
                    for_each_logit(x, V, tid, [&](int i, float v) {
                        const uint32_t key = order_key(v);
                        if (key > lo && key <= hi && (key > k_key || i <= k_limit))
                            add(key, to_fixed(__expf((v - gmax) * inv_t)));
                    });
                },
                tid, k_key, top_key, limit, fx, wsum, &sh_b, &sh_above, &above, &at);
            const fixed_t each = to_fixed(__expf((key_value(keep_key) - gmax) * inv_t));
            const unsigned long long stay = each ? (limit - above) / each + 1ull : ~0ull;
            const int upto = keep_key == k_key ? k_limit : 0x7fffffff;
            const fixed_t known = (at != FIXED_UNKNOWN && each && (!want_k || keep_key != k_key)) ? at / each : FIXED_UNKNOWN;
            tie_limit = tie_cut(ties_at(keep_key, upto), tid, V, stay, upto, known, fx, wsum, &sh_b, &sh_above);
        }
    }

    // ---- the draw over the whole row, in vocabulary order. Wave w has a run of the row (a multiple of 256
    // tokens); a lane reads four consecutive tokens of every 256. First the kept mass of every block of 256
    // tokens, and with them every wave's; then the wave in whose run the running sum passes the target finds
    // the block in which it does, and goes through that block again, token by token.
    {
        auto kept_mass = [&](int i, float v) {             // (a token beyond the run's end has none: exp(-inf))
            return (i < end && kept(order_key(v), i)) ? __expf((v - gmax) * inv_t) : 0.f;
        };
        __shared__ float bmass[CAND_WAVES][SAMPLE_BLOCKS];
        const int n_it = (end - beg + 255) / 256;            // this wave's blocks
        const bool by_block = seg / 256 <= SAMPLE_BLOCKS;    // (a vocabulary beyond 262,144: the whole run is gone through again)
        float mine = 0.f;
        for (int it0 = 0; it0 < n_it; it0 += 4) {            // four loads on their way
            float a[4][4];
#pragma unroll
            for (int j = 0; j < 4; ++j) load4(beg + 256 * (it0 + j) + 4 * lane, a[j]);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int i = beg + 256 * (it0 + j) + 4 * lane;
                float m = 0.f;
#pragma unroll
                for (int c = 0; c < 4; ++c) m += kept_mass(i + c, a[j][c]);
                m = wave_sum(m);
                if (by_block && lane == 0 && it0 + j < n_it) bmass[wave][it0 + j] = m;
                mine += m;
            }
        }
        __syncthreads();
        if (lane == 0) wmass[wave] = mine;
        __syncthreads();
        int owner;
        float before, target;
        pick_wave(wmass, u[row], owner, before, target);
        if (owner < 0) owner = 0;
        if (wave != owner) return;
        float run = before;
        int it_lo = 0, it_hi = n_it;
        if (by_block) {                                      // the block, as pick_wave finds the wave
            int ob = -1;
            float r2 = before;
            for (int it = 0; it < n_it; ++it) {
                const float bm = bmass[wave][it];
                if (bm > 0.f) {
                    ob = it;
                    run = r2;
                    if (r2 + bm > target) break;
                    r2 += bm;
                }
            }
            it_lo = max(ob, 0);
            it_hi = ob < 0 ? 0 : ob + 1;
        }
        int last_kept = -1, tok = -1;
        constexpr int AHEAD = 4;                             // loads on their way
        float a[AHEAD][4];
#pragma unroll
        for (int j = 0; j < AHEAD; ++j) load4(beg + 256 * (it_lo + j) + 4 * lane, a[j]);
        for (int it0 = it_lo; it0 < it_hi && tok < 0; it0 += AHEAD) {
#pragma unroll
            for (int j = 0; j < AHEAD; ++j) {
                const int i = it0 + j < it_hi ? beg + 256 * (it0 + j) + 4 * lane : end;      // (beyond the blocks asked for: nothing)
                float m[4], s[4];
#pragma unroll
                for (int c = 0; c < 4; ++c) m[c] = kept_mass(i + c, a[j][c]);
                s[0] = m[0]; s[1] = s[0] + m[1]; s[2] = s[1] + m[2]; s[3] = s[2] + m[3];
                const float upto = wave_running_sum(s[3], lane);
                const float base = run + (upto - s[3]);
                int first = -1;
#pragma unroll
                for (int c = 3; c >= 0; --c) {
                    const bool is_kept = i + c < end && kept(order_key(a[j][c]), i + c);
                    if (is_kept && base + s[c] > target) first = c;
                    if (is_kept) last_kept = max(last_kept, i + c);
                }
                const unsigned long long passed = __ballot(first >= 0);
                if (passed && tok < 0) {
                    const int who = __ffsll((long long)passed) - 1;
                    tok = __shfl(i + max(first, 0), who, 64);
                }
                run += __shfl(upto, 63, 64);
                load4(beg + 256 * (it0 + j + AHEAD) + 4 * lane, a[j]);                 // (beyond the run's end: -inf)
            }
        }
        if (tok < 0) {                                       // never passed: the last kept token of the run
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) last_kept = max(last_kept, __shfl_xor(last_kept, o, 64));
            tok = last_kept < 0 ? argmax : last_kept;
        }
        if (lane == 0) {
            out[2 * row] = tok;
            out[2 * row + 1] = __float_as_int(x[tok] - lse);
            if (path) path[row] = (want_k || want_p) ? 2 : 0;
        }
    }
}

// path (may be nullptr): per row 0 = no threshold was needed, 1 = thresholds and draw from the list of the
// largest logits, 2 = by passes over the whole row.
extern "C" int ra_sample_traced(const float* logits, int M, int V, const float* temperature,
                                const int* top_k, const float* top_p, const float* u, int* out, int* path,
                                void* stream) {
    if (M <= 0) return RA_OK;
    if (V <= 0) return RA_ERR_ARG;
    const size_t lds = (size_t)2 * CAND_WAVES * CAND_PER_WAVE * sizeof(float) + SEARCH_BUCKETS * sizeof(fixed_t);   // 80 KB
    static bool allowed = false;
    if (!allowed) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(sample_kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                (int)lds) != hipSuccess)
            return RA_ERR_ARG;
        allowed = true;
    }
    hipLaunchKernelGGL(sample_kernel, dim3(M), dim3(SAMPLE_THREADS), lds, (hipStream_t)stream, logits,
                       V, temperature, top_k, top_p, u, out, path);
    return ra_launch_status();
}

extern "C" int ra_sample(const float* logits, int M, int V, const float* temperature,
                         const int* top_k, const float* top_p, const float* u, int* out,
                         void* stream) {
    return ra_sample_traced(logits, M, V, temperature, top_k, top_p, u, out, nullptr, stream);
}
