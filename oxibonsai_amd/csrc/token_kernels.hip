// token_kernels.hip — token embedding lookup, top-k / top-p sampling and token bookkeeping of the on-device
// generation loop.
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>
#include <cstring>
#include <rocprim/device/device_radix_sort.hpp>

#include "device_utils.h"
#include "token_kernels.h"

// ---------------------------------------------------------------------------
// Token embedding lookup (the row copy that precedes the forward, crates/oxibonsai-model/src/model/types/mod.rs:647-658)
// from the table in its stored form; values as load_f32_tensor widens / dequantises them
// (crates/oxibonsai-model/src/model/weight_loaders.rs:24-86): F16 -> f32 exactly; Q1_0_g128 bit ? d : -d;
// TQ2_0_g128 codes 00 -> -d, 01 -> 0, 10 -> +d, 11 -> 0.  Grid = rows, 256 threads.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void embedding_gather_kernel(const uint8_t* __restrict__ table, int type, uint32_t vocab,
                                                                uint32_t h, const uint32_t* __restrict__ ids,
                                                                float* __restrict__ out) {
    const uint32_t row = blockIdx.x, id = ids[row];
    float* o = out + (size_t)row * h;
    if (id >= vocab) {
        for (uint32_t i = threadIdx.x; i < h; i += 256) o[i] = __int_as_float(0x7FC00000);
        return;
    }
    if (type == 0) {
        const float* src = reinterpret_cast<const float*>(table) + (size_t)id * h;
        for (uint32_t i = threadIdx.x; i < h; i += 256) o[i] = src[i];
    } else if (type == 1) {
        const __half* src = reinterpret_cast<const __half*>(table) + (size_t)id * h;
        for (uint32_t i = threadIdx.x; i < h; i += 256) o[i] = __half2float(src[i]);
    } else {
        const uint32_t bb = type == 41 ? 18u : 34u;
        const uint8_t* src = table + (size_t)id * (h / 128u) * bb;
        for (uint32_t i = threadIdx.x; i < h; i += 256) {
            const uint8_t* blk = src + (size_t)(i >> 7) * bb;
            const uint32_t j = i & 127u;
            float v;
            if (type == 41) {  // [d f16][qs 16]
                const float d = __half2float(__ushort_as_half((unsigned short)(blk[0] | (blk[1] << 8))));
                v = ((blk[2 + (j >> 3)] >> (j & 7u)) & 1u) ? d : -d;
            } else {           // [qs 32][d f16]
                const float d = __half2float(__ushort_as_half((unsigned short)(blk[32] | (blk[33] << 8))));
                const uint32_t code = (blk[j >> 2] >> (2u * (j & 3u))) & 3u;
                v = code == 0u ? -d : (code == 2u ? d : 0.0f);
            }
            o[i] = v;
        }
    }
}

__global__ void token_step_kernel(const uint32_t* __restrict__ tokens, uint32_t* __restrict__ history,
                                  uint32_t* __restrict__ pos, uint32_t batch) {
    const uint32_t b = blockIdx.x * blockDim.x + threadIdx.x;
    if (b < batch) {
        history[b] = tokens[b];
        pos[b] += 1u;
    }
}

// ---------------------------------------------------------------------------
// Sampling (Sampler::sample, crates/oxibonsai-runtime/src/sampling.rs:84-177).
// Stage 1, grid (parts, rows): a workgroup keeps its span of the logits in registers (EPT per thread, each thread's
// sorted descending).  Every wave pops the maximum of its 512 values top_k times with lane exchanges only (no
// barrier in the loop); the four sorted lists meet in LDS and wave 0 merges them the same way: the span's top_k
// in descending order, ties to the lower index.  Stage 2, one wave per row: a lane walks up to four of the parts'
// sorted lists (the next element of each already requested) and the same pop yields the row's top_k in descending
// order; lane 0 then walks the reference's arithmetic over those <= 128 values: v / temperature, exp(v - max) (formed by all lanes),
// sum, divide, top-p cut, renormalise, r = (xorshift64 / u64::MAX) as f32, cumulative pick (first candidate if
// none reaches r).  The reference leaves the candidates in whatever order its partial selection produces when
// top_p == 1; here the order is always descending.
// ---------------------------------------------------------------------------
#define OXB_TOPK_EPT 8
#define OXB_TOPK_SPAN (256 * OXB_TOPK_EPT)

// A candidate as one 64-bit key, larger = taken first: the logit's bits made monotone (sign flipped / inverted) above
// the inverted index, so values descend and equal values go by the lower index, as Sampler::sample's sort leaves
// them; 0 = empty.  -0 counts as +0 and a NaN ranks with -infinity.
__device__ __forceinline__ uint64_t cand_key(float v, uint32_t i) {
    uint32_t b = __float_as_uint(v);
    if (b == 0x80000000u) b = 0u;
    if ((b & 0x7FFFFFFFu) > 0x7F800000u) b = 0xFF800000u;
    const uint32_t u = (b & 0x80000000u) ? ~b : (b | 0x80000000u);
    return ((uint64_t)u << 32) | (uint64_t)(0xFFFFFFFFu - i);
}
__device__ __forceinline__ float key_value(uint64_t k) {
    const uint32_t u = (uint32_t)(k >> 32);
    return __uint_as_float((u & 0x80000000u) ? (u & 0x7FFFFFFFu) : ~u);
}
__device__ __forceinline__ uint32_t key_index(uint64_t k) { return 0xFFFFFFFFu - (uint32_t)k; }

// Largest key of the wave's 64 lanes, the same value in every lane: four DPP steps inside each row of 16 lanes, then
// the four row results through scalar registers - no LDS, no long-latency lane exchange.
__device__ __forceinline__ uint64_t wave_max_key(uint64_t k) {
    uint32_t hi = (uint32_t)(k >> 32), lo = (uint32_t)k;
#define OXB_KEY_STEP(N)                                                                  \
    {                                                                                    \
        const uint32_t h2 = dpp_u32<OXB_DPP_ROW_SHR(N)>(hi), l2 = dpp_u32<OXB_DPP_ROW_SHR(N)>(lo); \
        const bool take = h2 > hi || (h2 == hi && l2 > lo);                              \
        hi = take ? h2 : hi;                                                             \
        lo = take ? l2 : lo;                                                             \
    }
    OXB_KEY_STEP(1) OXB_KEY_STEP(2) OXB_KEY_STEP(4) OXB_KEY_STEP(8)
#undef OXB_KEY_STEP
    uint64_t best = 0;
#pragma unroll
    for (int r = 0; r < 4; r++) {  // lane 16 r + 15 holds its row's maximum
        const uint64_t c = ((uint64_t)(uint32_t)__builtin_amdgcn_readlane((int)hi, 16 * r + 15) << 32) |
                           (uint32_t)__builtin_amdgcn_readlane((int)lo, 16 * r + 15);
        best = c > best ? c : best;
    }
    return best;
}

__global__ __launch_bounds__(256) void topk_partial_kernel(const float* __restrict__ logits, uint32_t n, uint32_t top_k,
                                                            float* __restrict__ cv, uint32_t* __restrict__ ci) {
    __shared__ uint64_t lists[4][OXB_SAMPLE_MAX_TOP_K];
    const float* v = logits + (size_t)blockIdx.y * n;
    const uint32_t i0 = blockIdx.x * OXB_TOPK_SPAN, lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    uint64_t mine[OXB_TOPK_EPT];
#pragma unroll
    for (int e = 0; e < OXB_TOPK_EPT; e++) {
        const uint32_t i = i0 + threadIdx.x + 256u * e;
        mine[e] = i < n ? cand_key(v[i], i) : 0ull;
    }
    // sort the thread's own keys, largest first
#pragma unroll
    for (int a = 1; a < OXB_TOPK_EPT; a++)
#pragma unroll
        for (int b = a; b > 0; b--)
            if (mine[b] > mine[b - 1]) {
                const uint64_t t = mine[b];
                mine[b] = mine[b - 1];
                mine[b - 1] = t;
            }
    for (uint32_t j = 0; j < top_k; j++) {  // the wave's own top_k
        const uint64_t best = wave_max_key(mine[0]);
        if (best != 0 && mine[0] == best) {  // keys are unique: this lane offered it; pop by shifting the lane's list
#pragma unroll
            for (int e = 0; e + 1 < OXB_TOPK_EPT; e++) mine[e] = mine[e + 1];
            mine[OXB_TOPK_EPT - 1] = 0ull;
        }
        if (lane == 0) lists[wave][j] = best;
    }
    __syncthreads();
    if (wave != 0) return;
    // merge: lane w < 4 walks wave w's list
    const size_t out = ((size_t)blockIdx.y * gridDim.x + blockIdx.x) * top_k;
    uint32_t head = 0;
    for (uint32_t j = 0; j < top_k; j++) {
        const uint64_t c = (lane < 4 && head < top_k) ? lists[lane][head] : 0ull;
        const uint64_t best = wave_max_key(c);
        if (best != 0 && c == best) head++;
        if (lane == 0) cv[out + j] = key_value(best), ci[out + j] = best ? key_index(best) : 0xFFFFFFFFu;
    }
}

#define OXB_SAMPLE_LISTS_PER_LANE 4  // stage 2 walks up to 256 parts with one wave
#define OXB_SAMPLE_LDS_KEYS 6144     // the parts' lists are walked out of LDS when they fit (48 KB of keys)
template <bool IN_LDS>
__global__ __launch_bounds__(64) void sample_final_kernel(const float* __restrict__ cv, const uint32_t* __restrict__ ci,
                                                           uint32_t parts, uint32_t top_k, float temperature, float top_p,
                                                           uint64_t* __restrict__ rng, uint32_t* __restrict__ tokens) {
    __shared__ float pv[OXB_SAMPLE_MAX_TOP_K];
    __shared__ uint32_t pi[OXB_SAMPLE_MAX_TOP_K];
    __shared__ uint64_t keys[IN_LDS ? OXB_SAMPLE_LDS_KEYS : 1];
    const uint32_t row = blockIdx.x, lane = threadIdx.x;
    const float* lv = cv + (size_t)row * parts * top_k;
    const uint32_t* li = ci + (size_t)row * parts * top_k;
    if (IN_LDS) {  // one pass over the lists with every load in flight, instead of a trip to memory per pop
        const uint32_t total = parts * top_k;
        for (uint32_t e0 = 0; e0 < total; e0 += 64 * 16) {  // sixteen loads of each array in flight per lane
            uint32_t i[16];
            float v[16];
#pragma unroll
            for (int u = 0; u < 16; u++) {
                const uint32_t e = e0 + 64u * u + lane;
                i[u] = e < total ? li[e] : 0xFFFFFFFFu;
                v[u] = e < total ? lv[e] : 0.0f;
            }
#pragma unroll
            for (int u = 0; u < 16; u++) {
                const uint32_t e = e0 + 64u * u + lane;
                if (e < total) keys[e] = i[u] == 0xFFFFFFFFu ? 0ull : cand_key(v[u], i[u]);
            }
        }
        __syncthreads();
    }
    // lane t walks the sorted lists of parts t, t + 64, ...: `cur` is each list's head, `nxt` the element behind it
    uint64_t cur[OXB_SAMPLE_LISTS_PER_LANE], nxt[OXB_SAMPLE_LISTS_PER_LANE];
    uint32_t head[OXB_SAMPLE_LISTS_PER_LANE];
    auto fetch = [&](uint32_t part, uint32_t at) -> uint64_t {
        if (part >= parts || at >= top_k) return 0ull;
        if (IN_LDS) return keys[part * top_k + at];
        const uint32_t i = li[(size_t)part * top_k + at];
        return i == 0xFFFFFFFFu ? 0ull : cand_key(lv[(size_t)part * top_k + at], i);
    };
#pragma unroll
    for (int q = 0; q < OXB_SAMPLE_LISTS_PER_LANE; q++) {
        head[q] = 0;
        cur[q] = fetch(lane + 64u * q, 0);
        nxt[q] = fetch(lane + 64u * q, 1);
    }
    uint32_t k = 0;
    for (uint32_t j = 0; j < top_k; j++) {
        uint64_t c = cur[0];
#pragma unroll
        for (int q = 1; q < OXB_SAMPLE_LISTS_PER_LANE; q++) c = cur[q] > c ? cur[q] : c;
        const uint64_t best = wave_max_key(c);
        if (best == 0) break;  // fewer than top_k logits in the row (uniform: every lane sees it)
#pragma unroll
        for (int q = 0; q < OXB_SAMPLE_LISTS_PER_LANE; q++)
            if (cur[q] == best) {  // unique keys: one list of one lane
                head[q]++;
                cur[q] = nxt[q];
                nxt[q] = fetch(lane + 64u * q, head[q] + 1);
            }
        if (lane == 0) pv[j] = key_value(best), pi[j] = key_index(best);
        k = j + 1;
    }
    // pv[0..k) descending.  From here on: sampling.rs:104-176 on the k candidates.  The element-wise part on all
    // lanes (the exponential through double precision: the nearest f32, as libm's expf gives in all but rare cases),
    // the sums by lane 0 in the reference's order.
    __syncthreads();
    if (k > 0) {
        const float max_val = pv[0] / temperature;
        float e[(OXB_SAMPLE_MAX_TOP_K + 63) / 64];
#pragma unroll
        for (uint32_t q = 0; q < (OXB_SAMPLE_MAX_TOP_K + 63) / 64; q++) {
            const uint32_t j = lane + 64u * q;
            e[q] = j < k ? (float)exp((double)(pv[j] / temperature - max_val)) : 0.0f;
        }
        __syncthreads();
#pragma unroll
        for (uint32_t q = 0; q < (OXB_SAMPLE_MAX_TOP_K + 63) / 64; q++)
            if (lane + 64u * q < k) pv[lane + 64u * q] = e[q];
    }
    __syncthreads();
    if (lane != 0) return;
    float sum = 0.0f;
    for (uint32_t j = 0; j < k; j++) sum += pv[j];
    for (uint32_t j = 0; j < k; j++) pv[j] /= sum;
    if (top_p < 1.0f) {
        float cum = 0.0f;
        uint32_t cutoff = k ? k - 1 : 0;
        for (uint32_t j = 0; j < k; j++) {
            cum += pv[j];
            if (cum > top_p) {
                cutoff = j;
                break;
            }
        }
        k = cutoff + 1;
        float s2 = 0.0f;
        for (uint32_t j = 0; j < k; j++) s2 += pv[j];
        for (uint32_t j = 0; j < k; j++) pv[j] /= s2;
    }
    uint64_t x = rng[row];
    x ^= x << 13;
    x ^= x >> 7;
    x ^= x << 17;
    rng[row] = x;
    const float r = (float)((double)x / 18446744073709551615.0);
    uint32_t tok = pi[0];
    float cum = 0.0f;
    for (uint32_t j = 0; j < k; j++) {
        cum += pv[j];
        if (r <= cum) {
            tok = pi[j];
            break;
        }
    }
    tokens[row] = tok;
}

// ---------------------------------------------------------------------------
// Sampler::sample with top-k off (top_k = 0 or >= the vocabulary: the Creative preset, presets.rs:57-63).  The
// reference then works on the whole vocabulary in index order (sampling.rs:98-104): softmax with the sum taken
// element by element in f32 (:121-133), for top-p a stable descending sort (:136-137), the cumulative cut and the
// renormalising sum again element by element (:138-152), and the cumulative pick (:160-171).  f32 addition is not
// associative and over 150 000 nearly equal probabilities the order of the additions decides which token a draw
// lands on, so every one of these sums runs here as one chain in the reference's order (one wave per row: 64
// elements per load, added lane by lane); only the element-wise steps and the sort are parallel.
// ---------------------------------------------------------------------------
#define OXB_FULL_SPAN 2048u

__device__ __forceinline__ float block_max_256(float v, float* sm4) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    if ((threadIdx.x & 63u) == 0) sm4[threadIdx.x >> 6] = v;
    __syncthreads();
    return fmaxf(fmaxf(sm4[0], sm4[1]), fmaxf(sm4[2], sm4[3]));  // f32::max semantics: a NaN operand is dropped
}

__global__ __launch_bounds__(256) void full_max_kernel(const float* __restrict__ logits, uint32_t n, float* __restrict__ pmax) {
    __shared__ float sm4[4];
    const float* v = logits + (size_t)blockIdx.y * n;
    float mx = -INFINITY;
    for (uint32_t i = blockIdx.x * OXB_FULL_SPAN + threadIdx.x; i < min(n, (blockIdx.x + 1) * OXB_FULL_SPAN); i += 256) mx = fmaxf(mx, v[i]);
    mx = block_max_256(mx, sm4);
    if (threadIdx.x == 0) pmax[(size_t)blockIdx.y * gridDim.x + blockIdx.x] = mx;
}

// e[i] = exp(v[i] / T - max / T): the quotient and the difference in f32 as the reference forms them, the exponential
// through double precision, which rounds to the nearest f32 like libm's expf does in all but very rare cases.
__global__ __launch_bounds__(256) void full_exp_kernel(const float* __restrict__ logits, uint32_t n, float temperature,
                                                        const float* __restrict__ pmax, float* __restrict__ e_out,
                                                        uint32_t* __restrict__ iota) {
    __shared__ float sm4[4];
    const uint32_t row = blockIdx.y, parts = gridDim.x;
    float mx = -INFINITY;
    for (uint32_t j = threadIdx.x; j < parts; j += 256) mx = fmaxf(mx, pmax[(size_t)row * parts + j]);
    const float ms = block_max_256(mx, sm4) / temperature;  // max of the quotients = quotient of the max (T > 0, division is monotone)
    const float* v = logits + (size_t)row * n;
    for (uint32_t i = blockIdx.x * OXB_FULL_SPAN + threadIdx.x; i < min(n, (blockIdx.x + 1) * OXB_FULL_SPAN); i += 256) {
        const float x = v[i] / temperature;
        e_out[(size_t)row * n + i] = (float)exp((double)(x - ms));
        if (row == 0) iota[i] = i;
    }
}

// acc + x(lane 0) + x(lane 1) + ... + x(lane 63), added in that order.
__device__ __forceinline__ float chain64(float acc, float x) {
#pragma unroll
    for (int l = 0; l < 64; l++) acc += __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, x), l));
    return acc;
}

__device__ __forceinline__ uint32_t wave_sum_u32(uint32_t v) {
    v += dpp_u32<OXB_DPP_ROW_SHR(1)>(v);
    v += dpp_u32<OXB_DPP_ROW_SHR(2)>(v);
    v += dpp_u32<OXB_DPP_ROW_SHR(4)>(v);
    v += dpp_u32<OXB_DPP_ROW_SHR(8)>(v);  // lane 16 r + 15 holds the total of its row of 16 lanes
    return (uint32_t)__builtin_amdgcn_readlane((int)v, 15) + (uint32_t)__builtin_amdgcn_readlane((int)v, 31) +
           (uint32_t)__builtin_amdgcn_readlane((int)v, 47) + (uint32_t)__builtin_amdgcn_readlane((int)v, 63);
}

// The same result as C x chain64 (elements c * 64 + lane in ascending order) without the chain, where that is
// provable.  While the running sum s stays inside one binade its ulp u is fixed, and fl(s + x) = s + u * R(x / u) with
// R = round to nearest: the sum is an integer accumulation T += R_i of the mantissa T = s / u.  The increments do
// not depend on T except where x / u ends in exactly one half: such a tie goes to the even mantissa, so it adds
// floor(x / u) plus one if T + floor(x / u) is odd - and leaves T even.  Parity is therefore all the state there is:
// before a tie it is the parity of T at the previous tie (even) or at the start, flipped once per odd increment in
// between.  Every lane forms its increment from the bits of x; the odd increments and the ties of a chunk become two
// 64-bit lane masks, over which the carries of the ties are worked out with scalar bit operations; one wave-wide
// integer sum finishes the group.  Refused (false: the caller adds the elements one by one) if an element is negative,
// NaN, infinite or at least u * 2^23, if s is zero, subnormal or not finite, or if the mantissa would reach 2^24 (the
// binade is left; the terms are >= 0, so then and only then some partial sum leaves it too).
template <int C>
__device__ __forceinline__ bool chain_fast(float& acc, const float (&x)[C]) {
    const uint32_t sb = __float_as_uint(acc), es = sb >> 23;  // acc >= 0 here
    if (es == 0 || es >= 255) return false;
    const uint32_t T = (sb & 0x7FFFFFu) | 0x800000u;
    uint32_t f_sum = 0, carries = 0, par = T & 1u;
    bool bad = false;
#pragma unroll
    for (int c = 0; c < C; c++) {
        const uint32_t b = __float_as_uint(x[c]), ex0 = b >> 23;  // a set sign bit makes ex0 >= 256
        uint32_t m = b & 0x7FFFFFu;
        const uint32_t ex = ex0 ? ex0 : 1u;
        if (ex0) m |= 0x800000u;
        // x = m * 2^(ex - 150), u = 2^(es - 150): x / u = m / 2^shr with shr = es - ex
        const int shr = (int)es - (int)ex;
        uint32_t f = 0;
        bool tie = false;
        if (m != 0u) {  // (a -0 counts as +0)
            if (ex0 >= 255u || shr <= 0) {
                bad = true;
            } else if (shr <= 24) {
                const uint32_t rem = m & ((1u << shr) - 1u), half = 1u << (shr - 1);
                f = (m >> shr) + (rem > half ? 1u : 0u);
                tie = rem == half;
            }  // shr >= 25: less than half an ulp, the sum does not move
        }
        f_sum += f;
        const uint64_t odd = __builtin_amdgcn_ballot_w64((f & 1u) != 0u);
        uint64_t ties = __builtin_amdgcn_ballot_w64(tie);
        uint64_t done = 0;  // lanes up to and including the last tie handled
        while (ties) {
            const uint32_t i = (uint32_t)__builtin_ctzll(ties);
            ties &= ties - 1;
            const uint64_t below = (1ull << i) - 1ull;
            const uint32_t before = par ^ ((uint32_t)__builtin_popcountll(odd & below & ~done) & 1u);
            carries += before ^ (uint32_t)((odd >> i) & 1ull);  // T + floor odd -> one more, and T is even afterwards
            par = 0;
            done = below | (1ull << i);
        }
        par ^= (uint32_t)__builtin_popcountll(odd & ~done) & 1u;
    }
    if (__builtin_amdgcn_ballot_w64(bad) != 0ull) return false;
    const uint32_t total = T + wave_sum_u32(f_sum) + carries;  // <= 2^24 + 64 C * (2^23 + 1): no overflow for C <= 4
    if (total >= 0x1000000u) return false;
    acc = __uint_as_float((es << 23) | (total & 0x7FFFFFu));
    return true;
}

// acc + the wave's 64 values in lane order.
__device__ __forceinline__ float add64(float acc, float x) {
    float a = acc;
    const float xs[1] = {x};
    if (chain_fast<1>(a, xs)) return a;
    return chain64(acc, x);
}

// acc + the 256 values of cur in element order.
__device__ __forceinline__ float add256(float acc, const float (&cur)[4]) {
    float a = acc;
    if (chain_fast<4>(a, cur)) return a;
#pragma unroll
    for (int c = 0; c < 4; c++) acc = chain64(acc, cur[c]);
    return acc;
}

// What chain_fast needs from 256 elements when none of them is a rounding tie: the sum of the mantissa increments for a
// running sum with biased exponent es.  `refuse` is set if chain_fast would refuse the elements or if one is a tie.
__device__ __forceinline__ uint32_t increments256(uint32_t es, const float (&x)[4], bool& refuse) {
    uint32_t f_sum = 0;
    bool bad = es == 0 || es >= 255;
#pragma unroll
    for (int c = 0; c < 4; c++) {
        const uint32_t b = __float_as_uint(x[c]), ex0 = b >> 23;
        uint32_t m = b & 0x7FFFFFu;
        const uint32_t ex = ex0 ? ex0 : 1u;
        if (ex0) m |= 0x800000u;
        const int shr = (int)es - (int)ex;
        if (m != 0u) {
            if (ex0 >= 255u || shr <= 0) {
                bad = true;
            } else if (shr <= 24) {
                const uint32_t rem = m & ((1u << shr) - 1u), half = 1u << (shr - 1);
                f_sum += (m >> shr) + (rem > half ? 1u : 0u);
                bad |= rem == half;
            }
        }
    }
    refuse = __builtin_amdgcn_ballot_w64(bad) != 0ull;
    return wave_sum_u32(f_sum);
}

// The running f32 sum of x[0 .. n) (each element divided by `divisor` first if `divide`), taken in element order
// from L.acc, up to the first element at which pred(sum) holds: returns true and its position in `where`, or false
// with the whole sum.  L.acc holds the sum reached in either case.  One workgroup of four waves, all threads call:
//  * the row comes through two LDS tiles of 4096 elements, the next tile's loads in flight while this one is summed;
//  * the four waves take the four 256-element groups of a 1024-element batch at once, each forming its group's mantissa
//    increments for the binade the sum is in at the start of the batch (increments256).  If no group refuses and the
//    mantissa stays inside the binade, the batch's result is the integer sum - the order does not matter then;
//  * otherwise, or when pred holds after the batch, the first wave redoes the batch group by group in order
//    (add256, add64, and lane by lane around the crossing).
struct RowSum {
    float t[2][4096];
    uint32_t inc[4], refuse[4];
    float acc;
    uint32_t stop, where;
};
template <class Pred>
__device__ __forceinline__ bool run_sum(const float* __restrict__ x, uint32_t n, bool divide, float divisor, RowSum& L, Pred pred,
                                        uint32_t& where) {
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6;
    auto lane_value = [](float v, uint32_t l) { return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), (int)l)); };
    float r[16];
    auto fetch = [&](uint32_t base) {
#pragma unroll
        for (int j = 0; j < 16; j++) {
            const uint32_t i = base + 256u * j + tid;
            r[j] = i < n ? x[i] : 0.0f;  // adding +0 past the end changes nothing
        }
    };
    auto stash = [&](uint32_t buf) {
#pragma unroll
        for (int j = 0; j < 16; j++) L.t[buf][256u * j + tid] = divide ? r[j] / divisor : r[j];
    };
    if (tid == 0) L.stop = 0u;
    fetch(0);
    stash(0);
    __syncthreads();
    for (uint32_t base = 0, buf = 0; base < n; base += 4096u, buf ^= 1u) {
        const bool more = base + 4096u < n;  // uniform
        if (more) fetch(base + 4096u);
        for (uint32_t bb = 0; bb < 4096u && base + bb < n; bb += 1024u) {
            float cur[4];
#pragma unroll
            for (int c = 0; c < 4; c++) cur[c] = L.t[buf][bb + 256u * wave + 64u * c + lane];
            const uint32_t sb = __float_as_uint(L.acc), es = sb >> 23;
            bool refuse;
            const uint32_t inc = increments256(es, cur, refuse);
            if (lane == 0) L.inc[wave] = inc, L.refuse[wave] = refuse ? 1u : 0u;
            __syncthreads();
            if (wave == 0) {
                uint32_t total = (sb & 0x7FFFFFu) | 0x800000u;
                bool slow = false;
                for (uint32_t w = 0; w < 4 && base + bb + 256u * w < n; w++) {
                    total += L.inc[w];  // each < 2^30: no overflow before the check
                    slow |= L.refuse[w] != 0u || total >= 0x1000000u;
                }
                const float fast = __uint_as_float((es << 23) | (total & 0x7FFFFFu));
                if (!slow && !pred(fast)) {  // the terms are >= 0: no partial sum exceeds the last
                    if (lane == 0) L.acc = fast;
                } else {
                    float cum = L.acc;
                    bool found = false;
                    uint32_t at = 0;
                    for (uint32_t w = 0; w < 4 && base + bb + 256u * w < n && !found; w++) {
                        float q[4];
#pragma unroll
                        for (int c = 0; c < 4; c++) q[c] = L.t[buf][bb + 256u * w + 64u * c + lane];
                        const float all = add256(cum, q);
                        if (!pred(all)) {
                            cum = all;
                            continue;
                        }
                        for (uint32_t c = 0; c < 4 && !found; c++) {
                            const float qc = c == 0 ? q[0] : (c == 1 ? q[1] : (c == 2 ? q[2] : q[3]));
                            const float end = add64(cum, qc);
                            if (pred(end)) {
                                float s2 = cum;
                                for (uint32_t l = 0; l < 64; l++) {
                                    s2 += lane_value(qc, l);
                                    if (pred(s2)) {
                                        at = base + bb + 256u * w + 64u * c + l;
                                        cum = s2;
                                        found = true;
                                        break;
                                    }
                                }
                            } else {
                                cum = end;
                            }
                        }
                    }
                    if (lane == 0) {
                        L.acc = cum;
                        if (found) L.stop = 1u, L.where = at;
                    }
                }
            }
            __syncthreads();
            if (L.stop) break;
        }
        if (L.stop) break;  // uniform
        if (more) stash(buf ^ 1u);
        __syncthreads();
    }
    const bool hit = L.stop != 0u;
    if (hit) where = L.where;
    __syncthreads();  // everybody has read the result before the next run rewrites the flags and tiles
    return hit;
}

// sum[row] = e[row][0] + e[row][1] + ... in element order (sampling.rs:126-130).  One workgroup per row.
__global__ __launch_bounds__(256) void full_sum_kernel(const float* __restrict__ e, uint32_t stride, uint32_t n, float* __restrict__ sum) {
    __shared__ RowSum L;
    if (threadIdx.x == 0) L.acc = 0.0f;
    __syncthreads();
    uint32_t unused = 0;
    run_sum(e + (size_t)blockIdx.x * stride, n, false, 1.0f, L, [](float) { return false; }, unused);
    if (threadIdx.x == 0) sum[blockIdx.x] = L.acc;
}

__global__ __launch_bounds__(256) void full_prob_kernel(float* __restrict__ e, uint32_t stride, uint32_t n, const float* __restrict__ sum) {
    const float s = sum[blockIdx.y];
    float* x = e + (size_t)blockIdx.y * stride;
    for (uint32_t i = blockIdx.x * OXB_FULL_SPAN + threadIdx.x; i < min(n, (blockIdx.x + 1) * OXB_FULL_SPAN); i += 256) x[i] /= s;
}

// A top-k beyond what the selection kernels hold (129 .. vocabulary - 1): the whole row is sorted by v / T, descending and
// stable (equal values keep index order, -0 counted as +0: the order the selection route produces), and the first
// top_k entries go through the same softmax, cut and pick as above, in that order.
__global__ __launch_bounds__(256) void full_scale_kernel(const float* __restrict__ logits, uint32_t n, float temperature,
                                                          float* __restrict__ out, uint32_t* __restrict__ iota) {
    const float* v = logits + (size_t)blockIdx.y * n;
    for (uint32_t i = blockIdx.x * OXB_FULL_SPAN + threadIdx.x; i < min(n, (blockIdx.x + 1) * OXB_FULL_SPAN); i += 256) {
        out[(size_t)blockIdx.y * n + i] = v[i] / temperature + 0.0f;
        if (blockIdx.y == 0) iota[i] = i;
    }
}
__global__ __launch_bounds__(256) void sorted_exp_kernel(const float* __restrict__ sorted, uint32_t stride, uint32_t k, float* __restrict__ e_out) {
    const float* x = sorted + (size_t)blockIdx.y * stride;
    const float mx = x[0];
    for (uint32_t j = blockIdx.x * OXB_FULL_SPAN + threadIdx.x; j < min(k, (blockIdx.x + 1) * OXB_FULL_SPAN); j += 256)
        e_out[(size_t)blockIdx.y * stride + j] = (float)exp((double)(x[j] - mx));
}

// Top-p cut, renormalisation, draw and pick over the row's probabilities p (sorted descending with their token ids
// when top-p is on or top-k was taken by sorting, else in index order with ids = null).  One workgroup per row; every
// sum runs in element order (run_sum).
__global__ __launch_bounds__(256) void full_pick_kernel(const float* __restrict__ p_all, const uint32_t* __restrict__ ids_all, uint32_t stride,
                                                         uint32_t n, float top_p, uint64_t* __restrict__ rng, uint32_t* __restrict__ tokens) {
    __shared__ RowSum L;
    const uint32_t row = blockIdx.x, tid = threadIdx.x;
    const float* p = p_all + (size_t)row * stride;
    const uint32_t* ids = ids_all ? ids_all + (size_t)row * stride : nullptr;
    uint64_t x64 = rng[row];  // read by everybody before the first barrier; written once at the very end
    x64 ^= x64 << 13;
    x64 ^= x64 >> 7;
    x64 ^= x64 << 17;
    const float r = (float)((double)x64 / 18446744073709551615.0);
    auto restart = [&]() {
        if (tid == 0) L.acc = 0.0f;
        __syncthreads();
    };
    uint32_t m = n;
    float s2 = 1.0f;
    const bool cut = top_p < 1.0f;
    if (cut) {
        // position(|p| { cum += p; cum > top_p }).unwrap_or(len - 1), sampling.rs:138-146
        uint32_t cutoff = n - 1;
        restart();
        run_sum(p, n, false, 1.0f, L, [&](float v) { return v > top_p; }, cutoff);
        m = cutoff + 1;
        restart();  // the renormalising sum over the kept entries, :150-152
        uint32_t unused = 0;
        run_sum(p, m, false, 1.0f, L, [](float) { return false; }, unused);
        s2 = L.acc;
        __syncthreads();
    }
    uint32_t pick = 0;  // the fallback is the buffer's first entry, :173-174
    restart();
    run_sum(p, m, cut, s2, L, [&](float v) { return r <= v; }, pick);
    if (tid == 0) {
        rng[row] = x64;
        tokens[row] = ids ? ids[pick] : pick;
    }
}

hipError_t oxb_launch_embedding_gather(const void* d_table, int gguf_type, uint32_t vocab, uint32_t h, const uint32_t* d_ids,
                                       uint32_t n, float* d_out, hipStream_t st) {
    if (n == 0) return hipSuccess;
    if ((gguf_type != 0 && gguf_type != 1 && gguf_type != 41 && gguf_type != 42) || (gguf_type >= 41 && h % 128u)) return hipErrorInvalidValue;
    hipLaunchKernelGGL(embedding_gather_kernel, dim3(n), dim3(256), 0, st, static_cast<const uint8_t*>(d_table), gguf_type, vocab, h,
                       d_ids, d_out);
    return hipGetLastError();
}

hipError_t oxb_launch_token_step(const uint32_t* d_tokens, uint32_t* d_history, uint32_t* d_pos, uint32_t batch, hipStream_t st) {
    hipLaunchKernelGGL(token_step_kernel, dim3((batch + 63) / 64), dim3(64), 0, st, d_tokens, d_history, d_pos, batch);
    return hipGetLastError();
}

static uint32_t sample_parts(uint32_t n) { return (n + OXB_TOPK_SPAN - 1) / OXB_TOPK_SPAN; }

static size_t align256(size_t v) { return (v + 255u) & ~(size_t)255u; }

// Scratch of the top-k-off route: e / p [batch][n], sorted p [batch][n], sorted ids [batch][n], iota [n],
// part maxima [batch][parts], sums [batch], the sort's temporary storage.
struct FullWs { size_t e, ps, is, iota, pmax, sum, tmp, tmp_bytes, total; };
static hipError_t full_ws_layout(uint32_t n, uint32_t batch, FullWs* w) {
    size_t tmp = 0;
    hipError_t err = rocprim::radix_sort_pairs_desc(nullptr, tmp, (const float*)nullptr, (float*)nullptr, (const uint32_t*)nullptr,
                                                    (uint32_t*)nullptr, (unsigned int)n);
    if (err != hipSuccess) return err;
    const size_t rows = align256((size_t)n * 4 * batch), parts = (n + OXB_FULL_SPAN - 1) / OXB_FULL_SPAN;
    w->e = 0;
    w->ps = w->e + rows;
    w->is = w->ps + rows;
    w->iota = w->is + rows;
    w->pmax = w->iota + align256((size_t)n * 4);
    w->sum = w->pmax + align256((size_t)batch * parts * 4);
    w->tmp = w->sum + align256((size_t)batch * 4);
    w->tmp_bytes = tmp;
    w->total = w->tmp + align256(tmp);
    return hipSuccess;
}

size_t oxb_sample_ws_bytes(uint32_t n, uint32_t batch) {
    const size_t topk = (size_t)batch * sample_parts(n) * OXB_SAMPLE_MAX_TOP_K * 8;
    FullWs w;
    if (n > 0x7FFFFFFFu || full_ws_layout(n, batch, &w) != hipSuccess) return topk;
    return topk > w.total ? topk : w.total;
}

// top_k = 0: the filter is off; otherwise 128 < top_k < n.
static hipError_t launch_sample_full(const float* d_logits, uint32_t n, uint32_t batch, float temperature, uint32_t top_k, float top_p,
                                     uint64_t* d_rng, uint32_t* d_tokens, void* d_ws, hipStream_t st) {
    FullWs w;
    if (n > 0x7FFFFFFFu) return hipErrorInvalidValue;
    hipError_t err = full_ws_layout(n, batch, &w);
    if (err != hipSuccess) return err;
    uint8_t* base = static_cast<uint8_t*>(d_ws);
    float* e = reinterpret_cast<float*>(base + w.e);
    float* ps = reinterpret_cast<float*>(base + w.ps);
    uint32_t* is = reinterpret_cast<uint32_t*>(base + w.is);
    uint32_t* iota = reinterpret_cast<uint32_t*>(base + w.iota);
    float* pmax = reinterpret_cast<float*>(base + w.pmax);
    float* sum = reinterpret_cast<float*>(base + w.sum);
    const uint32_t parts = (n + OXB_FULL_SPAN - 1) / OXB_FULL_SPAN;
    auto sort_rows = [&]() -> hipError_t {  // e -> ps (descending, stable), iota -> is
        for (uint32_t b = 0; b < batch; b++) {
            size_t tmp = w.tmp_bytes;
            hipError_t r = rocprim::radix_sort_pairs_desc(base + w.tmp, tmp, e + (size_t)b * n, ps + (size_t)b * n, iota,
                                                          is + (size_t)b * n, (unsigned int)n, 0, 32, st);
            if (r != hipSuccess) return r;
        }
        return hipSuccess;
    };
    if (top_k != 0) {
        const uint32_t kparts = (top_k + OXB_FULL_SPAN - 1) / OXB_FULL_SPAN;
        hipLaunchKernelGGL(full_scale_kernel, dim3(parts, batch), dim3(256), 0, st, d_logits, n, temperature, e, iota);
        if ((err = sort_rows()) != hipSuccess) return err;
        hipLaunchKernelGGL(sorted_exp_kernel, dim3(kparts, batch), dim3(256), 0, st, ps, n, top_k, e);
        hipLaunchKernelGGL(full_sum_kernel, dim3(batch), dim3(256), 0, st, e, n, top_k, sum);
        hipLaunchKernelGGL(full_prob_kernel, dim3(kparts, batch), dim3(256), 0, st, e, n, top_k, sum);
        hipLaunchKernelGGL(full_pick_kernel, dim3(batch), dim3(256), 0, st, e, is, n, top_k, top_p, d_rng, d_tokens);
        return hipGetLastError();
    }
    hipLaunchKernelGGL(full_max_kernel, dim3(parts, batch), dim3(256), 0, st, d_logits, n, pmax);
    hipLaunchKernelGGL(full_exp_kernel, dim3(parts, batch), dim3(256), 0, st, d_logits, n, temperature, pmax, e, iota);
    hipLaunchKernelGGL(full_sum_kernel, dim3(batch), dim3(256), 0, st, e, n, n, sum);
    hipLaunchKernelGGL(full_prob_kernel, dim3(parts, batch), dim3(256), 0, st, e, n, n, sum);
    if (top_p < 1.0f) {
        if ((err = sort_rows()) != hipSuccess) return err;  // stable: equal probabilities keep index order, as sort_by does
        hipLaunchKernelGGL(full_pick_kernel, dim3(batch), dim3(256), 0, st, ps, is, n, n, top_p, d_rng, d_tokens);
    } else {
        hipLaunchKernelGGL(full_pick_kernel, dim3(batch), dim3(256), 0, st, e, (const uint32_t*)nullptr, n, n, top_p, d_rng, d_tokens);
    }
    return hipGetLastError();
}

hipError_t oxb_launch_sum_in_order(const float* d_x, uint32_t n, float* d_sum, hipStream_t st) {
    hipLaunchKernelGGL(full_sum_kernel, dim3(1), dim3(256), 0, st, d_x, n, n, d_sum);
    return hipGetLastError();
}

hipError_t oxb_launch_sample(const float* d_logits, uint32_t n, uint32_t batch, float temperature, uint32_t top_k, float top_p,
                             uint64_t* d_rng, uint32_t* d_tokens, void* d_ws, hipStream_t st) {
    const uint32_t parts = sample_parts(n);
    if (n == 0 || batch == 0 || !(temperature >= 1e-6f) || !d_ws) return hipErrorInvalidValue;
    if (top_k == 0 || top_k >= n)  // the filter is off (sampling.rs:111)
        return launch_sample_full(d_logits, n, batch, temperature, 0, top_p, d_rng, d_tokens, d_ws, st);
    if (top_k > OXB_SAMPLE_MAX_TOP_K) return launch_sample_full(d_logits, n, batch, temperature, top_k, top_p, d_rng, d_tokens, d_ws, st);
    if (parts > 64 * OXB_SAMPLE_LISTS_PER_LANE) return hipErrorInvalidValue;
    float* cv = reinterpret_cast<float*>(d_ws);
    uint32_t* ci = reinterpret_cast<uint32_t*>(d_ws) + (size_t)batch * parts * top_k;
    hipLaunchKernelGGL(topk_partial_kernel, dim3(parts, batch), dim3(256), 0, st, d_logits, n, top_k, cv, ci);
    if (parts * top_k <= OXB_SAMPLE_LDS_KEYS)
        hipLaunchKernelGGL(sample_final_kernel<true>, dim3(batch), dim3(64), 0, st, cv, ci, parts, top_k, temperature, top_p, d_rng, d_tokens);
    else
        hipLaunchKernelGGL(sample_final_kernel<false>, dim3(batch), dim3(64), 0, st, cv, ci, parts, top_k, temperature, top_p, d_rng, d_tokens);
    return hipGetLastError();
}
