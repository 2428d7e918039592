// token_kernels.hip — token embedding lookup, top-k / top-p sampling and token bookkeeping of the on-device
// generation loop.
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

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
// order; lane 0 then walks the reference's arithmetic over those <= 128 values: v / temperature, exp(v - max),
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
__global__ __launch_bounds__(64) void sample_final_kernel(const float* __restrict__ cv, const uint32_t* __restrict__ ci,
                                                           uint32_t parts, uint32_t top_k, float temperature, float top_p,
                                                           uint64_t* __restrict__ rng, uint32_t* __restrict__ tokens) {
    __shared__ float pv[OXB_SAMPLE_MAX_TOP_K];
    __shared__ uint32_t pi[OXB_SAMPLE_MAX_TOP_K];
    const uint32_t row = blockIdx.x, lane = threadIdx.x;
    const float* lv = cv + (size_t)row * parts * top_k;
    const uint32_t* li = ci + (size_t)row * parts * top_k;
    // lane t walks the sorted lists of parts t, t + 64, ...: `cur` is each list's head, `nxt` the element behind it
    uint64_t cur[OXB_SAMPLE_LISTS_PER_LANE], nxt[OXB_SAMPLE_LISTS_PER_LANE];
    uint32_t head[OXB_SAMPLE_LISTS_PER_LANE];
    auto fetch = [&](uint32_t part, uint32_t at) -> uint64_t {
        if (part >= parts || at >= top_k) return 0ull;
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
    if (lane != 0) return;
    // pv[0..k) descending.  From here on: sampling.rs:104-176 on the k candidates.
    for (uint32_t j = 0; j < k; j++) pv[j] = pv[j] / temperature;
    const float max_val = pv[0];
    float sum = 0.0f;
    for (uint32_t j = 0; j < k; j++) {
        pv[j] = expf(pv[j] - max_val);
        sum += pv[j];
    }
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

size_t oxb_sample_ws_bytes(uint32_t n, uint32_t batch) {
    return (size_t)batch * sample_parts(n) * OXB_SAMPLE_MAX_TOP_K * 8;
}

hipError_t oxb_launch_sample(const float* d_logits, uint32_t n, uint32_t batch, float temperature, uint32_t top_k, float top_p,
                             uint64_t* d_rng, uint32_t* d_tokens, void* d_ws, hipStream_t st) {
    const uint32_t parts = sample_parts(n);
    if (n == 0 || batch == 0 || top_k == 0 || top_k > OXB_SAMPLE_MAX_TOP_K || parts > 64 * OXB_SAMPLE_LISTS_PER_LANE || !(temperature >= 1e-6f) || !d_ws)
        return hipErrorInvalidValue;
    float* cv = reinterpret_cast<float*>(d_ws);
    uint32_t* ci = reinterpret_cast<uint32_t*>(d_ws) + (size_t)batch * parts * top_k;
    hipLaunchKernelGGL(topk_partial_kernel, dim3(parts, batch), dim3(256), 0, st, d_logits, n, top_k, cv, ci);
    hipLaunchKernelGGL(sample_final_kernel, dim3(batch), dim3(64), 0, st, cv, ci, parts, top_k, temperature, top_p, d_rng, d_tokens);
    return hipGetLastError();
}
