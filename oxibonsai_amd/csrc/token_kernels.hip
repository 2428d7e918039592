// token_kernels.hip — token embedding lookup, top-k / top-p sampling and token bookkeeping of the on-device
// generation loop.
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

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
// Stage 1, grid (parts, rows): a workgroup keeps its span of the logits in registers (EPT per thread, each
// thread's sorted descending) and pops the maximum top_k times: its top_k in descending order, ties to the lower
// index.  Stage 2, one workgroup per row: the same pop over the heads of the parts' sorted lists yields the
// row's top_k in descending order; thread 0 then walks the reference's arithmetic over those <= 128 values:
// v / temperature, exp(v - max), sum, divide, top-p cut, renormalise, r = (xorshift64 / u64::MAX) as f32,
// cumulative pick (first candidate if none reaches r).  The reference leaves the candidates in whatever order
// its partial selection produces when top_p == 1; here the order is always descending.
// ---------------------------------------------------------------------------
#define OXB_TOPK_EPT 8
#define OXB_TOPK_SPAN (256 * OXB_TOPK_EPT)

struct Cand {
    float v;
    uint32_t i;  // 0xFFFFFFFF: empty
};
__device__ __forceinline__ bool cand_before(const Cand& a, const Cand& b) {  // a is taken before b
    if (b.i == 0xFFFFFFFFu) return a.i != 0xFFFFFFFFu;
    if (a.i == 0xFFFFFFFFu) return false;
    return a.v > b.v || (a.v == b.v && a.i < b.i);
}
// Best candidate of the workgroup's 256 threads (every thread gets it) and the thread that offered it.
__device__ __forceinline__ Cand block_best(Cand c, uint32_t* owner, Cand* sc, uint32_t* so) {
    uint32_t who = threadIdx.x;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        Cand other;
        other.v = __shfl_xor(c.v, o, 64);
        other.i = __shfl_xor(c.i, o, 64);
        const uint32_t ow = __shfl_xor(who, o, 64);
        if (cand_before(other, c)) c = other, who = ow;
    }
    if ((threadIdx.x & 63u) == 0) sc[threadIdx.x >> 6] = c, so[threadIdx.x >> 6] = who;
    __syncthreads();
    c = sc[0], who = so[0];
#pragma unroll
    for (int w = 1; w < 4; w++)
        if (cand_before(sc[w], c)) c = sc[w], who = so[w];
    __syncthreads();
    *owner = who;
    return c;
}

__global__ __launch_bounds__(256) void topk_partial_kernel(const float* __restrict__ logits, uint32_t n, uint32_t top_k,
                                                            float* __restrict__ cv, uint32_t* __restrict__ ci) {
    __shared__ Cand sc[4];
    __shared__ uint32_t so[4];
    const float* v = logits + (size_t)blockIdx.y * n;
    const uint32_t i0 = blockIdx.x * OXB_TOPK_SPAN;
    Cand mine[OXB_TOPK_EPT];
#pragma unroll
    for (int e = 0; e < OXB_TOPK_EPT; e++) {
        const uint32_t i = i0 + threadIdx.x + 256u * e;
        mine[e].i = i < n ? i : 0xFFFFFFFFu;
        mine[e].v = i < n ? v[i] : 0.0f;
    }
    // sort the thread's own values, best first (a NaN compares false everywhere and sinks to wherever it is)
#pragma unroll
    for (int a = 1; a < OXB_TOPK_EPT; a++)
#pragma unroll
        for (int b = a; b > 0; b--)
            if (cand_before(mine[b], mine[b - 1])) {
                const Cand t = mine[b];
                mine[b] = mine[b - 1];
                mine[b - 1] = t;
            }
    const size_t out = ((size_t)blockIdx.y * gridDim.x + blockIdx.x) * top_k;
    for (uint32_t j = 0; j < top_k; j++) {
        uint32_t owner;
        const Cand best = block_best(mine[0], &owner, sc, so);
        if (threadIdx.x == owner) {  // pop: shift the thread's list
#pragma unroll
            for (int e = 0; e + 1 < OXB_TOPK_EPT; e++) mine[e] = mine[e + 1];
            mine[OXB_TOPK_EPT - 1].i = 0xFFFFFFFFu;
        }
        if (threadIdx.x == 0) cv[out + j] = best.v, ci[out + j] = best.i;
    }
}

__global__ __launch_bounds__(256) void sample_final_kernel(const float* __restrict__ cv, const uint32_t* __restrict__ ci,
                                                            uint32_t parts, uint32_t top_k, float temperature, float top_p,
                                                            uint64_t* __restrict__ rng, uint32_t* __restrict__ tokens) {
    __shared__ Cand sc[4];
    __shared__ uint32_t so[4];
    __shared__ float pv[OXB_SAMPLE_MAX_TOP_K];
    __shared__ uint32_t pi[OXB_SAMPLE_MAX_TOP_K];
    const uint32_t row = blockIdx.x;
    const float* lv = cv + (size_t)row * parts * top_k;
    const uint32_t* li = ci + (size_t)row * parts * top_k;
    // thread t < parts walks part t's sorted list
    uint32_t head = 0;
    uint32_t k = 0;
    for (uint32_t j = 0; j < top_k; j++) {
        Cand c;
        c.i = 0xFFFFFFFFu, c.v = 0.0f;
        if (threadIdx.x < parts && head < top_k) {
            c.v = lv[(size_t)threadIdx.x * top_k + head];
            c.i = li[(size_t)threadIdx.x * top_k + head];
        }
        uint32_t owner;
        const Cand best = block_best(c, &owner, sc, so);
        if (best.i == 0xFFFFFFFFu) break;  // fewer than top_k logits in the row (uniform: every thread sees it)
        if (threadIdx.x == owner) head++;
        if (threadIdx.x == 0) pv[j] = best.v, pi[j] = best.i;
        k = j + 1;
    }
    if (threadIdx.x != 0) return;
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
    if (n == 0 || batch == 0 || top_k == 0 || top_k > OXB_SAMPLE_MAX_TOP_K || parts > 256 || !(temperature >= 1e-6f) || !d_ws)
        return hipErrorInvalidValue;
    float* cv = reinterpret_cast<float*>(d_ws);
    uint32_t* ci = reinterpret_cast<uint32_t*>(d_ws) + (size_t)batch * parts * top_k;
    hipLaunchKernelGGL(topk_partial_kernel, dim3(parts, batch), dim3(256), 0, st, d_logits, n, top_k, cv, ci);
    hipLaunchKernelGGL(sample_final_kernel, dim3(batch), dim3(256), 0, st, cv, ci, parts, top_k, temperature, top_p, d_rng, d_tokens);
    return hipGetLastError();
}
