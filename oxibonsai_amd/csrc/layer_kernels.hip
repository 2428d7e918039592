// layer_kernels.hip — the Qwen3 layer glue between the quantised GEMVs, for gfx950.
//
// Reference sequence (one decode token, crates/oxibonsai-kernels/src/gpu_backend/
// cuda_full_layer/encode_ternary.rs:142-290, CPU twin crates/oxibonsai-model/src/block/types/forward.rs:92-408):
//   RMSNorm -> QKV GEMV -> per-head QK-RMSNorm + half-split RoPE -> FP16 KV store ->
//   attention over seq_len -> O GEMV + residual -> RMSNorm -> gate||up GEMV -> SiLU(g)*u -> down GEMV + residual.
// Every kernel that produces a GEMV input writes the int8 digit planes directly
// (quant_device.h) instead of an fp32 vector, so no separate quantisation pass runs.
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

#include "layer_kernels.h"
#include "quant_device.h"

#define OXB_LAYER_THREADS 512

__device__ __forceinline__ float block_sum(float v, float* red) {  // two barriers; red: blockDim.x / 64 floats
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    if ((threadIdx.x & 63u) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    float s = 0.f;
    for (uint32_t i = 0; i < (blockDim.x >> 6); i++) s += red[i];
    __syncthreads();
    return s;
}

// ---------------------------------------------------------------------------
// RMSNorm fused with the activation quantiser (rms_norm: crates/oxibonsai-kernels/src/
// simd_float_ops.rs:204-215; GPU twin rmsnorm_weighted_v2, gpu_backend/cuda_kernels.rs:335-374).
// out[i] = w[i] * x[i] * (1 / sqrt(mean(x^2) + eps)); the normalised vector lives only in LDS.
// Grid: one workgroup per vector of the pass.
// ---------------------------------------------------------------------------
template <int FMT>
__global__ __launch_bounds__(OXB_LAYER_THREADS) void rmsnorm_quant_kernel(const float* __restrict__ x,
                                                                           const float* __restrict__ w, float eps,
                                                                           uint32_t h, uint32_t NC,
                                                                           uint32_t* __restrict__ xq,
                                                                           int32_t* __restrict__ cneg,
                                                                           int32_t* __restrict__ xexp,
                                                                           float* __restrict__ normed_out) {
    extern __shared__ float lds_x[];  // [h]
    __shared__ float red[OXB_LAYER_THREADS / 64];
    __shared__ int bad_flag;
    const uint32_t n = blockIdx.x, tid = threadIdx.x;
    const float* xn = x + (size_t)n * h;
    float ss = 0.f;
    for (uint32_t i = tid; i < h; i += OXB_LAYER_THREADS) {
        const float v = xn[i];
        lds_x[i] = v;
        ss += v * v;
    }
    ss = block_sum(ss, red);
    const float inv_rms = 1.0f / sqrtf(ss / (float)h + eps);
    float mx = 0.f;
    int bad = 0;
    for (uint32_t i = tid; i < h; i += OXB_LAYER_THREADS) {
        const float v = w[i] * lds_x[i] * inv_rms;
        lds_x[i] = v;
        if (normed_out) normed_out[(size_t)n * h + i] = v;
        bad |= oxb_not_finite(v);
        mx = fmaxf(mx, fabsf(v));
    }
    bool any_bad;
    mx = block_absmax(mx, bad, red, &bad_flag, &any_bad);  // its barriers also publish lds_x
    quantise_vector<FMT>(lds_x, h, oxb_nblk_pad(h), NC, n, mx, any_bad, xq, cneg, xexp);
}

// ---------------------------------------------------------------------------
// SwiGLU fused with the quantiser: act[i] = silu(gate[i]) * up[i], silu(x) = x / (1 + exp(-x))
// (crates/oxibonsai-kernels/src/simd_float_ops.rs:217-236; GPU twin swiglu_fused, cuda_kernels.rs:394-401).
// gu = [gate: inter | up: inter] per vector.
// ---------------------------------------------------------------------------
template <int FMT>
__global__ __launch_bounds__(OXB_LAYER_THREADS) void swiglu_quant_kernel(const float* __restrict__ gu, uint32_t inter,
                                                                          uint32_t NC, uint32_t* __restrict__ xq,
                                                                          int32_t* __restrict__ cneg,
                                                                          int32_t* __restrict__ xexp) {
    extern __shared__ float lds_x[];  // [inter]
    __shared__ float red[OXB_LAYER_THREADS / 64];
    __shared__ int bad_flag;
    const uint32_t n = blockIdx.x, tid = threadIdx.x;
    const float* g = gu + (size_t)n * 2 * inter;
    const float* u = g + inter;
    float mx = 0.f;
    int bad = 0;
    for (uint32_t i = tid; i < inter; i += OXB_LAYER_THREADS) {
        const float gv = g[i];
        const float v = (gv / (1.0f + expf(-gv))) * u[i];
        lds_x[i] = v;
        bad |= oxb_not_finite(v);
        mx = fmaxf(mx, fabsf(v));
    }
    bool any_bad;
    mx = block_absmax(mx, bad, red, &bad_flag, &any_bad);
    quantise_vector<FMT>(lds_x, inter, oxb_nblk_pad(inter), NC, n, mx, any_bad, xq, cneg, xexp);
}

// ---------------------------------------------------------------------------
// Per-head QK-RMSNorm + half-split RoPE + FP16 KV store
// (fused_qk_norm_rope + fused_kv_store, gpu_backend/cuda_attn_kernels.rs:160-251;
//  CPU: block/types/forward.rs:179-213, rope pairs (d, d + hd/2) simd_float_ops.rs:240-253).
// Grid (nq + nkv, batch); block = 128 threads.  Q heads go to q_rope (fp32), K heads (after RoPE)
// and the raw V head go to the cache at position pos[b], rounded to f16 (round-to-nearest-even).
// Cache layout: [seq][layer][kv_head][max_seq][hd], K and V in separate arrays.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(128) void qk_norm_rope_store_kernel(OxbQkParams p) {
    __shared__ float red[2];
    const uint32_t head = blockIdx.x, b = blockIdx.y, tid = threadIdx.x, hd = p.hd, half = hd >> 1;
    const bool is_q = head < p.nq;
    const uint32_t hh = is_q ? head : head - p.nq;
    const float* in = p.qkv + (size_t)b * p.qkv_stride + (is_q ? (size_t)hh * hd : (size_t)(p.nq + hh) * hd);
    const float* w = is_q ? p.q_norm : p.k_norm;
    const uint32_t pos = p.pos[b];
    float ss = 0.f;
    for (uint32_t d = tid; d < hd; d += 128) ss += in[d] * in[d];
    ss = block_sum(ss, red);
    const float inv_rms = 1.0f / sqrtf(ss / (float)hd + p.eps);
    const float* cs = p.cos_t + (size_t)pos * half;
    const float* sn = p.sin_t + (size_t)pos * half;
    const size_t cache_off = ((((size_t)b * p.n_layers + p.layer) * p.nkv + hh) * p.max_seq + pos) * hd;
    for (uint32_t d = tid; d < half; d += 128) {
        const float lo = w[d] * in[d] * inv_rms, hi = w[d + half] * in[d + half] * inv_rms;
        const float c = cs[d], s = sn[d];
        const float o_lo = lo * c - hi * s, o_hi = lo * s + hi * c;
        if (is_q) {
            float* q = p.q_rope + ((size_t)b * p.nq + hh) * hd;
            q[d] = o_lo;
            q[d + half] = o_hi;
        } else {
            p.k_cache[cache_off + d] = __float2half_rn(o_lo);
            p.k_cache[cache_off + d + half] = __float2half_rn(o_hi);
        }
    }
    if (!is_q) {
        const float* v = p.qkv + (size_t)b * p.qkv_stride + (size_t)(p.nq + p.nkv + hh) * hd;
        for (uint32_t d = tid; d < hd; d += 128) p.v_cache[cache_off + d] = __float2half_rn(v[d]);
    }
}

// ---------------------------------------------------------------------------
// Decode attention, split over the KV sequence (flash-decode).  softmax(q K^T / sqrt(hd)) V with
// GQA (kv_head = q_head / (nq / nkv)) over positions 0..pos[b]
// (batched_attn_scores_v2 / batched_softmax / batched_attn_weighted_sum, cuda_attn_kernels.rs:264-438;
//  CPU: block/functions.rs:78-127 -> layers/attention_fused.rs:329-400).
// Grid (n_splits, nkv, batch), 256 threads.  A workgroup serves all q heads of one kv head for one
// chunk of positions, so K and V are read once per group: scores with one position per thread,
// then the weighted sum with eight head dimensions and a slice of the positions per thread.  It writes the un-normalised partial
// output, the chunk maximum and the chunk sum; attn_combine_kernel merges the chunks.
// ---------------------------------------------------------------------------
#define OXB_ATTN_THREADS 256
#define OXB_ATTN_MAXG 8  // q heads per kv head supported

__global__ __launch_bounds__(OXB_ATTN_THREADS) void attn_decode_kernel(OxbAttnParams p) {
    extern __shared__ float smem[];  // q[G][hd] | sc[G][chunk] | red[G][4] | accs[slices][G][hd]
    const uint32_t split = blockIdx.x, kvh = blockIdx.y, b = blockIdx.z, tid = threadIdx.x;
    const uint32_t hd = p.hd, G = p.nq / p.nkv, chunk = p.chunk;
    const uint32_t seq_len = p.pos[b] + 1;
    const uint32_t s0 = split * chunk;
    const uint32_t s1 = (s0 + chunk) < seq_len ? (s0 + chunk) : seq_len;
    float* part = p.part + (((size_t)b * p.nq + (size_t)kvh * G) * p.n_splits + split) * (hd + 2);
    const size_t part_head = (size_t)p.n_splits * (hd + 2);
    if (s0 >= seq_len) {  // nothing in this chunk: mark it empty for every head of the group
        if (tid < G) {
            part[tid * part_head + hd] = -INFINITY;
            part[tid * part_head + hd + 1] = 0.f;
        }
        return;
    }
    float* q_s = smem;
    float* sc = q_s + G * hd;
    float* red = sc + G * chunk;
    float* accs = red + OXB_ATTN_MAXG * 4;
    for (uint32_t i = tid; i < G * hd; i += OXB_ATTN_THREADS) q_s[i] = p.q[((size_t)b * p.nq + (size_t)kvh * G) * hd + i];
    __syncthreads();
    const size_t base = (((size_t)b * p.n_layers + p.layer) * p.nkv + kvh) * p.max_seq * hd;
    const __half* K = p.k_cache + base;
    const __half* V = p.v_cache + base;

    // scores: one position per thread
    float lmax[OXB_ATTN_MAXG];
#pragma unroll
    for (int h = 0; h < OXB_ATTN_MAXG; h++) lmax[h] = -INFINITY;
    for (uint32_t t = s0 + tid; t < s1; t += OXB_ATTN_THREADS) {
        float dot[OXB_ATTN_MAXG];
#pragma unroll
        for (int h = 0; h < OXB_ATTN_MAXG; h++) dot[h] = 0.f;
        const uint4* kr = reinterpret_cast<const uint4*>(K + (size_t)t * hd);
        for (uint32_t d8 = 0; d8 < hd / 8; d8++) {
            const uint4 kk = kr[d8];
            const __half2* k2 = reinterpret_cast<const __half2*>(&kk);
            float kf[8];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const float2 f = __half22float2(k2[i]);
                kf[2 * i] = f.x;
                kf[2 * i + 1] = f.y;
            }
#pragma unroll
            for (int h = 0; h < OXB_ATTN_MAXG; h++) {
                if ((uint32_t)h < G) {
                    const float* qh = q_s + h * hd + d8 * 8;
#pragma unroll
                    for (int i = 0; i < 8; i++) dot[h] = fmaf(qh[i], kf[i], dot[h]);
                }
            }
        }
#pragma unroll
        for (int h = 0; h < OXB_ATTN_MAXG; h++) {
            if ((uint32_t)h < G) {
                const float s = dot[h] * p.scale;
                sc[h * chunk + (t - s0)] = s;
                lmax[h] = fmaxf(lmax[h], s);
            }
        }
    }
    // chunk maximum per head
#pragma unroll
    for (int h = 0; h < OXB_ATTN_MAXG; h++) {
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) lmax[h] = fmaxf(lmax[h], __shfl_xor(lmax[h], o, 64));
        if ((tid & 63u) == 0) red[h * 4 + (tid >> 6)] = lmax[h];
    }
    __syncthreads();
    float m[OXB_ATTN_MAXG], lsum[OXB_ATTN_MAXG];
#pragma unroll
    for (int h = 0; h < OXB_ATTN_MAXG; h++) {
        m[h] = fmaxf(fmaxf(red[h * 4], red[h * 4 + 1]), fmaxf(red[h * 4 + 2], red[h * 4 + 3]));
        lsum[h] = 0.f;
    }
    __syncthreads();
    // exponentials and their sum
    for (uint32_t t = s0 + tid; t < s1; t += OXB_ATTN_THREADS) {
#pragma unroll
        for (int h = 0; h < OXB_ATTN_MAXG; h++) {
            if ((uint32_t)h < G) {
                const float e = expf(sc[h * chunk + (t - s0)] - m[h]);
                sc[h * chunk + (t - s0)] = e;
                lsum[h] += e;
            }
        }
    }
#pragma unroll
    for (int h = 0; h < OXB_ATTN_MAXG; h++) {
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) lsum[h] += __shfl_xor(lsum[h], o, 64);
        if ((tid & 63u) == 0) red[h * 4 + (tid >> 6)] = lsum[h];
    }
    __syncthreads();  // also publishes the exponentials
    // weighted sum of V: thread -> (group of 8 dimensions, slice of positions); one 16-byte load per position
    const uint32_t n_grp = hd / 8, n_slices = OXB_ATTN_THREADS / n_grp, grp = tid % n_grp, slice = tid / n_grp;
    float acc[OXB_ATTN_MAXG][8];
#pragma unroll
    for (int h = 0; h < OXB_ATTN_MAXG; h++)
#pragma unroll
        for (int i = 0; i < 8; i++) acc[h][i] = 0.f;
#pragma unroll 4
    for (uint32_t t = s0 + slice; t < s1; t += n_slices) {
        const uint4 vv = *reinterpret_cast<const uint4*>(V + (size_t)t * hd + grp * 8);
        const __half2* v2 = reinterpret_cast<const __half2*>(&vv);
        float vf[8];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const float2 f = __half22float2(v2[i]);
            vf[2 * i] = f.x;
            vf[2 * i + 1] = f.y;
        }
#pragma unroll
        for (int h = 0; h < OXB_ATTN_MAXG; h++) {
            if ((uint32_t)h < G) {
                const float pr = sc[h * chunk + (t - s0)];
#pragma unroll
                for (int i = 0; i < 8; i++) acc[h][i] = fmaf(pr, vf[i], acc[h][i]);
            }
        }
    }
#pragma unroll
    for (int h = 0; h < OXB_ATTN_MAXG; h++)
        if ((uint32_t)h < G) {
#pragma unroll
            for (int i = 0; i < 8; i++) accs[(slice * G + h) * hd + grp * 8 + i] = acc[h][i];
        }
    __syncthreads();
    for (uint32_t i = tid; i < G * hd; i += OXB_ATTN_THREADS) {
        float v = 0.f;
        for (uint32_t s = 0; s < n_slices; s++) v += accs[s * G * hd + i];
        part[(i / hd) * part_head + (i % hd)] = v;
    }
    if (tid < G) {
        part[tid * part_head + hd] = m[tid];
        part[tid * part_head + hd + 1] = red[tid * 4] + red[tid * 4 + 1] + red[tid * 4 + 2] + red[tid * 4 + 3];
    }
}

// Merge the chunk results of one q head: grid (nq, batch), hd threads.
__global__ __launch_bounds__(256) void attn_combine_kernel(OxbAttnParams p, float* __restrict__ out) {
    const uint32_t qh = blockIdx.x, b = blockIdx.y, d = threadIdx.x, hd = p.hd;
    const float* part = p.part + ((size_t)b * p.nq + qh) * p.n_splits * (hd + 2);
    const uint32_t used = (p.pos[b] + p.chunk) / p.chunk;  // chunks that hold positions 0..pos
    float M = -INFINITY;
    for (uint32_t s = 0; s < used; s++) M = fmaxf(M, part[(size_t)s * (hd + 2) + hd]);
    float L = 0.f, acc = 0.f;
    for (uint32_t s = 0; s < used; s++) {
        const float* ps = part + (size_t)s * (hd + 2);
        const float wgt = expf(ps[hd] - M);
        L = fmaf(ps[hd + 1], wgt, L);
        acc = fmaf(ps[d], wgt, acc);
    }
    out[((size_t)b * p.nq + qh) * hd + d] = L > 0.f ? acc / L : 0.f;
}

// ---------------------------------------------------------------------------
// Greedy selection: index of the first maximum (strict '>', as argmax_f32, cuda_kernels.rs:407-436).
// One workgroup per vector.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(1024) void argmax_kernel(const float* __restrict__ logits, uint32_t n,
                                                       uint32_t* __restrict__ out) {
    __shared__ float sv[16];
    __shared__ uint32_t si[16];
    const float* v = logits + (size_t)blockIdx.x * n;
    float best = -INFINITY;
    uint32_t idx = 0xFFFFFFFFu;
    for (uint32_t i = threadIdx.x; i < n; i += 1024) {
        const float x = v[i];
        if (idx == 0xFFFFFFFFu || x > best) { best = x; idx = i; }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        const float ob = __shfl_xor(best, o, 64);
        const uint32_t oi = __shfl_xor(idx, o, 64);
        if (ob > best || (ob == best && oi < idx)) { best = ob; idx = oi; }
    }
    if ((threadIdx.x & 63u) == 0) { sv[threadIdx.x >> 6] = best; si[threadIdx.x >> 6] = idx; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < 16; w++)
            if (sv[w] > best || (sv[w] == best && si[w] < idx)) { best = sv[w]; idx = si[w]; }
        out[blockIdx.x] = idx == 0xFFFFFFFFu ? 0u : idx;
    }
}

// ---------------------------------------------------------------------------
// Launchers
// ---------------------------------------------------------------------------
hipError_t oxb_launch_rmsnorm_quant(int fmt, const float* d_x, const float* d_w, float eps, uint32_t h, uint32_t nb,
                                    uint32_t* d_xq, int32_t* d_cneg, int32_t* d_xexp, float* d_normed_or_null,
                                    hipStream_t st) {
    const size_t shm = (size_t)h * sizeof(float);
    if (fmt == OXB_FMT_Q1)
        hipLaunchKernelGGL(rmsnorm_quant_kernel<OXB_FMT_Q1>, dim3(nb), dim3(OXB_LAYER_THREADS), shm, st, d_x, d_w, eps,
                           h, 8 * nb, d_xq, d_cneg, d_xexp, d_normed_or_null);
    else
        hipLaunchKernelGGL(rmsnorm_quant_kernel<OXB_FMT_TQ2>, dim3(nb), dim3(OXB_LAYER_THREADS), shm, st, d_x, d_w,
                           eps, h, 8 * nb, d_xq, d_cneg, d_xexp, d_normed_or_null);
    return hipGetLastError();
}

hipError_t oxb_launch_swiglu_quant(int fmt, const float* d_gu, uint32_t inter, uint32_t nb, uint32_t* d_xq,
                                   int32_t* d_cneg, int32_t* d_xexp, hipStream_t st) {
    const size_t shm = (size_t)inter * sizeof(float);
    if (fmt == OXB_FMT_Q1)
        hipLaunchKernelGGL(swiglu_quant_kernel<OXB_FMT_Q1>, dim3(nb), dim3(OXB_LAYER_THREADS), shm, st, d_gu, inter,
                           8 * nb, d_xq, d_cneg, d_xexp);
    else
        hipLaunchKernelGGL(swiglu_quant_kernel<OXB_FMT_TQ2>, dim3(nb), dim3(OXB_LAYER_THREADS), shm, st, d_gu, inter,
                           8 * nb, d_xq, d_cneg, d_xexp);
    return hipGetLastError();
}

hipError_t oxb_launch_qk_norm_rope_store(const OxbQkParams& p, uint32_t batch, hipStream_t st) {
    hipLaunchKernelGGL(qk_norm_rope_store_kernel, dim3(p.nq + p.nkv, batch), dim3(128), 0, st, p);
    return hipGetLastError();
}

size_t oxb_attn_smem_bytes(uint32_t nq, uint32_t nkv, uint32_t hd, uint32_t chunk) {
    const uint32_t G = nq / nkv, slices = OXB_ATTN_THREADS / (hd / 8);
    return ((size_t)G * hd + (size_t)G * chunk + OXB_ATTN_MAXG * 4 + (size_t)slices * G * hd) * sizeof(float);
}

hipError_t oxb_launch_attn_decode(const OxbAttnParams& p, uint32_t batch, float* d_out, hipStream_t st) {
    hipLaunchKernelGGL(attn_decode_kernel, dim3(p.n_splits, p.nkv, batch), dim3(OXB_ATTN_THREADS),
                       oxb_attn_smem_bytes(p.nq, p.nkv, p.hd, p.chunk), st, p);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(attn_combine_kernel, dim3(p.nq, batch), dim3(p.hd), 0, st, p, d_out);
    return hipGetLastError();
}

hipError_t oxb_launch_argmax(const float* d_logits, uint32_t n, uint32_t batch, uint32_t* d_out, hipStream_t st) {
    hipLaunchKernelGGL(argmax_kernel, dim3(batch), dim3(1024), 0, st, d_logits, n, d_out);
    return hipGetLastError();
}
