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

#define OXB_LAYER_THREADS 256

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
// Grid (vectors of the pass, parts): every part repeats the reduction (the vector is a few KB in
// L2) and quantises its share of the blocks.  x and w are fetched together, EPT elements per thread.
// The quantiser's exponent does not need the exact maximum, only a bound: |out[i]| <= max|w| * sqrt(h)
// because |x[i]| / rms <= sqrt(h).  With 54-bit fixed point the slack of sqrt(h) costs no mantissa bit
// of any element within 2^22 / sqrt(h) of the largest one.
// ---------------------------------------------------------------------------
template <int FMT, int EPT>
__global__ __launch_bounds__(OXB_LAYER_THREADS) void rmsnorm_quant_kernel(const float* __restrict__ x,
                                                                           const float* __restrict__ w, float eps,
                                                                           float w_absmax, uint32_t h, uint32_t NC,
                                                                           uint32_t* __restrict__ xq,
                                                                           int32_t* __restrict__ cneg,
                                                                           int32_t* __restrict__ xexp,
                                                                           float* __restrict__ normed_out) {
    extern __shared__ float lds_x[];  // [h]
    __shared__ float red[OXB_LAYER_THREADS / 64];
    const uint32_t n = blockIdx.x, tid = threadIdx.x;
    const float* xn = x + (size_t)n * h;
    float xv[EPT], wv[EPT];
#pragma unroll
    for (int e = 0; e < EPT; e++) {
        const uint32_t i = tid + (uint32_t)e * OXB_LAYER_THREADS;
        xv[e] = i < h ? xn[i] : 0.f;
        wv[e] = i < h ? w[i] : 0.f;
    }
    float ss = 0.f;
#pragma unroll
    for (int e = 0; e < EPT; e++) ss = fmaf(xv[e], xv[e], ss);
    ss = block_sum(ss, red);
    const float inv_rms = 1.0f / sqrtf(ss / (float)h + eps);
#pragma unroll
    for (int e = 0; e < EPT; e++) {
        const uint32_t i = tid + (uint32_t)e * OXB_LAYER_THREADS;
        const float v = wv[e] * xv[e] * inv_rms;
        if (i < h) {
            lds_x[i] = v;
            if (normed_out && blockIdx.y == 0) normed_out[(size_t)n * h + i] = v;
        }
    }
    __syncthreads();
    // a NaN or infinity anywhere in x or w shows up in the sum of squares or in the bound
    const float bound = w_absmax * sqrtf((float)h);
    const bool any_bad = oxb_not_finite(ss) || oxb_not_finite(bound);
    quantise_vector<FMT>(lds_x, h, oxb_nblk_pad(h), NC, n, ss > 0.f ? bound : 0.f, any_bad, xq, cneg, xexp, blockIdx.y,
                         gridDim.y);
}

// ---------------------------------------------------------------------------
// SwiGLU fused with the quantiser: act[i] = silu(gate[i]) * up[i], silu(x) = x / (1 + exp(-x))
// (crates/oxibonsai-kernels/src/simd_float_ops.rs:217-236; GPU twin swiglu_fused, cuda_kernels.rs:394-401).
// gu = [gate: inter | up: inter] per vector.  Grid (vectors, parts), 1024 threads.
// ---------------------------------------------------------------------------
#define OXB_SWIGLU_THREADS 1024
template <int FMT>
__global__ __launch_bounds__(OXB_SWIGLU_THREADS) void swiglu_quant_kernel(const float* __restrict__ gu, uint32_t inter,
                                                                           uint32_t NC, uint32_t* __restrict__ xq,
                                                                           int32_t* __restrict__ cneg,
                                                                           int32_t* __restrict__ xexp) {
    extern __shared__ float lds_x[];  // [inter]
    __shared__ float red[OXB_SWIGLU_THREADS / 64];
    __shared__ int bad_flag;
    const uint32_t n = blockIdx.x, tid = threadIdx.x;
    const float* g = gu + (size_t)n * 2 * inter;
    const float* u = g + inter;
    float mx = 0.f;
    int bad = 0;
    for (uint32_t i = tid * 4; i < inter; i += OXB_SWIGLU_THREADS * 4) {  // inter % 128 == 0
        const float4 g4 = *reinterpret_cast<const float4*>(g + i), u4 = *reinterpret_cast<const float4*>(u + i);
        float4 a;
        a.x = (g4.x / (1.0f + expf(-g4.x))) * u4.x;
        a.y = (g4.y / (1.0f + expf(-g4.y))) * u4.y;
        a.z = (g4.z / (1.0f + expf(-g4.z))) * u4.z;
        a.w = (g4.w / (1.0f + expf(-g4.w))) * u4.w;
        *reinterpret_cast<float4*>(lds_x + i) = a;
        bad |= oxb_not_finite(a.x) | oxb_not_finite(a.y) | oxb_not_finite(a.z) | oxb_not_finite(a.w);
        mx = fmaxf(mx, fmaxf(fmaxf(fabsf(a.x), fabsf(a.y)), fmaxf(fabsf(a.z), fabsf(a.w))));
    }
    bool any_bad;
    mx = block_absmax(mx, bad, red, &bad_flag, &any_bad);
    quantise_vector<FMT>(lds_x, inter, oxb_nblk_pad(inter), NC, n, mx, any_bad, xq, cneg, xexp, blockIdx.y, gridDim.y);
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
    const uint32_t pos = p.pos ? p.pos[b] : p.pos_base + b;
    const uint32_t seq = p.pos ? b : p.seq;
    float ss = 0.f;
    for (uint32_t d = tid; d < hd; d += 128) ss += in[d] * in[d];
    ss = block_sum(ss, red);
    const float inv_rms = 1.0f / sqrtf(ss / (float)hd + p.eps);
    const float* cs = p.cos_t + (size_t)pos * half;
    const float* sn = p.sin_t + (size_t)pos * half;
    const size_t cache_off = ((((size_t)seq * p.n_layers + p.layer) * p.nkv + hh) * p.max_seq + pos) * hd;
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
#define OXB_ATTN_CHUNK 128  // KV positions per workgroup

__device__ __forceinline__ void unpack8(const v4i& u, float f[8]) {
    const __half2* h2 = reinterpret_cast<const __half2*>(&u);
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const float2 t = __half22float2(h2[i]);
        f[2 * i] = t.x;
        f[2 * i + 1] = t.y;
    }
}

// HD = head dimension, GM = q heads per kv head rounded up to a power of two (loops over heads are
// unrolled to GM and predicated on the real count G).
template <int HD, int GM>
__global__ __launch_bounds__(OXB_ATTN_THREADS) void attn_decode_kernel(OxbAttnParams p) {
    constexpr int NG = HD / 8;                       // 16-byte groups per row
    constexpr int NSL = OXB_ATTN_THREADS / NG;       // position slices in the weighted-sum phase
    constexpr int PPS = OXB_ATTN_CHUNK / NSL;        // positions per slice
    __shared__ float sc[GM * OXB_ATTN_CHUNK];
    __shared__ float red[GM * 4];
    __shared__ float accs[NSL * GM * HD];
    // blockIdx.y = kv head * nsub + sub: with more than GM q heads per kv head the group is served
    // by nsub workgroups of up to GM heads each
    const uint32_t nsub = gridDim.y / p.nkv, kvh = blockIdx.y / nsub, sub = blockIdx.y % nsub;
    const uint32_t split = blockIdx.x, b = blockIdx.z, tid = threadIdx.x;
    const uint32_t Gall = p.nq / p.nkv, h0 = kvh * Gall + sub * GM;  // first q head served here
    const uint32_t G = (Gall - sub * GM) < (uint32_t)GM ? (Gall - sub * GM) : (uint32_t)GM;
    const uint32_t seq_len = p.pos[b] + 1;
    const uint32_t s0 = split * OXB_ATTN_CHUNK;
    const uint32_t s1 = (s0 + OXB_ATTN_CHUNK) < seq_len ? (s0 + OXB_ATTN_CHUNK) : seq_len;
    float* part = p.part + (((size_t)b * p.nq + h0) * p.n_splits + split) * (HD + 2);
    const size_t part_head = (size_t)p.n_splits * (HD + 2);
    if (s0 >= seq_len) {  // nothing in this chunk: mark it empty for every head of the group
        if (tid < G) {
            part[tid * part_head + HD] = -INFINITY;
            part[tid * part_head + HD + 1] = 0.f;
        }
        return;
    }
    const size_t base = (((size_t)b * p.n_layers + p.layer) * p.nkv + kvh) * p.max_seq * HD;
    const __half* K = p.k_cache + base;
    const __half* V = p.v_cache + base;
    const uint32_t t = s0 + tid;
    const bool live = tid < OXB_ATTN_CHUNK && t < s1;  // the threads that own one position in the softmax phase

    // scores: lanes walk the K rows 16 bytes at a time, so one wave load covers whole rows back to
    // back (fully coalesced); every pass handles RPP rows of the chunk, all passes are in flight at once
    constexpr int RPP = OXB_ATTN_THREADS / NG, NPASS = OXB_ATTN_CHUNK / RPP;
    const uint32_t ch = tid % NG, rr = tid / NG;
    float qf[GM][8];  // this lane's 8 dimensions of every q head
#pragma unroll
    for (int h = 0; h < GM; h++) {
        if ((uint32_t)h < G) {
            const float* qp = p.q + ((size_t)b * p.nq + h0 + h) * HD + ch * 8;
            const float4 qa = *reinterpret_cast<const float4*>(qp), qb = *reinterpret_cast<const float4*>(qp + 4);
            qf[h][0] = qa.x; qf[h][1] = qa.y; qf[h][2] = qa.z; qf[h][3] = qa.w;
            qf[h][4] = qb.x; qf[h][5] = qb.y; qf[h][6] = qb.z; qf[h][7] = qb.w;
        } else {
#pragma unroll
            for (int j = 0; j < 8; j++) qf[h][j] = 0.f;
        }
    }
    // K rows of the score phase and V rows of the weighted-sum phase, all requested now: both depend
    // only on pos.  Buffer loads return 0 past s1 without a branch or a select after the load.
    const __amdgpu_buffer_rsrc_t rk = make_rsrc(K, p.max_seq * HD * 2u), rv = make_rsrc(V, p.max_seq * HD * 2u);
    v4i kreg[NPASS];
#pragma unroll
    for (int i = 0; i < NPASS; i++) {
        const uint32_t tk = s0 + (uint32_t)i * RPP + rr;
        kreg[i] = buf_load_b128(rk, tk < s1 ? (tk * HD + ch * 8u) * 2u : OXB_OOB);
    }
    const uint32_t grp = tid % NG, slice = tid / NG;
    v4i vreg[PPS];
#pragma unroll
    for (int i = 0; i < PPS; i++) {
        const uint32_t tv = s0 + slice + (uint32_t)i * NSL;
        vreg[i] = buf_load_b128(rv, tv < s1 ? (tv * HD + grp * 8u) * 2u : OXB_OOB);
    }
    float lmax[GM];
#pragma unroll
    for (int h = 0; h < GM; h++) lmax[h] = -INFINITY;
#pragma unroll
    for (int i = 0; i < NPASS; i++) {
        float kf[8];
        unpack8(kreg[i], kf);
        const uint32_t lt = (uint32_t)i * RPP + rr;  // position within the chunk
#pragma unroll
        for (int h = 0; h < GM; h++) {
            float d = 0.f;
#pragma unroll
            for (int j = 0; j < 8; j++) d = fmaf(qf[h][j], kf[j], d);
            // add the NG partial sums of the row: they sit in consecutive lanes
            d += dpp_f32<0x111>(d);                    // row_shr:1
            if (NG > 2) d += dpp_f32<0x112>(d);        // row_shr:2
            if (NG > 4) d += dpp_f32<0x114>(d);        // row_shr:4
            if (NG > 8) d += dpp_f32<0x118>(d);        // row_shr:8
            if (NG > 16) d += __shfl_up(d, 16, 64);    // head_dim 256: two 16-lane rows per K row
            if (ch == NG - 1 && (uint32_t)h < G) {
                const float sv = (s0 + lt < s1) ? d * p.scale : -INFINITY;
                sc[h * OXB_ATTN_CHUNK + lt] = sv;
                lmax[h] = fmaxf(lmax[h], sv);
            }
        }
    }
    // chunk maximum per head
    float m[GM];
#pragma unroll
    for (int h = 0; h < GM; h++) {
        float sv = lmax[h];
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) sv = fmaxf(sv, __shfl_xor(sv, o, 64));
        if ((tid & 63u) == 0) red[h * 4 + (tid >> 6)] = sv;
    }
    __syncthreads();  // also publishes the scores
#pragma unroll
    for (int h = 0; h < GM; h++) m[h] = fmaxf(fmaxf(red[h * 4], red[h * 4 + 1]), fmaxf(red[h * 4 + 2], red[h * 4 + 3]));
    __syncthreads();
    // exponentials and their sum: one position per thread
#pragma unroll
    for (int h = 0; h < GM; h++) {
        float e = 0.f;
        if ((uint32_t)h < G) {
            if (tid < OXB_ATTN_CHUNK) {
                e = live ? expf(sc[h * OXB_ATTN_CHUNK + tid] - m[h]) : 0.f;
                sc[h * OXB_ATTN_CHUNK + tid] = e;
            }
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) e += __shfl_xor(e, o, 64);
        if ((tid & 63u) == 0) red[h * 4 + (tid >> 6)] = e;
    }
    __syncthreads();  // publishes the exponentials and the per-wave sums
    // weighted sum of V: thread -> (group of 8 dimensions, slice of positions)
    float acc[GM][8];
#pragma unroll
    for (int h = 0; h < GM; h++)
#pragma unroll
        for (int i = 0; i < 8; i++) acc[h][i] = 0.f;
#pragma unroll
    for (int i = 0; i < PPS; i++) {
        float vf[8];
        unpack8(vreg[i], vf);
        const uint32_t lt = slice + (uint32_t)i * NSL;  // position within the chunk; exponentials past s1 are 0
#pragma unroll
        for (int h = 0; h < GM; h++) {
            if ((uint32_t)h < G) {
                const float pr = sc[h * OXB_ATTN_CHUNK + lt];
#pragma unroll
                for (int j = 0; j < 8; j++) acc[h][j] = fmaf(pr, vf[j], acc[h][j]);
            }
        }
    }
#pragma unroll
    for (int h = 0; h < GM; h++)
        if ((uint32_t)h < G) {
            *reinterpret_cast<float4*>(&accs[(slice * GM + h) * HD + grp * 8]) = make_float4(acc[h][0], acc[h][1], acc[h][2], acc[h][3]);
            *reinterpret_cast<float4*>(&accs[(slice * GM + h) * HD + grp * 8 + 4]) = make_float4(acc[h][4], acc[h][5], acc[h][6], acc[h][7]);
        }
    __syncthreads();
    for (uint32_t i = tid; i < G * HD; i += OXB_ATTN_THREADS) {
        const uint32_t h = i / HD, d = i % HD;
        float v = 0.f;
#pragma unroll
        for (int s = 0; s < NSL; s++) v += accs[(s * GM + h) * HD + d];
        part[h * part_head + d] = v;
    }
    if (tid < G) {
        float mm = m[0];
#pragma unroll
        for (int h = 1; h < GM; h++) mm = (tid == (uint32_t)h) ? m[h] : mm;
        part[tid * part_head + HD] = mm;
        part[tid * part_head + HD + 1] = red[tid * 4] + red[tid * 4 + 1] + red[tid * 4 + 2] + red[tid * 4 + 3];
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
template <int FMT>
static hipError_t launch_rmsnorm_fmt(const float* d_x, const float* d_w, float eps, float w_absmax, uint32_t h,
                                     uint32_t nb, uint32_t* d_xq, int32_t* d_cneg, int32_t* d_xexp, float* d_normed,
                                     hipStream_t st) {
    const size_t shm = (size_t)h * sizeof(float);
    const dim3 grid(nb, oxb_quant_parts(h)), block(OXB_LAYER_THREADS);
    const uint32_t ept = (h + OXB_LAYER_THREADS - 1) / OXB_LAYER_THREADS;
#define OXB_RMS_CASE(E)                                                                                              \
    if (ept <= E) {                                                                                                  \
        hipLaunchKernelGGL((rmsnorm_quant_kernel<FMT, E>), grid, block, shm, st, d_x, d_w, eps, w_absmax, h, 8 * nb, \
                           d_xq, d_cneg, d_xexp, d_normed);                                                          \
        return hipGetLastError();                                                                                    \
    }
    OXB_RMS_CASE(4) OXB_RMS_CASE(8) OXB_RMS_CASE(16) OXB_RMS_CASE(32) OXB_RMS_CASE(64)
#undef OXB_RMS_CASE
    return hipErrorInvalidValue;  // h > 16384
}

hipError_t oxb_launch_rmsnorm_quant(int fmt, const float* d_x, const float* d_w, float eps, float w_absmax, uint32_t h,
                                    uint32_t nb, uint32_t* d_xq, int32_t* d_cneg, int32_t* d_xexp,
                                    float* d_normed_or_null, hipStream_t st) {
    return fmt == OXB_FMT_Q1
               ? launch_rmsnorm_fmt<OXB_FMT_Q1>(d_x, d_w, eps, w_absmax, h, nb, d_xq, d_cneg, d_xexp, d_normed_or_null, st)
               : launch_rmsnorm_fmt<OXB_FMT_TQ2>(d_x, d_w, eps, w_absmax, h, nb, d_xq, d_cneg, d_xexp, d_normed_or_null, st);
}

hipError_t oxb_launch_swiglu_quant(int fmt, const float* d_gu, uint32_t inter, uint32_t nb, uint32_t* d_xq,
                                   int32_t* d_cneg, int32_t* d_xexp, hipStream_t st) {
    const size_t shm = (size_t)inter * sizeof(float);
    const dim3 grid(nb, oxb_quant_parts(inter)), block(OXB_SWIGLU_THREADS);
    if (fmt == OXB_FMT_Q1)
        hipLaunchKernelGGL(swiglu_quant_kernel<OXB_FMT_Q1>, grid, block, shm, st, d_gu, inter, 8 * nb, d_xq, d_cneg, d_xexp);
    else
        hipLaunchKernelGGL(swiglu_quant_kernel<OXB_FMT_TQ2>, grid, block, shm, st, d_gu, inter, 8 * nb, d_xq, d_cneg, d_xexp);
    return hipGetLastError();
}

hipError_t oxb_launch_qk_norm_rope_store(const OxbQkParams& p, uint32_t batch, hipStream_t st) {
    hipLaunchKernelGGL(qk_norm_rope_store_kernel, dim3(p.nq + p.nkv, batch), dim3(128), 0, st, p);
    return hipGetLastError();
}

template <int HD>
static hipError_t launch_attn_hd(const OxbAttnParams& p, uint32_t batch, hipStream_t st) {
    const uint32_t G = p.nq / p.nkv;
    const dim3 block(OXB_ATTN_THREADS);
    if (G == 1) hipLaunchKernelGGL((attn_decode_kernel<HD, 1>), dim3(p.n_splits, p.nkv, batch), block, 0, st, p);
    else if (G == 2) hipLaunchKernelGGL((attn_decode_kernel<HD, 2>), dim3(p.n_splits, p.nkv, batch), block, 0, st, p);
    else hipLaunchKernelGGL((attn_decode_kernel<HD, 4>), dim3(p.n_splits, p.nkv * ((G + 3) / 4), batch), block, 0, st, p);
    return hipGetLastError();
}

hipError_t oxb_launch_attn_decode(const OxbAttnParams& p, uint32_t batch, float* d_out, hipStream_t st) {
    if (p.chunk != OXB_ATTN_CHUNK) return hipErrorInvalidValue;
    hipError_t e;
    switch (p.hd) {
        case 32: e = launch_attn_hd<32>(p, batch, st); break;
        case 64: e = launch_attn_hd<64>(p, batch, st); break;
        case 128: e = launch_attn_hd<128>(p, batch, st); break;
        case 256: e = launch_attn_hd<256>(p, batch, st); break;
        default: return hipErrorInvalidValue;
    }
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(attn_combine_kernel, dim3(p.nq, batch), dim3(p.hd), 0, st, p, d_out);
    return hipGetLastError();
}

hipError_t oxb_launch_argmax(const float* d_logits, uint32_t n, uint32_t batch, uint32_t* d_out, hipStream_t st) {
    hipLaunchKernelGGL(argmax_kernel, dim3(batch), dim3(1024), 0, st, d_logits, n, d_out);
    return hipGetLastError();
}
