// layer_kernels.hip — the Qwen3 layer glue between the quantised GEMVs, for gfx950.
//
// Reference sequence (one decode token, crates/oxibonsai-kernels/src/gpu_backend/
// cuda_full_layer/encode_ternary.rs:142-290, CPU twin crates/oxibonsai-model/src/block/types/forward.rs:92-408):
//   RMSNorm -> QKV GEMV -> per-head QK-RMSNorm + half-split RoPE -> FP16 KV store ->
//   attention over seq_len -> O GEMV + residual -> RMSNorm -> gate||up GEMV -> SiLU(g)*u -> down GEMV + residual.
// RMSNorm, the residual adds and SwiGLU live in the GEMV kernel's prologue and epilogues (gemv_kernels.hip); here
// are the attention kernels, the merge of their slots, the KV row quantiser and the greedy selection.
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

#include <type_traits>

#include "device_utils.h"
#include "kv_quant_device.h"
#include "layer_kernels.h"
#include "gemv_pack_device.h"

// ---------------------------------------------------------------------------
// Per-head QK-RMSNorm + half-split RoPE + KV store (fp16, or quantised rows: kv_quant_device.h)
// (fused_qk_norm_rope + fused_kv_store, gpu_backend/cuda_attn_kernels.rs:160-251;
//  CPU: block/types/forward.rs:179-213, rope pairs (d, d + hd/2) simd_float_ops.rs:240-253).
// Grid (head groups, rows); block = 256 threads = 4 waves, a wave takes OXB_QK_HEADS_PER_WAVE heads of one row one
// after the other: a lane holds the rotation pairs (d, d + hd/2) for d = lane, lane + 64, every reduction stays inside
// the wave.  Q heads go to q_rope (fp32), K heads (after RoPE) and the raw V head go to the cache row of position
// pos[b], rounded to f16 (round-to-nearest-even) or quantised.
// ---------------------------------------------------------------------------
#define OXB_QK_HEADS_PER_WAVE 2
template <int KVM>
__global__ __launch_bounds__(256) void qk_norm_rope_store_kernel(OxbQkParams p) {
    constexpr bool QC = KVM != OXB_KV_F16;
    constexpr int KI = 2, VI = 4;  // pairs / values per lane at head_dim 256
    const uint32_t b = blockIdx.y, lane = threadIdx.x & 63u, hd = p.hd, half = hd >> 1;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const uint32_t pos = p.pos ? p.pos[b] : p.pos_base + b;
    const uint32_t seq = p.pos ? b : p.seq;
    const float* row_in = p.qkv + (size_t)b * p.qkv_stride;
    float cs[KI], sn[KI];
#pragma unroll
    for (int it = 0; it < KI; it++) {
        const uint32_t d = lane + 64 * it;
        cs[it] = d < half ? p.cos_t[(size_t)pos * half + d] : 0.f;
        sn[it] = d < half ? p.sin_t[(size_t)pos * half + d] : 0.f;
    }
    // without a q_rope buffer only the K and V heads are handled (the consumer of Q does its own norm + RoPE)
    const uint32_t first_head = p.q_rope ? 0u : p.nq;
    const uint32_t head0 = first_head + (blockIdx.x * 4 + wave) * OXB_QK_HEADS_PER_WAVE;
#pragma unroll
    for (uint32_t j = 0; j < OXB_QK_HEADS_PER_WAVE; j++) {
        const uint32_t head = head0 + j;
        if (head >= p.nq + p.nkv) break;  // wave-uniform
        const bool is_q = head < p.nq;
        const uint32_t hh = is_q ? head : head - p.nq;
        const float* in = row_in + (size_t)head * hd;  // q heads, then k heads
        const float* w = is_q ? p.q_norm : p.k_norm;
        float lo[KI], hi[KI], ss = 0.f;
#pragma unroll
        for (int it = 0; it < KI; it++) {
            const uint32_t d = lane + 64 * it;
            lo[it] = d < half ? in[d] : 0.f;
            hi[it] = d < half ? in[d + half] : 0.f;
            ss = fmaf(lo[it], lo[it], fmaf(hi[it], hi[it], ss));
        }
        ss = wave_sum_f32(ss);
        const float inv_rms = 1.0f / sqrtf(ss / (float)hd + p.eps);
        float o_lo[KI], o_hi[KI], kmax = 0.f;
#pragma unroll
        for (int it = 0; it < KI; it++) {
            const uint32_t d = lane + 64 * it;
            const float a = d < half ? w[d] * lo[it] * inv_rms : 0.f, c = d < half ? w[d + half] * hi[it] * inv_rms : 0.f;
            o_lo[it] = a * cs[it] - c * sn[it];
            o_hi[it] = a * sn[it] + c * cs[it];
            kmax = fmaxf(kmax, fmaxf(fabsf(o_lo[it]), fabsf(o_hi[it])));
        }
        if (is_q) {
            float* q = p.q_rope + ((size_t)b * p.nq + hh) * hd;
#pragma unroll
            for (int it = 0; it < KI; it++) {
                const uint32_t d = lane + 64 * it;
                if (d < half) q[d] = o_lo[it], q[d + half] = o_hi[it];
            }
            continue;
        }
        const size_t row = kv_row(p.kv, seq, p.layer, hh, pos), cache_off = row * hd;
        const float* v = row_in + (size_t)(p.nq + p.nkv + hh) * hd;
        float vv[VI], vmax = 0.f;
#pragma unroll
        for (int it = 0; it < VI; it++) {
            const uint32_t d = lane + 64 * it;
            vv[it] = d < hd ? v[d] : 0.f;
            vmax = fmaxf(vmax, fabsf(vv[it]));
        }
        if constexpr (QC) {
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) {
                kmax = fmaxf(kmax, __shfl_xor(kmax, o, 64));
                vmax = fmaxf(vmax, __shfl_xor(vmax, o, 64));
            }
            const float ks = kv_row_scale<KVM>(kmax), vs = kv_row_scale<KVM>(vmax);
            uint8_t* kc = reinterpret_cast<uint8_t*>(p.k_cache) + cache_off;
            uint8_t* vc = reinterpret_cast<uint8_t*>(p.v_cache) + cache_off;
#pragma unroll
            for (int it = 0; it < KI; it++) {
                const uint32_t d = lane + 64 * it;
                if (d < half) {
                    kc[d] = (uint8_t)kv_encode<KVM>(o_lo[it], ks);
                    kc[d + half] = (uint8_t)kv_encode<KVM>(o_hi[it], ks);
                }
            }
#pragma unroll
            for (int it = 0; it < VI; it++) {
                const uint32_t d = lane + 64 * it;
                if (d < hd) vc[d] = (uint8_t)kv_encode<KVM>(vv[it], vs);
            }
            if (lane == 0) {
                p.k_scale[row] = ks;
                p.v_scale[row] = vs;
            }
        } else {
            __half* kc = reinterpret_cast<__half*>(p.k_cache) + cache_off;
            __half* vc = reinterpret_cast<__half*>(p.v_cache) + cache_off;
#pragma unroll
            for (int it = 0; it < KI; it++) {
                const uint32_t d = lane + 64 * it;
                if (d < half) {
                    kc[d] = __float2half_rn(o_lo[it]);
                    kc[d + half] = __float2half_rn(o_hi[it]);
                }
            }
#pragma unroll
            for (int it = 0; it < VI; it++) {
                const uint32_t d = lane + 64 * it;
                if (d < hd) vc[d] = __float2half_rn(vv[it]);
            }
        }
    }
}

// Rows of f32 values -> quantised cache rows (codes + scale), one wave per row; the arithmetic of the attention
// kernels' own stores, exposed for callers that fill a cache themselves and for tests.
template <int KVM>
__global__ __launch_bounds__(64) void kv_quantize_rows_kernel(const float* __restrict__ x, uint32_t n, uint8_t* __restrict__ codes,
                                                               float* __restrict__ scales) {
    const float* row = x + (size_t)blockIdx.x * n;
    float mx = 0.f;
    for (uint32_t d = threadIdx.x; d < n; d += 64) mx = fmaxf(mx, fabsf(row[d]));
    mx = wave_max_f32(mx);
    const float scale = kv_row_scale<KVM>(mx);
    for (uint32_t d = threadIdx.x; d < n; d += 64) codes[(size_t)blockIdx.x * n + d] = (uint8_t)kv_encode<KVM>(row[d], scale);
    if (threadIdx.x == 0) scales[blockIdx.x] = scale;
}

// Quantised rows back to f32 as attention reads them, code * scale (dequantize_row, kv_cache_quant.rs:69-71, 545-556):
// the codes are widened four at a time by the routine the attention kernels use (kv_dec4), which is what this is for.
template <int KVM>
__global__ __launch_bounds__(256) void kv_dequantize_rows_kernel(const uint32_t* __restrict__ codes4, const float* __restrict__ scales,
                                                                 uint32_t n, uint64_t total4, float* __restrict__ out) {
    const uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x;  // one dword of four codes; n % 4 == 0
    if (i >= total4) return;
    uint32_t lo, hi;
    kv_dec4<KVM>(codes4[i], lo, hi);
    const kvh2_t a = __builtin_bit_cast(kvh2_t, lo), b = __builtin_bit_cast(kvh2_t, hi);
    const float sc = scales[(i * 4) / n];
    out[i * 4 + 0] = (float)a[0] * sc;
    out[i * 4 + 1] = (float)a[1] * sc;
    out[i * 4 + 2] = (float)b[0] * sc;
    out[i * 4 + 3] = (float)b[1] * sc;
}

hipError_t oxb_launch_kv_dequantize_rows(int kv_mode, const uint8_t* d_codes, const float* d_scales, uint32_t n_rows, uint32_t n,
                                         float* d_out, hipStream_t st) {
    if (n_rows == 0 || n == 0 || (n & 3u)) return hipErrorInvalidValue;
    const uint64_t total4 = (uint64_t)n_rows * n / 4;
    const dim3 grid((uint32_t)((total4 + 255) / 256));
    if (kv_mode == OXB_KV_I8)
        hipLaunchKernelGGL(kv_dequantize_rows_kernel<OXB_KV_I8>, grid, dim3(256), 0, st, (const uint32_t*)d_codes, d_scales, n, total4, d_out);
    else if (kv_mode == OXB_KV_FP8_E4M3)
        hipLaunchKernelGGL(kv_dequantize_rows_kernel<OXB_KV_FP8_E4M3>, grid, dim3(256), 0, st, (const uint32_t*)d_codes, d_scales, n, total4, d_out);
    else return hipErrorInvalidValue;
    return hipGetLastError();
}

hipError_t oxb_launch_kv_quantize_rows(int kv_mode, const float* d_x, uint32_t n_rows, uint32_t n, uint8_t* d_codes, float* d_scales,
                                       hipStream_t st) {
    if (n_rows == 0 || n == 0) return hipErrorInvalidValue;
    if (kv_mode == OXB_KV_I8) hipLaunchKernelGGL(kv_quantize_rows_kernel<OXB_KV_I8>, dim3(n_rows), dim3(64), 0, st, d_x, n, d_codes, d_scales);
    else if (kv_mode == OXB_KV_FP8_E4M3)
        hipLaunchKernelGGL(kv_quantize_rows_kernel<OXB_KV_FP8_E4M3>, dim3(n_rows), dim3(64), 0, st, d_x, n, d_codes, d_scales);
    else return hipErrorInvalidValue;
    return hipGetLastError();
}

#define OXB_ATTN_CHUNK 128  // KV positions per chunk of the split-KV decode attention

// ---------------------------------------------------------------------------
// Decode attention, split over the KV sequence (flash-decode), on the matrix cores: softmax(q K^T / sqrt(hd)) V
// with GQA (kv_head = q_head / (nq / nkv)) over positions 0..pos[b]
// (batched_attn_scores_v2 / batched_softmax / batched_attn_weighted_sum, cuda_attn_kernels.rs:264-438;
//  CPU: block/functions.rs:78-127 -> layers/attention_fused.rs:329-400), fused with what precedes it in the layer:
// per-head QK-RMSNorm, RoPE and the FP16 store of the new position's K and V (fused_qk_norm_rope + fused_kv_store,
// cuda_attn_kernels.rs:160-251).  Grid (n_splits, nkv, batch), 256 threads = 4 waves.  It writes, per q head and
// slot, the un-normalised partial output, the running maximum and the running sum; the last workgroup of a
// (sequence, kv head) to finish merges the slots (attn_last_arrival, attn_merge_heads).
// A workgroup serves all q heads of one kv head (<= 16, the columns of the MFMA tiles) for one slot of the KV
// sequence: slot s walks chunks s, s + n_splits, ... of 128 positions, wave w takes keys [32w, 32w + 32) of each.
//   S^T[key][head] = sum_d K[key][d] Q[head][d]     A = K rows straight from the cache, B = Q * scale as fp16 hi + lo
//   O^T[d][head]  += sum_key V[key][d] P[head][key]  A = V gathered from the wave's LDS copy of the block,
//                                                    B = the lane's own probabilities as fp16 hi + lo
// so scores and weighted sums keep fp32-level accuracy.  Every wave runs its own online softmax; the four results
// meet in LDS.  The workgroup whose slot holds the new position computes K (norm + RoPE) and V of that position,
// stores them to the cache and, after a barrier, reads them back like any other row.
// ---------------------------------------------------------------------------
typedef _Float16 v8h_t __attribute__((ext_vector_type(8)));

// Options of the kernel (template KVM, fields window / sinks):
//  * quantised cache rows (kv_quant_device.h): one byte per value plus an f32 scale per row.  The codes enter the
//    matrix cores as exact fp16 numbers; the K row scale multiplies the score, the V row scale the probability
//    (relative to a running largest scale `u`, so that the fp16 hi + lo pair of the product stays in range; the
//    accumulator is kept in units of u and rescaled like the running maximum of the softmax).  A lane takes a
//    contiguous quarter of a K row (hd / 4 bytes), so the Q operand follows that order.
//  * sliding window with attention sinks (is_in_window, crates/oxibonsai-model/src/layers/sliding_window.rs:173-189):
//    the first `sinks` keys stay visible, the others while pos - key < window - sinks; chunks without a visible key
//    are not walked.  window == 0: every key up to pos is visible.
#define OXB_ATTN_MERGE_LDS_BYTES(heads_per) ((heads_per) * 65 * 4 + 12 + 256 * 16)  // LDS attn_merge_heads needs
__device__ __forceinline__ void attn_merge_heads(const OxbAttnParams& p, uint32_t b, uint32_t h_first, uint32_t nh, uint32_t heads_per,
                                                 float* sm, float* __restrict__ out);

// The workgroups of one (sequence, kv head) count themselves off once their slot results are written; the last one
// to arrive merges the slots of the group's heads into the attention output, so that no second launch is needed.
// The counter returns to 0 for the next launch.  The slot results travel between workgroups (other CUs, other XCDs)
// through agent-coherent stores and loads: every store of this workgroup has been acknowledged by memory before its
// count is added, and the merge's loads bypass the caches that another workgroup's stores do not reach.
__device__ __forceinline__ bool attn_last_arrival(const OxbAttnParams& p, uint32_t b, uint32_t kvh, uint32_t expected, uint32_t* flag) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (threadIdx.x == 0) {
        uint32_t* ctr = p.done + (size_t)b * p.nkv + kvh;
        const uint32_t prev = atomicAdd(ctr, 1u);
        const uint32_t last = prev + 1u == expected ? 1u : 0u;
        if (last) atomicExch(ctr, 0u);
        *flag = last;
    }
    __syncthreads();
    return *flag != 0u;
}

template <int HD, int KVM, bool OPT>  // OPT: a window and / or a paged cache may be in use (else neither costs anything)
__global__ __launch_bounds__(256) void attn_decode_fused_kernel(OxbAttnParams p) {
    constexpr bool QC = KVM != OXB_KV_F16;
    constexpr int KS = HD / 32, NS = HD / 16, VSTR = HD + 8;
    constexpr int VPR = QC ? HD / 16 : HD / 8;  // 16-byte pieces per V row
    constexpr int VL = 32 * VPR / 64;           // pieces of the wave's 32-row V block per lane
    // V block per wave; after the loop the merge buffers.  Q * scale of the group's heads has an area of its own, so
    // that a wave whose Q operands are in registers starts staging V without waiting for the others.
    __shared__ __attribute__((aligned(16))) _Float16 vs_all[4][32 * VSTR];
    __shared__ __attribute__((aligned(16))) _Float16 qs[2][16 * HD];  // fp16 hi and lo parts, as the B operands take them
    __shared__ uint32_t last_flag;
    __shared__ __attribute__((aligned(16))) _Float16 kv_new[2][HD];  // the new position's K and V rows as stored (fp16 cache)
    static_assert(sizeof(vs_all) >= OXB_ATTN_MERGE_LDS_BYTES(16), "the merge's slot weights and partial sums must fit in the V slices");
    const uint32_t tid = threadIdx.x, lane = tid & 63u, qi = lane & 15u, g = lane >> 4;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
    const uint32_t slot = blockIdx.x, kvh = blockIdx.y, b = blockIdx.z;
    const uint32_t G = p.nq / p.nkv, h0 = kvh * G, half = HD / 2;
    const uint32_t pos = p.pos[b], seq_len = pos + 1;
    const uint32_t n_chunks = (seq_len + OXB_ATTN_CHUNK - 1) / OXB_ATTN_CHUNK;
    if (slot >= n_chunks) return;  // never read by the merge
    // visible keys: [0, sink_n) and [lo, seq_len)
    const uint32_t window = OPT ? p.window : 0u;
    const uint32_t budget = window > p.sinks ? window - p.sinks : 0u;
    const uint32_t lo = window ? (seq_len > budget ? seq_len - budget : 0u) : 0u;
    const uint32_t sink_n = window ? min(p.sinks, seq_len) : 0u;
    const uint32_t sink_chunks = (sink_n + OXB_ATTN_CHUNK - 1) / OXB_ATTN_CHUNK, lo_chunk = lo / OXB_ATTN_CHUNK;
    auto next_needed = [&](uint32_t c) {  // first chunk >= c of this slot's walk that holds a visible key
        if (c >= sink_chunks && c < lo_chunk) c += (lo_chunk - c + p.n_splits - 1) / p.n_splits * p.n_splits;
        return c;
    };
    const bool owner = (pos / OXB_ATTN_CHUNK) % p.n_splits == slot;  // this workgroup stores the new position
    const uint32_t first = next_needed(slot);
    float* part = p.part + (((size_t)b * p.nq + h0) * p.n_splits + slot) * (HD + OXB_ATTN_PART_PAD);
    const size_t part_head = (size_t)p.n_splits * (HD + OXB_ATTN_PART_PAD);
    // slot results go out through agent-coherent stores: a workgroup of this same launch merges them
    const __amdgpu_buffer_rsrc_t r_out = make_rsrc(part, (uint32_t)(G * part_head * 4u));
    auto put = [&](size_t idx, float v) { buf_store_b32_coherent(r_out, (uint32_t)idx * 4u, v); };
    if (first >= n_chunks && !owner) {  // nothing visible in this slot's chunks: an empty result for the merge
        for (uint32_t i = tid; i < G * HD; i += 256) {
            const uint32_t h = i / HD, d = i % HD;
            put(h * part_head + d, 0.f);
            if (d == 0) {
                put(h * part_head + HD, -INFINITY);
                put(h * part_head + HD + 1, 0.f);
            }
        }
        if (attn_last_arrival(p, b, kvh, min(n_chunks, p.n_splits), &last_flag))
            attn_merge_heads(p, b, h0, G, G, reinterpret_cast<float*>(&vs_all[0][0]), p.out_merged);
        return;
    }
    const float* qkv = p.qkv + (size_t)b * p.qkv_stride;
    const float* cs = p.cos_t + (size_t)pos * half;
    const float* sn = p.sin_t + (size_t)pos * half;
    typedef typename std::conditional<QC, uint8_t, _Float16>::type cache_t;
    cache_t* Kc = reinterpret_cast<cache_t*>(p.k_cache);
    cache_t* Vc = reinterpret_cast<cache_t*>(p.v_cache);
    float* Ksc = p.k_scale;  // one scale per row
    float* Vsc = p.v_scale;
    // Row of a position of this (sequence, layer, kv head): an offset in a contiguous cache; in a paged one the page
    // number comes from the sequence's table.  Pages hold 16 positions or more, so the 32 keys of a wave's block lie in
    // at most two pages - those of keys key0 .. key0 + 15 and key0 + 16 .. key0 + 31, the same for every lane - which
    // are looked up (one broadcast load each) one chunk before the rows are requested, so that no row load waits for
    // a lookup.  (Keeping the table in LDS instead was measured slower: the 8 KB cost a workgroup per CU.)
    const bool paged = OPT && p.kv.page_table != nullptr;
    const uint32_t pshift = p.kv.page_shift, pmask = (1u << pshift) - 1u;
    const size_t row0 = paged ? ((size_t)(p.layer * p.nkv + kvh) * p.kv.n_pages) << pshift : kv_row(p.kv, b, p.layer, kvh, 0);
    const uint32_t* tbl = paged ? p.kv.page_table + (size_t)b * p.kv.table_stride : nullptr;  // covers whole chunks
    auto pages_of = [&](uint32_t chunk, uint32_t& pa, uint32_t& pb) {
        pa = pb = 0;
        if (!paged) return;
        const uint32_t key0 = chunk * OXB_ATTN_CHUNK + 32 * wave, i0 = key0 >> pshift, i1 = (key0 + 16) >> pshift;
        pa = (uint32_t)__builtin_amdgcn_readfirstlane((int)tbl[i0]);
        pb = (uint32_t)__builtin_amdgcn_readfirstlane((int)tbl[i1]);
    };
    // key: a position of the block that starts at key0 (or, for a block past the end, the last position, whose row
    // is then read from a wrong but existing page: such a block is masked as a whole)
    auto row_of = [&](uint32_t key, uint32_t key0, uint32_t pa, uint32_t pb) -> size_t {
        if (!paged) return row0 + key;
        return row0 + ((size_t)(((key - key0) & 16u) ? pb : pa) << pshift) + (key & pmask);
    };

    // K rows of the two 16-key tiles (A operands) and this lane's pieces of the 32-key V block of a chunk.
    // Rows past the last key repeat it; their scores are masked.
    v8h_t k0r[QC ? 1 : KS], k1r[QC ? 1 : KS];
    kvi2_t k0q[QC ? KS : 1], k1q[QC ? KS : 1];
    float4 ksc0, ksc1, vsc0, vsc1;  // row scales of the lane's keys 4g .. 4g+3 and 16+4g .. 16+4g+3
    v4i vr[VL];
    auto load_k = [&](uint32_t chunk, uint32_t pa, uint32_t pb) {
        const uint32_t key0 = chunk * OXB_ATTN_CHUNK + 32 * wave;
        const size_t kr0 = row_of(min(key0 + qi, seq_len - 1), key0, pa, pb), kr1 = row_of(min(key0 + 16 + qi, seq_len - 1), key0, pa, pb);
#pragma unroll
        for (int s = 0; s < KS; s++) {
            if constexpr (QC) {
                k0q[s] = *reinterpret_cast<const kvi2_t*>(Kc + kr0 * HD + (HD / 4) * g + 8 * s);
                k1q[s] = *reinterpret_cast<const kvi2_t*>(Kc + kr1 * HD + (HD / 4) * g + 8 * s);
            } else {
                k0r[s] = *reinterpret_cast<const v8h_t*>(Kc + kr0 * HD + 32 * s + 8 * g);
                k1r[s] = *reinterpret_cast<const v8h_t*>(Kc + kr1 * HD + 32 * s + 8 * g);
            }
        }
        if constexpr (QC) {  // scales of positions past the last key are never used (their scores are masked)
            ksc0 = *reinterpret_cast<const float4*>(Ksc + row_of(min(key0 + 4 * g, (seq_len - 1) & ~3u), key0, pa, pb));
            ksc1 = *reinterpret_cast<const float4*>(Ksc + row_of(min(key0 + 16 + 4 * g, (seq_len - 1) & ~3u), key0, pa, pb));
        }
    };
    auto load_v = [&](uint32_t chunk, uint32_t pa, uint32_t pb) {
        const uint32_t key0 = chunk * OXB_ATTN_CHUNK + 32 * wave;
#pragma unroll
        for (int i = 0; i < VL; i++) {
            const uint32_t id = i * 64 + lane, col = id % VPR;
            const size_t row = row_of(min(key0 + id / VPR, seq_len - 1), key0, pa, pb);
            vr[i] = *reinterpret_cast<const v4i*>(reinterpret_cast<const uint8_t*>(Vc + row * HD) + col * 16);
        }
        if constexpr (QC) {
            vsc0 = *reinterpret_cast<const float4*>(Vsc + row_of(min(key0 + 4 * g, (seq_len - 1) & ~3u), key0, pa, pb));
            vsc1 = *reinterpret_cast<const float4*>(Vsc + row_of(min(key0 + 16 + 4 * g, (seq_len - 1) & ~3u), key0, pa, pb));
        }
    };

    // With an fp16 cache the rows of the first chunk are requested before anything else, so that their way from HBM
    // overlaps the Q prologue.  In the workgroup that stores the new position that row is not in the cache yet (and
    // rows past the end repeat it): it is patched in from LDS below, with the very values the cache receives.
    // With a quantised cache there is no such patch: every workgroup requests early except the one whose first chunk
    // holds the new position, which waits until its own stores of that row have landed.
    constexpr bool EARLY = !QC;
    const uint32_t pos_chunk = pos / OXB_ATTN_CHUNK;
    const bool early = EARLY || !(owner && pos_chunk == first);  // (the same for the whole workgroup)
    uint32_t na = 0, nb = 0;  // pages of the chunk whose rows are requested next
    auto request_first = [&]() {
        if (first < n_chunks) {
            uint32_t pa, pb;
            pages_of(first, pa, pb);
            load_k(first, pa, pb);
            load_v(first, pa, pb);
            const uint32_t second = next_needed(first + p.n_splits);
            if (second < n_chunks) pages_of(second, na, nb);
        }
    };
    // Inputs of the prologue, requested before the cache rows: loads return in issue order, so whatever the prologue
    // waits for must not queue behind the rows from HBM.  Lane d holds elements d and d + hd/2 of a head (the RoPE pair).
    constexpr int KI = (HD / 2 + 63) / 64;
    struct HeadIn { float lo[KI], hi[KI]; };
    auto load_head = [&](const float* in, HeadIn& r) {
#pragma unroll
        for (int it = 0; it < KI; it++) {
            const uint32_t d = lane + 64 * it;
            r.lo[it] = d < half ? in[d] : 0.f;
            r.hi[it] = d < half ? in[d + half] : 0.f;
        }
    };
    // sum of squares in the order of a strided walk over the head (all low halves, then all high halves)
    auto head_inv_rms = [&](const HeadIn& r) {
        float ss = 0.f;
#pragma unroll
        for (int it = 0; it < KI; it++) ss = fmaf(r.lo[it], r.lo[it], ss);
#pragma unroll
        for (int it = 0; it < KI; it++) ss = fmaf(r.hi[it], r.hi[it], ss);
        ss = wave_sum_f32(ss);
        return 1.0f / sqrtf(ss / (float)HD + p.eps);
    };
    HeadIn q_in, cs_sn, qn, kv_in, kn;  // cs_sn: lo = cos, hi = sin; kv_in: the new K row (wave 0) or V row (wave 1) of the owner
    {
#pragma unroll
        for (int it = 0; it < KI; it++) {
            const uint32_t d = lane + 64 * it;
            cs_sn.lo[it] = d < half ? cs[d] : 0.f;
            cs_sn.hi[it] = d < half ? sn[d] : 0.f;
        }
        load_head(p.q_norm, qn);
        if (wave < G) load_head(qkv + (size_t)(h0 + wave) * HD, q_in);
        if (owner && wave == 0) {
            load_head(qkv + (size_t)(p.nq + kvh) * HD, kv_in);
            load_head(p.k_norm, kn);
        } else if (owner && wave == 1) {
            load_head(qkv + (size_t)(p.nq + p.nkv + kvh) * HD, kv_in);
        }
    }
    __builtin_amdgcn_sched_barrier(0);
    if (early) request_first();
    __builtin_amdgcn_sched_barrier(0);
    // --- Q of the group's heads: RMSNorm over the head, RoPE on the pairs (d, d + hd/2), times 1/sqrt(hd) ---
    for (uint32_t h = wave; h < G; h += 4) {
        if (h != wave) load_head(qkv + (size_t)(h0 + h) * HD, q_in);
        const float inv = head_inv_rms(q_in);
#pragma unroll
        for (int it = 0; it < KI; it++) {
            const uint32_t d = lane + 64 * it;
            if (d < half) {
                const float lo_ = qn.lo[it] * q_in.lo[it] * inv, hi_ = qn.hi[it] * q_in.hi[it] * inv;
                // split into fp16 hi + lo here, once per value (not once per lane that reads it)
                const float qa = (lo_ * cs_sn.lo[it] - hi_ * cs_sn.hi[it]) * p.scale, qb = (lo_ * cs_sn.hi[it] + hi_ * cs_sn.lo[it]) * p.scale;
                const _Float16 ha = (_Float16)qa, hb = (_Float16)qb;
                qs[0][h * HD + d] = ha;
                qs[1][h * HD + d] = (_Float16)(qa - (float)ha);
                qs[0][h * HD + d + half] = hb;
                qs[1][h * HD + d + half] = (_Float16)(qb - (float)hb);
            }
        }
    }
    // --- K and V of the new position, by the workgroup whose slot walks its chunk (wave 0 and wave 1) ---
    const size_t new_row = kv_row(p.kv, b, p.layer, kvh, pos);
    if (owner) {
        if (wave == 0) {
            const float inv = head_inv_rms(kv_in);
            float klo[KI], khi[KI], mx = 0.f;
#pragma unroll
            for (int it = 0; it < KI; it++) {
                const uint32_t d = lane + 64 * it;
                klo[it] = khi[it] = 0.f;
                if (d < half) {
                    const float lo_ = kn.lo[it] * kv_in.lo[it] * inv, hi_ = kn.hi[it] * kv_in.hi[it] * inv;
                    klo[it] = lo_ * cs_sn.lo[it] - hi_ * cs_sn.hi[it];
                    khi[it] = lo_ * cs_sn.hi[it] + hi_ * cs_sn.lo[it];
                    mx = fmaxf(mx, fmaxf(fabsf(klo[it]), fabsf(khi[it])));
                }
            }
            float scale = 1.f;
            if constexpr (QC) {
                mx = wave_max_f32(mx);
                scale = kv_row_scale<KVM>(mx);
                if (lane == 0) Ksc[new_row] = scale;
            }
#pragma unroll
            for (int it = 0; it < KI; it++) {
                const uint32_t d = lane + 64 * it;
                if (d < half) {
                    if constexpr (QC) {
                        Kc[new_row * HD + d] = (uint8_t)kv_encode<KVM>(klo[it], scale);
                        Kc[new_row * HD + d + half] = (uint8_t)kv_encode<KVM>(khi[it], scale);
                    } else {
                        Kc[new_row * HD + d] = kv_new[0][d] = (_Float16)klo[it];
                        Kc[new_row * HD + d + half] = kv_new[0][d + half] = (_Float16)khi[it];
                    }
                }
            }
        } else if (wave == 1) {
            float mx = 0.f;
#pragma unroll
            for (int it = 0; it < KI; it++) mx = fmaxf(mx, fmaxf(fabsf(kv_in.lo[it]), fabsf(kv_in.hi[it])));
            float scale = 1.f;
            if constexpr (QC) {
                mx = wave_max_f32(mx);
                scale = kv_row_scale<KVM>(mx);
                if (lane == 0) Vsc[new_row] = scale;
            }
#pragma unroll
            for (int it = 0; it < KI; it++) {
                const uint32_t d = lane + 64 * it;
                if (d < half) {
                    if constexpr (QC) {
                        Vc[new_row * HD + d] = (uint8_t)kv_encode<KVM>(kv_in.lo[it], scale);
                        Vc[new_row * HD + d + half] = (uint8_t)kv_encode<KVM>(kv_in.hi[it], scale);
                    } else {
                        Vc[new_row * HD + d] = kv_new[1][d] = (_Float16)kv_in.lo[it];
                        Vc[new_row * HD + d + half] = kv_new[1][d + half] = (_Float16)kv_in.hi[it];
                    }
                }
            }
        }
    }
    // publishes qs and the LDS copy of the new rows.  The requested cache rows stay in flight across it, unless this
    // workgroup will read the new position's rows back from the cache (requests after the prologue, or a walk of
    // several chunks that ends in the new position's): then the stores must have landed first.
    if (owner && !(EARLY && pos_chunk == first)) __syncthreads();
    else lds_barrier();
    if (!early) request_first();

    // B operands: lane (head = qi, g) holds the eight Q values that meet its K values in step s, as hi + lo: one
    // 16-byte LDS read each.  Columns past the group's heads repeat head 0; nothing of them is ever stored.
    v8h_t qh[KS], ql[KS];
    const uint32_t hq = qi < G ? qi : 0u;
#pragma unroll
    for (int s = 0; s < KS; s++) {
        const uint32_t d = QC ? (HD / 4) * g + 8 * s : 32 * s + 8 * g;
        qh[s] = *reinterpret_cast<const v8h_t*>(&qs[0][hq * HD + d]);
        ql[s] = *reinterpret_cast<const v8h_t*>(&qs[1][hq * HD + d]);
    }
    v4f O[NS];
#pragma unroll
    for (int i = 0; i < NS; i++) O[i] = (v4f){0.f, 0.f, 0.f, 0.f};
    float m_run = -INFINITY, l_run = 0.f, u_run = QC ? 0.f : 1.f;  // u_run: the unit of O (largest V row scale so far)
    _Float16* vs = vs_all[wave];

    for (uint32_t chunk = first; chunk < n_chunks;) {
        const uint32_t key0 = chunk * OXB_ATTN_CHUNK + 32 * wave;
        const uint32_t nxt = next_needed(chunk + p.n_splits);
        const bool more = nxt < n_chunks;
        // rows of the new position (and the repeats of it past the end) come from LDS where they were requested early
        const bool patch = EARLY && owner && chunk == pos_chunk && chunk == first;
        chunk = nxt;
        // stage the V block in the wave's LDS slice (the previous block's gathers were issued before: LDS runs in
        // order) and request the next chunk's
#pragma unroll
        for (int i = 0; i < VL; i++) {
            const uint32_t id = i * 64 + lane;
            if constexpr (QC) {
                uint32_t d[8];
                kv_dec4<KVM>((uint32_t)vr[i].x, d[0], d[1]);
                kv_dec4<KVM>((uint32_t)vr[i].y, d[2], d[3]);
                kv_dec4<KVM>((uint32_t)vr[i].z, d[4], d[5]);
                kv_dec4<KVM>((uint32_t)vr[i].w, d[6], d[7]);
                _Float16* dst = vs + (id / VPR) * VSTR + (id % VPR) * 16;
                *reinterpret_cast<v4i*>(dst) = (v4i){(int)d[0], (int)d[1], (int)d[2], (int)d[3]};
                *reinterpret_cast<v4i*>(dst + 8) = (v4i){(int)d[4], (int)d[5], (int)d[6], (int)d[7]};
            } else {
                v4i piece = vr[i];
                if (patch && key0 + id / VPR >= pos) piece = *reinterpret_cast<const v4i*>(&kv_new[1][(id % VPR) * 8]);
                *reinterpret_cast<v4i*>(vs + (id / VPR) * VSTR + (id % VPR) * 8) = piece;
            }
        }
        const float4 vc0 = vsc0, vc1 = vsc1;
        if (more) load_v(nxt, na, nb);
        v4f s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < KS; s++) {
            v8h_t a0, a1;
            if constexpr (QC) {
                a0 = kv_dec8<KVM>(k0q[s]);
                a1 = kv_dec8<KVM>(k1q[s]);
            } else {
                a0 = k0r[s];
                a1 = k1r[s];
                if (patch) {
                    if (key0 + qi >= pos) a0 = *reinterpret_cast<const v8h_t*>(&kv_new[0][32 * s + 8 * g]);
                    if (key0 + 16 + qi >= pos) a1 = *reinterpret_cast<const v8h_t*>(&kv_new[0][32 * s + 8 * g]);
                }
            }
            s0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(a0, qh[s], s0, 0, 0, 0);
            s0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(a0, ql[s], s0, 0, 0, 0);
            s1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(a1, qh[s], s1, 0, 0, 0);
            s1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(a1, ql[s], s1, 0, 0, 0);
        }
        const float4 kc0 = ksc0, kc1 = ksc1;
        if (more) {
            load_k(nxt, na, nb);
            const uint32_t after = next_needed(nxt + p.n_splits);
            if (after < n_chunks) pages_of(after, na, nb);  // used by the next iteration's requests
        }
        // this wave's quarter of the chunk holds no visible key (past the end, or outside the window)
        if (!(key0 < sink_n || max(key0, lo) < min(key0 + 32, seq_len))) continue;
        // this lane: head qi, keys key0 + 4g + v and key0 + 16 + 4g + v
        float sv[8];
        bool vis[8];
        float mx = -INFINITY;
#pragma unroll
        for (int v = 0; v < 4; v++) {
            const uint32_t ka = key0 + 4 * g + v, kb = ka + 16;
            vis[v] = ka < sink_n || (ka >= lo && ka < seq_len);
            vis[4 + v] = kb < sink_n || (kb >= lo && kb < seq_len);
        }
        if constexpr (QC) {
            const float ka[8] = {kc0.x, kc0.y, kc0.z, kc0.w, kc1.x, kc1.y, kc1.z, kc1.w};
#pragma unroll
            for (int v = 0; v < 4; v++) {
                s0[v] *= ka[v];
                s1[v] *= ka[4 + v];
            }
        }
#pragma unroll
        for (int v = 0; v < 4; v++) {
            sv[v] = vis[v] ? s0[v] : -INFINITY;
            sv[4 + v] = vis[4 + v] ? s1[v] : -INFINITY;
            mx = fmaxf(mx, fmaxf(sv[v], sv[4 + v]));
        }
        mx = max_rows4(mx);
        const float m_new = fmaxf(m_run, mx);      // finite: the block holds a visible key
        float alpha = __expf(m_run - m_new);         // 0 for the wave's first block
        float vw[8] = {1.f, 1.f, 1.f, 1.f, 1.f, 1.f, 1.f, 1.f};  // V row scales of the lane's keys in units of u_run
        if constexpr (QC) {
            const float va[8] = {vc0.x, vc0.y, vc0.z, vc0.w, vc1.x, vc1.y, vc1.z, vc1.w};
            float vmx = 0.f;
#pragma unroll
            for (int e = 0; e < 8; e++) vmx = fmaxf(vmx, vis[e] ? va[e] : 0.f);
            vmx = max_rows4(vmx);
            const float u_new = fmaxf(u_run, vmx);  // > 0: a visible row's scale is at least f32::EPSILON
            const float inv_u = 1.0f / u_new;
#pragma unroll
            for (int e = 0; e < 8; e++) vw[e] = vis[e] ? va[e] * inv_u : 0.f;
            l_run = l_run * alpha;                  // the sum is rescaled by the softmax factor only
            alpha *= u_run * inv_u;                 // the accumulator also changes its unit
            u_run = u_new;
        } else {
            l_run = l_run * alpha;
        }
        float sum = 0.f;
        v8h_t ph, pl;
#pragma unroll
        for (int e = 0; e < 8; e++) {
            const float pe = __expf(sv[e] - m_new);
            sum += pe;
            const float pv = QC ? pe * vw[e] : pe;
            const _Float16 hi = (_Float16)pv;
            ph[e] = hi;
            pl[e] = (_Float16)(pv - (float)hi);
        }
        sum = sum_rows4(sum);
        l_run += sum;
        m_run = m_new;
        // O^T += V^T P^T; A operand gathered from the staged block
#pragma unroll
        for (int sl = 0; sl < NS; sl++) {
            // a[e] = V[4 g + e][16 sl + qi], a[4 + e] = V[16 + 4 g + e][16 sl + qi]: two transposing LDS reads.  The 16 lanes
            // of a block hand in the addresses of a 4 x 16 tile (lane i: row i / 4, columns 4 (i % 4) .. + 3) and lane j
            // receives column j.
            const _Float16* tile = vs + (4 * g + (qi >> 2)) * VSTR + 16 * sl + 4 * (qi & 3u);
            const v4h_t t0 = lds_read_tr16(tile), t1 = lds_read_tr16(tile + 16 * VSTR);
            const v8h_t a = {t0[0], t0[1], t0[2], t0[3], t1[0], t1[1], t1[2], t1[3]};
#pragma unroll
            for (int v = 0; v < 4; v++) O[sl][v] *= alpha;
            O[sl] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, ph, O[sl], 0, 0, 0);
            O[sl] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, pl, O[sl], 0, 0, 0);
        }
    }
    // --- merge the four waves: lane (head = qi, g) holds O[head][16 sl + 4 g + v], m_run, l_run ---
    __syncthreads();  // the V slices are dead: reuse them
    static_assert(sizeof(vs_all) >= (4 * 16 * HD + 2 * 4 * 16) * sizeof(float), "merge buffers must fit in the V slices");
    float* mo = reinterpret_cast<float*>(&vs_all[0][0]);  // [wave][head 16][HD], then [wave][head 16] m, [wave][head 16] l
    float* mm = mo + 4 * 16 * HD;
    float* ml = mm + 4 * 16;
    if (qi < G) {
#pragma unroll
        for (int sl = 0; sl < NS; sl++)
            *reinterpret_cast<float4*>(&mo[(wave * 16 + qi) * HD + 16 * sl + 4 * g]) =
                make_float4(O[sl][0] * u_run, O[sl][1] * u_run, O[sl][2] * u_run, O[sl][3] * u_run);
    }
    if (g == 0) {
        mm[wave * 16 + qi] = m_run;
        ml[wave * 16 + qi] = l_run;
    }
    __syncthreads();
    for (uint32_t i = tid; i < G * HD; i += 256) {
        const uint32_t h = i / HD, d = i % HD;
        const float M = fmaxf(fmaxf(mm[h], mm[16 + h]), fmaxf(mm[32 + h], mm[48 + h]));
        float o = 0.f, l = 0.f;
#pragma unroll
        for (int w = 0; w < 4; w++) {
            const float wgt = mm[w * 16 + h] == -INFINITY ? 0.f : __expf(mm[w * 16 + h] - M);  // a wave that saw no key
            o = fmaf(mo[(w * 16 + h) * HD + d], wgt, o);
            l = fmaf(ml[w * 16 + h], wgt, l);
        }
        if (p.out_single) {  // the only slot: what the merge would compute (weight 1, times 1 / sum)
            p.out_single[((size_t)b * p.nq + h0 + h) * HD + d] = o * (l > 0.f ? 1.0f / l : 0.f);
            continue;
        }
        put(h * part_head + d, o);
        if (d == 0) {
            put(h * part_head + HD, M);
            put(h * part_head + HD + 1, l);
        }
    }
    if (p.out_single) return;
    if (attn_last_arrival(p, b, kvh, min(n_chunks, p.n_splits), &last_flag))  // (the barrier inside also retires mo / mm / ml)
        attn_merge_heads(p, b, h0, G, G, reinterpret_cast<float*>(&vs_all[0][0]), p.out_merged);
}

// Merge the slot results of heads h_first .. h_first + nh - 1 of sequence b into the attention output
// [batch][nq * hd] (fp32), the input of the O projection, by the 256 threads of a workgroup: per head one wave works
// out the softmax weights of the slots (one slot per lane); the weighted slot outputs of a group of four dimensions
// are added by NPAR threads, thread j taking slots j, j + NPAR, ... in ascending order, and the NPAR sums meet in LDS
// in thread order.  Every thread requests its first 16 slot outputs before the weights are worked out; NPAR is the
// smallest of 1, 2, 4 that covers the slots in use with those requests (one round trip to memory for the whole merge),
// as far as 256 threads allow for the heads' nh * hd / 4 groups.
// sm: heads_per * 65 floats of LDS ([head][64] slot weights | [head] 1 / sum), then 256 float4 for the partial sums.
// The slot results were written by other workgroups of this same launch: agent-coherent loads.
__device__ __forceinline__ void attn_merge_heads(const OxbAttnParams& p, uint32_t b, uint32_t h_first, uint32_t nh, uint32_t heads_per,
                                                 float* sm, float* __restrict__ out) {
    const uint32_t tid = threadIdx.x, lane = tid & 63u, hd = p.hd, qd = p.nq * hd;
    const uint32_t stride = hd + OXB_ATTN_PART_PAD;
    float* wts = sm;
    float* inv_l = wts + heads_per * 64;
    float4* sums = reinterpret_cast<float4*>(sm + ((heads_per * 65 + 3) & ~3u));
    // The merged outputs once more, for the quantiser at the end: 128 groups of four, in the entries of `sums` that the
    // partial sums never use (those are written by threads tg and up, and with 128 groups tg >= 128).
    float4* keep = sums;
    const bool pack = p.pack_out != nullptr && nh * hd == 512u;
    const uint32_t e0 = h_first * hd;
    const uint32_t n_chunks = (p.pos[b] + p.chunk) / p.chunk;  // chunks that hold positions 0..pos
    const uint32_t used = n_chunks < p.n_splits ? n_chunks : p.n_splits;
    const float* part = p.part + (size_t)b * p.nq * p.n_splits * stride;
    const __amdgpu_buffer_rsrc_t r_part = make_rsrc(part, p.nq * p.n_splits * stride * 4u);
    auto ld4 = [&](const float* q) -> float4 {
        const v4f v = buf_load_f128_coherent(r_part, (uint32_t)(q - part) * 4u);
        return make_float4(v.x, v.y, v.z, v.w);
    };
    auto ld1 = [&](const float* q) -> float { return buf_load_f32_coherent(r_part, (uint32_t)(q - part) * 4u); };
    const uint32_t groups = nh * hd / 4;
    // as few threads per group as keep all slots within the first 16 requests (more would only add the LDS step)
    const uint32_t npar_max = groups <= 64 ? 4u : groups <= 128 ? 2u : 1u;
    const uint32_t npar = used <= 16u || npar_max == 1u ? 1u : (used <= 32u || npar_max == 2u ? 2u : 4u);
    const uint32_t tg = 256u / npar, sh = tid / tg, egl = tid % tg;  // this thread: group egl (+ tg, ...), slots sh + npar u
    constexpr int PRE = 16;
    float4 pre[PRE];
    // the maxima and sums of the wave's first head are requested ahead of the slot outputs: loads return in issue
    // order, and the weights are worked out while the outputs are still on their way
    float mv0 = -INFINITY, lv0 = 0.f;
    if ((tid >> 6) < nh) {
        const float* ph = part + ((size_t)(h_first + (tid >> 6)) * p.n_splits + lane) * stride + hd;
        if (lane < used) mv0 = ld1(ph), lv0 = ld1(ph + 1);
    }
    {
        const uint32_t e = e0 + egl * 4;
        const float* ph = part + (size_t)(e / hd) * p.n_splits * stride + e % hd;
#pragma unroll
        for (int u = 0; u < PRE; u++) {
            const uint32_t sl = sh + npar * u;
            pre[u] = (egl < groups && sl < used) ? ld4(ph + (size_t)sl * stride) : make_float4(0.f, 0.f, 0.f, 0.f);
        }
    }
    for (uint32_t hh = tid >> 6; hh < nh; hh += 4) {
        const float* ph = part + ((size_t)(h_first + hh) * p.n_splits + lane) * stride + hd;
        const bool first_head = hh == (tid >> 6);
        const float mv = first_head ? mv0 : (lane < used ? ld1(ph) : -INFINITY), lv = first_head ? lv0 : (lane < used ? ld1(ph + 1) : 0.f);
        float M = mv;
        M = wave_max_f32(M);
        const float w = lane < used ? __expf(mv - M) : 0.f;
        float L = w * lv;
        L = wave_sum_f32(L);
        wts[hh * 64 + lane] = w;
        if (lane == 0) inv_l[hh] = L > 0.f ? 1.0f / L : 0.f;
    }
    __syncthreads();
    for (uint32_t eg0 = 0; eg0 < groups; eg0 += tg) {  // uniform trip count: the barrier below is reached by every thread
        const uint32_t eg = eg0 + egl, e = e0 + eg * 4;
        const bool live = eg < groups;
        const uint32_t h = live ? e / hd : h_first, d = e % hd, hh = h - h_first;
        const float* ph = part + (size_t)h * p.n_splits * stride + d;
        float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
        // PRE requests in flight at a time; slots past `used` count as zeros with weight 0
        auto fold = [&](const float4 (&v)[PRE], uint32_t u0) {
#pragma unroll
            for (int u = 0; u < PRE; u++) {
                const uint32_t sl = sh + npar * (u0 + u);
                const float w = sl < used ? wts[hh * 64 + sl] : 0.f;
                acc.x = fmaf(v[u].x, w, acc.x), acc.y = fmaf(v[u].y, w, acc.y), acc.z = fmaf(v[u].z, w, acc.z), acc.w = fmaf(v[u].w, w, acc.w);
            }
        };
        uint32_t u0 = 0;
        if (eg0 == 0) {  // the group whose first slots are already here
            fold(pre, 0);
            u0 = PRE;
        }
        for (; live && sh + npar * u0 < used; u0 += PRE) {
            float4 v[PRE];
#pragma unroll
            for (int u = 0; u < PRE; u++) {
                const uint32_t sl = sh + npar * (u0 + u);
                v[u] = sl < used ? ld4(ph + (size_t)sl * stride) : make_float4(0.f, 0.f, 0.f, 0.f);
            }
            fold(v, u0);
        }
        if (npar > 1) {  // (then all groups fit one pass)
            if (sh) sums[tid] = acc;
            __syncthreads();
            if (!sh)
                for (uint32_t j = 1; j < npar; j++) {
                    const float4 o = sums[j * tg + egl];
                    acc.x += o.x, acc.y += o.y, acc.z += o.z, acc.w += o.w;
                }
        }
        if (live && !sh) {
            const float il = inv_l[hh];
            acc.x *= il, acc.y *= il, acc.z *= il, acc.w *= il;
            *reinterpret_cast<float4*>(out + (size_t)b * qd + e) = acc;
            if (pack) keep[eg] = acc;
        }
    }
    if (pack) {  // (uniform) one wave quantises the 512 outputs for the O projection: superblock e0 / 512 of vector b
        __syncthreads();
        if (tid < 64) {
            const float* kf = reinterpret_cast<const float*>(keep);
            float xe[2][4];
            if (p.pack_fmt == OXB_FMT_Q1) {
#pragma unroll
                for (int pass = 0; pass < 2; pass++)
#pragma unroll
                    for (int bb = 0; bb < 4; bb++) xe[pass][bb] = kf[gemv_pack_elem<OXB_FMT_Q1>(tid, pass, bb)];
                gemv_pack_write<OXB_FMT_Q1>(xe, 0.f, tid, e0 / 512u, b, p.pack_n_sb, p.pack_nvg, p.pack_out);
            } else {
#pragma unroll
                for (int pass = 0; pass < 2; pass++)
#pragma unroll
                    for (int bb = 0; bb < 4; bb++) xe[pass][bb] = kf[gemv_pack_elem<OXB_FMT_TQ2>(tid, pass, bb)];
                gemv_pack_write<OXB_FMT_TQ2>(xe, 0.f, tid, e0 / 512u, b, p.pack_n_sb, p.pack_nvg, p.pack_out);
            }
        }
    }
}

// ---------------------------------------------------------------------------
// Greedy selection: index of the first maximum (strict '>', as argmax_f32, cuda_kernels.rs:407-436).
// Two stages: grid (parts, vectors) workgroups each reduce a contiguous span to (value, index), then one
// wave per vector merges the parts; ties go to the lower index at every step.
// ---------------------------------------------------------------------------
__device__ __forceinline__ void argmax_merge(float& best, uint32_t& idx, float ob, uint32_t oi) {
    if (oi != 0xFFFFFFFFu && (idx == 0xFFFFFFFFu || ob > best || (ob == best && oi < idx))) { best = ob; idx = oi; }
}

__global__ __launch_bounds__(256) void argmax_partial_kernel(const float* __restrict__ logits, uint32_t n, uint32_t span,
                                                              float* __restrict__ pv, uint32_t* __restrict__ pi) {
    __shared__ float sv[4];
    __shared__ uint32_t si[4];
    const float* v = logits + (size_t)blockIdx.y * n;
    const uint32_t i0 = blockIdx.x * span, i1 = min(i0 + span, n);
    float best = -INFINITY;
    uint32_t idx = 0xFFFFFFFFu;
    for (uint32_t i = i0 + threadIdx.x; i < i1; i += 256) {
        const float x = v[i];
        if (idx == 0xFFFFFFFFu || x > best) { best = x; idx = i; }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) argmax_merge(best, idx, __shfl_xor(best, o, 64), __shfl_xor(idx, o, 64));
    if ((threadIdx.x & 63u) == 0) { sv[threadIdx.x >> 6] = best; si[threadIdx.x >> 6] = idx; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < 4; w++) argmax_merge(best, idx, sv[w], si[w]);
        pv[blockIdx.y * gridDim.x + blockIdx.x] = best;
        pi[blockIdx.y * gridDim.x + blockIdx.x] = idx;
    }
}

__global__ __launch_bounds__(64) void argmax_final_kernel(const float* __restrict__ pv, const uint32_t* __restrict__ pi,
                                                           uint32_t parts, uint32_t* __restrict__ out, uint32_t* __restrict__ host_copy) {
    float best = -INFINITY;
    uint32_t idx = 0xFFFFFFFFu;
    for (uint32_t i = threadIdx.x; i < parts; i += 64) argmax_merge(best, idx, pv[blockIdx.x * parts + i], pi[blockIdx.x * parts + i]);
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) argmax_merge(best, idx, __shfl_xor(best, o, 64), __shfl_xor(idx, o, 64));
    if (threadIdx.x == 0) {
        out[blockIdx.x] = idx == 0xFFFFFFFFu ? 0u : idx;
        if (host_copy) {  // pinned host memory: the caller reads it after synchronising, without a copy of its own
            host_copy[blockIdx.x] = idx == 0xFFFFFFFFu ? 0u : idx;
            __threadfence_system();
        }
    }
}

// Pinned host staging -> device: the hidden rows and positions of a decode call, in one launch ahead of the step's
// graph (two small asynchronous copies cost more than the step's first kernel).
__global__ __launch_bounds__(256) void stage_in_kernel(const float4* __restrict__ h_hidden, uint32_t n4, const uint32_t* __restrict__ h_pos,
                                                        uint32_t n_pos, float4* __restrict__ hidden, uint32_t* __restrict__ pos) {
    const uint32_t i = blockIdx.x * 256 + threadIdx.x;
    if (i < n4) hidden[i] = h_hidden[i];
    if (i < n_pos) pos[i] = h_pos[i];
}

hipError_t oxb_launch_stage_in(const float* h_hidden, uint32_t n_floats, const uint32_t* h_pos, uint32_t n_pos, float* d_hidden,
                               uint32_t* d_pos, hipStream_t st) {
    if ((n_floats & 3u) || n_floats == 0) return hipErrorInvalidValue;
    const uint32_t n4 = n_floats / 4, n = n4 > n_pos ? n4 : n_pos;
    hipLaunchKernelGGL(stage_in_kernel, dim3((n + 255) / 256), dim3(256), 0, st, reinterpret_cast<const float4*>(h_hidden), n4, h_pos, n_pos,
                       reinterpret_cast<float4*>(d_hidden), d_pos);
    return hipGetLastError();
}

// ---------------------------------------------------------------------------
// Launchers
// ---------------------------------------------------------------------------
hipError_t oxb_launch_qk_norm_rope_store(const OxbQkParams& p, uint32_t batch, hipStream_t st) {
    if (p.hd > 256 || p.kv_mode > OXB_KV_FP8_E4M3 || (p.kv_mode != OXB_KV_F16 && (!p.k_scale || !p.v_scale))) return hipErrorInvalidValue;
    const uint32_t per_wg = 4 * OXB_QK_HEADS_PER_WAVE;
    const dim3 grid(((p.q_rope ? p.nq : 0u) + p.nkv + per_wg - 1) / per_wg, batch), block(256);
    if (p.kv_mode == OXB_KV_I8) hipLaunchKernelGGL(qk_norm_rope_store_kernel<OXB_KV_I8>, grid, block, 0, st, p);
    else if (p.kv_mode == OXB_KV_FP8_E4M3) hipLaunchKernelGGL(qk_norm_rope_store_kernel<OXB_KV_FP8_E4M3>, grid, block, 0, st, p);
    else hipLaunchKernelGGL(qk_norm_rope_store_kernel<OXB_KV_F16>, grid, block, 0, st, p);
    return hipGetLastError();
}

hipError_t oxb_launch_attn_decode(const OxbAttnParams& p, uint32_t batch, hipStream_t st) {
    if (p.chunk != OXB_ATTN_CHUNK || p.n_splits == 0 || p.n_splits > OXB_ATTN_MAX_SPLITS || p.nq % p.nkv || p.nq / p.nkv > 16 ||
        !p.qkv || !p.q_norm || !p.k_norm || !p.cos_t || !p.sin_t || p.kv_mode > OXB_KV_FP8_E4M3 || (p.out_single && p.n_splits != 1) || (!p.out_single && (!p.done || !p.out_merged)) ||
        (p.kv_mode != OXB_KV_F16 && (!p.k_scale || !p.v_scale)) ||
        (p.kv.page_table ? (p.kv.page_shift < 4 || p.kv.page_shift > 7) : (p.kv.row_stride % OXB_ATTN_CHUNK != 0 || p.kv.row_stride < p.max_seq)))
        return hipErrorInvalidValue;
    const dim3 grid(p.n_splits, p.nkv, batch), block(256);
    const bool opt = p.window != 0 || p.kv.page_table != nullptr;
    switch (p.hd) {
#define OXB_ATTN_LAUNCH(HD_, KVM_)                                                                                   \
    if (opt) hipLaunchKernelGGL((attn_decode_fused_kernel<HD_, KVM_, true>), grid, block, 0, st, p);                 \
    else hipLaunchKernelGGL((attn_decode_fused_kernel<HD_, KVM_, false>), grid, block, 0, st, p);
#define OXB_ATTN_CASE(HD_)                                         \
    case HD_:                                                      \
        if (p.kv_mode == OXB_KV_I8) {                              \
            OXB_ATTN_LAUNCH(HD_, OXB_KV_I8)                        \
        } else if (p.kv_mode == OXB_KV_FP8_E4M3) {                 \
            OXB_ATTN_LAUNCH(HD_, OXB_KV_FP8_E4M3)                  \
        } else {                                                   \
            OXB_ATTN_LAUNCH(HD_, OXB_KV_F16)                       \
        }                                                          \
        break;
        OXB_ATTN_CASE(32)
        OXB_ATTN_CASE(64)
        OXB_ATTN_CASE(128)
        OXB_ATTN_CASE(256)
#undef OXB_ATTN_LAUNCH
#undef OXB_ATTN_CASE
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

// RMSNorm of `nvec` vectors of n values (simd_float_ops.rs:204-215): out = w * x / sqrt(mean(x^2) + eps), w == nullptr
// copies x.  One workgroup per vector.  The fused paths carry their norms inside the GEMV / GEMM kernels; this one
// finishes a forward that ends at the normed hidden state (no LM head on the device).
__global__ __launch_bounds__(256) void rmsnorm_kernel(const float* __restrict__ x, const float* __restrict__ w, uint32_t n,
                                                      float eps, float* __restrict__ out) {
    __shared__ float part[4];
    const float* xv = x + (size_t)blockIdx.x * n;
    float* ov = out + (size_t)blockIdx.x * n;
    const uint32_t tid = threadIdx.x;
    if (!w) {
        for (uint32_t i = tid; i < n; i += 256) ov[i] = xv[i];
        return;
    }
    float ss = 0.f;
    for (uint32_t i = tid; i < n; i += 256) ss += xv[i] * xv[i];
    ss = wave_sum_f32(ss);
    if ((tid & 63u) == 0) part[tid >> 6] = ss;
    __syncthreads();
    const float inv_rms = 1.0f / sqrtf((part[0] + part[1] + part[2] + part[3]) / (float)n + eps);
    for (uint32_t i = tid; i < n; i += 256) ov[i] = w[i] * xv[i] * inv_rms;
}

hipError_t oxb_launch_rmsnorm(const float* d_x, const float* d_w, uint32_t n, uint32_t nvec, float eps, float* d_out, hipStream_t st) {
    if (n == 0 || nvec == 0 || !d_x || !d_out) return hipErrorInvalidValue;
    hipLaunchKernelGGL(rmsnorm_kernel, dim3(nvec), dim3(256), 0, st, d_x, d_w, n, eps, d_out);
    return hipGetLastError();
}

uint32_t oxb_argmax_parts(uint32_t n) {
    const uint32_t p = (n + 2047u) / 2048u;
    return p < 1 ? 1 : (p > OXB_ARGMAX_MAX_PARTS ? OXB_ARGMAX_MAX_PARTS : p);
}

hipError_t oxb_launch_argmax(const float* d_logits, uint32_t n, uint32_t batch, uint32_t* d_out, void* d_ws, hipStream_t st,
                             uint32_t* host_copy_or_null) {
    if (n == 0 || batch == 0 || !d_ws) return hipErrorInvalidValue;
    const uint32_t parts = oxb_argmax_parts(n), span = (n + parts - 1) / parts;
    float* pv = reinterpret_cast<float*>(d_ws);
    uint32_t* pi = reinterpret_cast<uint32_t*>(d_ws) + (size_t)batch * parts;
    hipLaunchKernelGGL(argmax_partial_kernel, dim3(parts, batch), dim3(256), 0, st, d_logits, n, span, pv, pi);
    hipLaunchKernelGGL(argmax_final_kernel, dim3(batch), dim3(64), 0, st, pv, pi, parts, d_out, host_copy_or_null);
    return hipGetLastError();
}
