// prefill_kernels.hip — causal attention of the prefill pipeline over the FP16 KV cache on the matrix cores
// (the row-wise RMSNorm of the pipeline lives in the GEMM's activation packer, SwiGLU in the gate || up GEMM's
// epilogue, gemm_kernels.hip).
//
// The reference's prefill (gpu_backend/cuda_prefill/encode_q1.rs:123-300, encode_ternary.rs:114-314) batches
// the projections but walks the tokens one by one through its decode attention kernels
// (cuda_prefill/mod.rs:36-39); here all M query tokens of a sequence attend in one launch.
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

#include "device_utils.h"
#include "prefill_kernels.h"

typedef _Float16 v8h __attribute__((ext_vector_type(8)));

// ---------------------------------------------------------------------------
// Causal attention of M query tokens (positions pos_start .. pos_start + M - 1) over keys 0 .. own position
// of one sequence, GQA, online softmax (semantics: block/functions.rs:78-127 -> layers/attention_fused.rs:329-400
// applied per token).  One wave = 16 queries of one q head.
//
// Both products run on v_mfma_f32_16x16x32_f16 in transposed form, so the score tile comes out with the
// query in the lane (column) and needs no transposition before the second product:
//   S^T[key][q]  = sum_d K[key][d] Q[q][d]      A = K rows (16 bytes per lane),
//                                               B = Q * scale, split into fp16 hi + lo (two MFMAs: the
//                                               scores keep fp32-level accuracy)
//   O^T[d][q]   += sum_key V[key][d] P[q][key]  B = the lane's own 8 probabilities of a 32-key block,
//                                               A = V gathered for exactly those 8 keys
// Lane (q = lane % 16, g = lane / 16) holds keys {4g..4g+3} and {16+4g..16+4g+3} of each 32-key block.
//
// The four waves of a workgroup walk the same keys and values: they take `hpw` q heads of ONE kv head (4, 2 or 1,
// whatever divides the group) times 4 / hpw consecutive query tiles.  Each 32-key block of K and V is fetched once
// per workgroup into LDS, double-buffered: while block i is being used, block i+1 waits in registers and is
// written to the other buffer before the barrier that ends the block.  Waves of an earlier query tile see the
// last block(s) fully masked.
// ---------------------------------------------------------------------------
template <int HD>
__global__ __launch_bounds__(256) void attn_prefill_kernel(OxbPrefillAttnParams p, uint32_t hpw) {
    constexpr int KS = HD / 32, NS = HD / 16;
    constexpr int STR = HD + 8;                      // LDS row stride in fp16 (16 bytes of padding: conflict-free rows)
    constexpr int PIECES = 32 * HD / 8;              // 16-byte pieces of a 32-key block
    constexpr int PP = (PIECES + 255) / 256;         // pieces per thread
    __shared__ __attribute__((aligned(16))) _Float16 ks[2][32 * STR];
    __shared__ __attribute__((aligned(16))) _Float16 vs[2][32 * STR];
    const uint32_t tid = threadIdx.x, lane = tid & 63u, qi = lane & 15u, g = lane >> 4;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(tid >> 6));
    const uint32_t n_qt = (p.M + 15u) / 16u, hq = p.nq / hpw, tpw = 4u / hpw, n_tg = (n_qt + tpw - 1) / tpw;
    const uint32_t tg = n_tg - 1 - blockIdx.x / hq;                       // long (late) query tiles first
    const uint32_t head = (blockIdx.x % hq) * hpw + wave % hpw;
    const uint32_t qt_own = tg * tpw + wave / hpw;
    const bool active = qt_own < n_qt;                                    // a tile past the end: the wave only helps with the loads
    const uint32_t qt = active ? qt_own : n_qt - 1;
    const uint32_t kvh = head / (p.nq / p.nkv);                           // the same for the four waves
    const uint32_t t_q = min(qt * 16 + qi, p.M - 1);                      // rows past M repeat the last one and are not stored
    const uint32_t qpos = p.pos_start + t_q;
    const uint32_t kv_len = p.pos_start + min((tg * tpw + tpw - 1) * 16 + 15, p.M - 1) + 1;  // keys the workgroup's last query sees
    const _Float16* K = reinterpret_cast<const _Float16*>(p.k_cache) + (size_t)kvh * p.max_seq * HD;
    const _Float16* V = reinterpret_cast<const _Float16*>(p.v_cache) + (size_t)kvh * p.max_seq * HD;

    v8h qh[KS], ql[KS];
    {
        const float* qr = p.q + ((size_t)t_q * p.nq + head) * HD + 8 * g;
#pragma unroll
        for (int s = 0; s < KS; s++) {
            const float4 a = *reinterpret_cast<const float4*>(qr + 32 * s), b = *reinterpret_cast<const float4*>(qr + 32 * s + 4);
            const float f[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const float x = f[e] * p.scale;
                const _Float16 hi = (_Float16)x;
                qh[s][e] = hi;
                ql[s][e] = (_Float16)(x - (float)hi);
            }
        }
    }
    v4f O[NS];
#pragma unroll
    for (int i = 0; i < NS; i++) O[i] = (v4f){0.f, 0.f, 0.f, 0.f};
    float m_run = -INFINITY, l_run = 0.f;

    // this thread's pieces of a block: piece id = i * 256 + tid -> row id / (HD / 8), 16-byte column id % (HD / 8);
    // rows past the last key repeat it (their scores are masked, their probabilities 0)
    v4i kreg[PP], vreg[PP];
    auto fetch = [&](uint32_t key0) {
#pragma unroll
        for (int i = 0; i < PP; i++) {
            const uint32_t id = i * 256 + tid;
            if (PIECES % 256 == 0 || id < (uint32_t)PIECES) {
                const uint32_t row = min(key0 + id / (HD / 8), kv_len - 1), col = id % (HD / 8);
                kreg[i] = *reinterpret_cast<const v4i*>(K + (size_t)row * HD + col * 8);
                vreg[i] = *reinterpret_cast<const v4i*>(V + (size_t)row * HD + col * 8);
            }
        }
    };
    auto stash = [&](int buf) {
#pragma unroll
        for (int i = 0; i < PP; i++) {
            const uint32_t id = i * 256 + tid;
            if (PIECES % 256 == 0 || id < (uint32_t)PIECES) {
                *reinterpret_cast<v4i*>(&ks[buf][(id / (HD / 8)) * STR + (id % (HD / 8)) * 8]) = kreg[i];
                *reinterpret_cast<v4i*>(&vs[buf][(id / (HD / 8)) * STR + (id % (HD / 8)) * 8]) = vreg[i];
            }
        }
    };
    fetch(0);
    stash(0);
    if (32 < kv_len) fetch(32);
    __syncthreads();

    int buf = 0;
    for (uint32_t key0 = 0; key0 < kv_len; key0 += 32) {
        const _Float16* kb = ks[buf];
        const _Float16* vb = vs[buf];
        v4f s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < KS; s++) {
            const v8h k0 = *reinterpret_cast<const v8h*>(kb + qi * STR + 32 * s + 8 * g);
            const v8h k1 = *reinterpret_cast<const v8h*>(kb + (16 + qi) * STR + 32 * s + 8 * g);
            s0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(k0, qh[s], s0, 0, 0, 0);
            s0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(k0, ql[s], s0, 0, 0, 0);
            s1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(k1, qh[s], s1, 0, 0, 0);
            s1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(k1, ql[s], s1, 0, 0, 0);
        }
        float sv[8];
        float mx = -INFINITY;
#pragma unroll
        for (int v = 0; v < 4; v++) {
            sv[v] = key0 + 4 * g + v <= qpos ? s0[v] : -INFINITY;
            sv[4 + v] = key0 + 16 + 4 * g + v <= qpos ? s1[v] : -INFINITY;
            mx = fmaxf(mx, fmaxf(sv[v], sv[4 + v]));
        }
        mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        const float m_new = fmaxf(m_run, mx);       // finite from the first block on: key 0 is visible to every query
        const float alpha = __expf(m_run - m_new);  // 0 for the first block
        float sum = 0.f;
        v8h pb;
#pragma unroll
        for (int e = 0; e < 8; e++) {
            const float pe = __expf(sv[e] - m_new);
            sum += pe;
            pb[e] = (_Float16)pe;
        }
        sum += __shfl_xor(sum, 16, 64);
        sum += __shfl_xor(sum, 32, 64);
        l_run = l_run * alpha + sum;
        m_run = m_new;
#pragma unroll
        for (int sl = 0; sl < NS; sl++) {
            v8h a;
#pragma unroll
            for (int e = 0; e < 8; e++) a[e] = vb[(e < 4 ? 4 * g + e : 16 + 4 * g + e - 4) * STR + 16 * sl + qi];
#pragma unroll
            for (int v = 0; v < 4; v++) O[sl][v] *= alpha;
            O[sl] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, pb, O[sl], 0, 0, 0);
        }
        // the next block goes into the other buffer (last read one block ago, before the previous barrier);
        // the block after it is requested now
        if (key0 + 32 < kv_len) {
            stash(buf ^ 1);
            if (key0 + 64 < kv_len) fetch(key0 + 64);
        }
        __syncthreads();
        buf ^= 1;
    }
    if (active && qt * 16 + qi < p.M) {
        const float inv = 1.0f / l_run;
        float* o = p.out + ((size_t)(qt * 16 + qi) * p.nq + head) * HD + 4 * g;
#pragma unroll
        for (int sl = 0; sl < NS; sl++)
            *reinterpret_cast<float4*>(o + 16 * sl) = make_float4(O[sl][0] * inv, O[sl][1] * inv, O[sl][2] * inv, O[sl][3] * inv);
    }
}

hipError_t oxb_launch_attn_prefill(const OxbPrefillAttnParams& p, hipStream_t st) {
    if (p.M == 0 || p.nq == 0 || p.nkv == 0 || p.nq % p.nkv || p.pos_start + p.M > p.max_seq) return hipErrorInvalidValue;
    const uint32_t G = p.nq / p.nkv, hpw = G % 4u == 0 ? 4u : (G % 2u == 0 ? 2u : 1u), tpw = 4u / hpw;
    const uint32_t n_qt = (p.M + 15u) / 16u, grid = ((n_qt + tpw - 1) / tpw) * (p.nq / hpw);
    switch (p.hd) {
        case 32: hipLaunchKernelGGL(attn_prefill_kernel<32>, dim3(grid), dim3(256), 0, st, p, hpw); break;
        case 64: hipLaunchKernelGGL(attn_prefill_kernel<64>, dim3(grid), dim3(256), 0, st, p, hpw); break;
        case 128: hipLaunchKernelGGL(attn_prefill_kernel<128>, dim3(grid), dim3(256), 0, st, p, hpw); break;
        case 256: hipLaunchKernelGGL(attn_prefill_kernel<256>, dim3(grid), dim3(256), 0, st, p, hpw); break;
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}
