// prefill_kernels.hip — causal attention of the prefill pipeline over the FP16 KV cache on the matrix cores
// (the row-wise RMSNorm and SwiGLU of the pipeline live in the GEMM's activation packer, gemm_kernels.hip).
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
// applied per token).  One wave = 16 queries of one q head, working on its own: no barriers; the wave stages
// each 32-key V block in its private slice of LDS, from where the transposed operand is gathered.
//
// Both products run on v_mfma_f32_16x16x32_f16 in transposed form, so the score tile comes out with the
// query in the lane (column) and needs no transposition before the second product:
//   S^T[key][q]  = sum_d K[key][d] Q[q][d]      A = K rows straight from the cache (16 bytes per lane),
//                                               B = Q * scale, split into fp16 hi + lo (two MFMAs: the
//                                               scores keep fp32-level accuracy)
//   O^T[d][q]   += sum_key V[key][d] P[q][key]  B = the lane's own 8 probabilities of a 32-key block,
//                                               A = V gathered for exactly those 8 keys
// Lane (q = lane % 16, g = lane / 16) holds keys {4g..4g+3} and {16+4g..16+4g+3} of each 32-key block.
// ---------------------------------------------------------------------------
template <int HD>
__global__ __launch_bounds__(256) void attn_prefill_kernel(OxbPrefillAttnParams p) {
    constexpr int KS = HD / 32;        // MFMA k-steps over the head dimension
    constexpr int NS = HD / 16;        // 16-wide slices of the output
    constexpr int VL = HD / 16;        // 16-byte pieces of a 32-key V block per lane
    constexpr int VSTR = HD + 8;       // LDS row stride in fp16: 16 bytes of padding keep the gathers conflict-free
    __shared__ __attribute__((aligned(16))) _Float16 vs_all[4][32 * VSTR];  // one V block per wave
    const uint32_t lane = threadIdx.x & 63u, qi = lane & 15u, g = lane >> 4;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    _Float16* vs = vs_all[wave];
    const uint32_t n_qt = (p.M + 15u) / 16u;
    const uint32_t task = blockIdx.x * 4 + wave;
    if (task >= n_qt * p.nq) return;
    const uint32_t qt = n_qt - 1 - task / p.nq, head = task % p.nq;  // long (late) query tiles first
    const uint32_t kvh = head / (p.nq / p.nkv);
    const uint32_t t_last = min(qt * 16 + 15, p.M - 1);
    const uint32_t t_q = min(qt * 16 + qi, p.M - 1);        // rows past M repeat the last one and are not stored
    const uint32_t qpos = p.pos_start + t_q;
    const uint32_t kv_len = p.pos_start + t_last + 1;       // keys the last query of the tile sees
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

    // K rows of the two 16-key tiles (A operands) and this lane's pieces of the 32-key V block, one block ahead.
    // Rows past the last key repeat it; their scores are masked.
    v8h k0r[KS], k1r[KS];
    v4i vr[VL];
    auto load_k = [&](uint32_t key0) {
        const uint32_t kr0 = min(key0 + qi, kv_len - 1), kr1 = min(key0 + 16 + qi, kv_len - 1);
#pragma unroll
        for (int s = 0; s < KS; s++) {
            k0r[s] = *reinterpret_cast<const v8h*>(K + (size_t)kr0 * HD + 32 * s + 8 * g);
            k1r[s] = *reinterpret_cast<const v8h*>(K + (size_t)kr1 * HD + 32 * s + 8 * g);
        }
    };
    auto load_v = [&](uint32_t key0) {  // piece i of the lane: row (i * 64 + lane) / (HD / 8), 16-byte column (..) % (HD / 8)
#pragma unroll
        for (int i = 0; i < VL; i++) {
            const uint32_t id = i * 64 + lane, row = min(key0 + id / (HD / 8), kv_len - 1), col = id % (HD / 8);
            vr[i] = *reinterpret_cast<const v4i*>(V + (size_t)row * HD + col * 8);
        }
    };
    load_k(0);
    load_v(0);

    for (uint32_t key0 = 0; key0 < kv_len; key0 += 32) {
        // stage the V block (the previous block's reads were issued before this point: LDS runs in order)
#pragma unroll
        for (int i = 0; i < VL; i++) {
            const uint32_t id = i * 64 + lane;
            *reinterpret_cast<v4i*>(vs + (id / (HD / 8)) * VSTR + (id % (HD / 8)) * 8) = vr[i];
        }
        load_v(key0 + 32);
        // scores of keys key0 .. key0+31 for the 16 queries
        v4f s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < KS; s++) {
            s0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(k0r[s], qh[s], s0, 0, 0, 0);
            s0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(k0r[s], ql[s], s0, 0, 0, 0);
            s1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(k1r[s], qh[s], s1, 0, 0, 0);
            s1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(k1r[s], ql[s], s1, 0, 0, 0);
        }
        // this lane: query qi, keys key0 + 4g + v and key0 + 16 + 4g + v
        float sv[8];
        float mx = -INFINITY;
#pragma unroll
        for (int v = 0; v < 4; v++) {
            sv[v] = key0 + 4 * g + v <= qpos ? s0[v] : -INFINITY;
            sv[4 + v] = key0 + 16 + 4 * g + v <= qpos ? s1[v] : -INFINITY;
            mx = fmaxf(mx, fmaxf(sv[v], sv[4 + v]));
        }
        load_k(key0 + 32);
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
        // O^T += V^T P^T; A operand: V[key(g, e)][16 slice + qi] gathered from the staged block
        // (rows past the last key hold a repeated row; their probabilities are 0)
#pragma unroll
        for (int sl = 0; sl < NS; sl++) {
            v8h a;
#pragma unroll
            for (int e = 0; e < 8; e++) a[e] = vs[(e < 4 ? 4 * g + e : 16 + 4 * g + e - 4) * VSTR + 16 * sl + qi];
#pragma unroll
            for (int v = 0; v < 4; v++) O[sl][v] *= alpha;
            O[sl] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, pb, O[sl], 0, 0, 0);
        }
    }
    // lane (q = qi, g) holds O[q][16 sl + 4g + v]
    if (qt * 16 + qi < p.M) {
        const float inv = 1.0f / l_run;
        float* o = p.out + ((size_t)(qt * 16 + qi) * p.nq + head) * HD + 4 * g;
#pragma unroll
        for (int sl = 0; sl < NS; sl++)
            *reinterpret_cast<float4*>(o + 16 * sl) = make_float4(O[sl][0] * inv, O[sl][1] * inv, O[sl][2] * inv, O[sl][3] * inv);
    }
}

hipError_t oxb_launch_attn_prefill(const OxbPrefillAttnParams& p, hipStream_t st) {
    if (p.M == 0 || p.nq == 0 || p.nkv == 0 || p.nq % p.nkv || p.pos_start + p.M > p.max_seq) return hipErrorInvalidValue;
    const uint32_t tasks = ((p.M + 15u) / 16u) * p.nq, grid = (tasks + 3) / 4;
    switch (p.hd) {
        case 32: hipLaunchKernelGGL(attn_prefill_kernel<32>, dim3(grid), dim3(256), 0, st, p); break;
        case 64: hipLaunchKernelGGL(attn_prefill_kernel<64>, dim3(grid), dim3(256), 0, st, p); break;
        case 128: hipLaunchKernelGGL(attn_prefill_kernel<128>, dim3(grid), dim3(256), 0, st, p); break;
        case 256: hipLaunchKernelGGL(attn_prefill_kernel<256>, dim3(grid), dim3(256), 0, st, p); break;
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}
