// prefill_kernels.hip — causal attention of the prefill pipeline over the KV cache (fp16 or quantised rows) on the matrix cores
// (the row-wise RMSNorm of the pipeline lives in the GEMM's activation packer, SwiGLU in the gate || up GEMM's
// epilogue, gemm_kernels.hip).
//
// The reference's prefill (gpu_backend/cuda_prefill/encode_q1.rs:123-300, encode_ternary.rs:114-314) batches
// the projections but walks the tokens one by one through its decode attention kernels
// (cuda_prefill/mod.rs:36-39); here all M query tokens of a sequence attend in one launch.
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

#include <type_traits>

#include "device_utils.h"
#include "kv_quant_device.h"
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
// Options as in the decode attention: quantised cache rows (template KVM; the codes are widened to exact fp16
// numbers on their way into LDS, V already multiplied by its row scale there, the K row scale multiplies the
// score) and a sliding window with attention sinks (key visible to the query at qpos iff key < sinks or
// qpos - key < window - sinks; blocks no query of the workgroup can see are skipped).
template <int HD, int KVM, bool OPT>  // OPT: a window and / or a paged cache may be in use (else neither costs anything)
__global__ __launch_bounds__(256) void attn_prefill_kernel(OxbPrefillAttnParams p, uint32_t hpw) {
    constexpr bool QC = KVM != OXB_KV_F16;
    constexpr int KS = HD / 32, NS = HD / 16;
    constexpr int STR = HD + 8;                      // LDS row stride in fp16 (16 bytes of padding: conflict-free rows)
    constexpr int PPR = QC ? HD / 16 : HD / 8;       // 16-byte pieces per cache row
    constexpr int PIECES = 32 * PPR;                 // pieces of a 32-key block
    constexpr int PP = (PIECES + 255) / 256;         // pieces per thread
    __shared__ __attribute__((aligned(16))) _Float16 ks[2][32 * STR];
    __shared__ __attribute__((aligned(16))) _Float16 vs[2][32 * STR];
    __shared__ __attribute__((aligned(16))) float kscale[2][32];                // K row scales of the block (quantised cache)
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
    typedef typename std::conditional<QC, uint8_t, _Float16>::type cache_t;
    const cache_t* K = reinterpret_cast<const cache_t*>(p.k_cache);
    const cache_t* V = reinterpret_cast<const cache_t*>(p.v_cache);
    const float* Ksc = p.k_scale;
    const float* Vsc = p.v_scale;
    const bool paged = OPT && p.kv.page_table != nullptr;
    const uint32_t window = OPT ? p.window : 0u;
    const size_t row0 = paged ? 0 : kv_row(p.kv, p.seq, p.layer, kvh, 0);
    auto row_of = [&](uint32_t key) -> size_t { return paged ? kv_row(p.kv, p.seq, p.layer, kvh, key) : row0 + key; };
    // sliding window: this query sees [0, sinks) and (qpos - budget, qpos]; the workgroup's earliest query sits at
    // q_first, so no query of it sees a key in [sinks, q_first + 1 - budget): whole 32-key blocks in there are skipped
    const uint32_t budget = window > p.sinks ? window - p.sinks : 0u;
    const uint32_t q_first = p.pos_start + tg * tpw * 16;
    const uint32_t skip_from = window ? (p.sinks + 31u) & ~31u : 0u;
    const uint32_t skip_to = window && q_first + 1 > budget ? (q_first + 1 - budget) & ~31u : 0u;
    auto next_block = [&](uint32_t key0) {  // the block after key0 that some query may see
        key0 += 32;
        return key0 >= skip_from && key0 < skip_to ? skip_to : key0;
    };

    // Q of this lane's query: per-head RMSNorm, RoPE on the pairs (d, d + hd/2), times 1/sqrt(hd)
    // (fused_qk_norm_rope, gpu_backend/cuda_attn_kernels.rs:160-226), then split into fp16 hi + lo.  The lane holds
    // elements 32 s + 8 g + e; for hd >= 64 both elements of a pair are its own (steps s and s + KS / 2), for hd = 32
    // the partner sits in lane g ^ 2.
    v8h qh[KS], ql[KS];
    {
        constexpr int half = HD / 2;
        const float* qr = p.qkv + (size_t)t_q * p.qkv_stride + (size_t)head * HD + 8 * g;
        float x[KS][8], ss = 0.f;
#pragma unroll
        for (int s = 0; s < KS; s++) {
            const float4 a = *reinterpret_cast<const float4*>(qr + 32 * s), b = *reinterpret_cast<const float4*>(qr + 32 * s + 4);
            const float f[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
            for (int e = 0; e < 8; e++) {
                x[s][e] = f[e];
                ss = fmaf(f[e], f[e], ss);
            }
        }
        ss = sum_rows4(ss);
        const float inv = 1.0f / sqrtf(ss / (float)HD + p.eps);
#pragma unroll
        for (int s = 0; s < KS; s++)
#pragma unroll
            for (int e = 0; e < 8; e++) x[s][e] = p.q_norm[32 * s + 8 * g + e] * x[s][e] * inv;
        const float* cs = p.cos_t + (size_t)qpos * half;
        const float* sn = p.sin_t + (size_t)qpos * half;
        float r[KS][8];
        if constexpr (KS >= 2) {
#pragma unroll
            for (int s = 0; s < KS / 2; s++)
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    const int d = 32 * s + 8 * (int)g + e;  // < half
                    const float lo = x[s][e], hi = x[s + KS / 2][e], c = cs[d], sv = sn[d];
                    r[s][e] = lo * c - hi * sv;
                    r[s + KS / 2][e] = lo * sv + hi * c;
                }
        } else {  // hd = 32: lanes g = 0, 1 hold the first half, g = 2, 3 the second
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const float mine = x[0][e], other = __shfl_xor(mine, 32, 64);
                const int d = 8 * (int)(g & 1u) + e;
                const float c = cs[d], sv = sn[d];
                r[0][e] = g < 2 ? mine * c - other * sv : other * sv + mine * c;
            }
        }
#pragma unroll
        for (int s = 0; s < KS; s++)
#pragma unroll
            for (int e = 0; e < 8; e++) {
                const float v = r[s][e] * p.scale;
                const _Float16 hi = (_Float16)v;
                qh[s][e] = hi;
                ql[s][e] = (_Float16)(v - (float)hi);
            }
    }
    v4f O[NS];
#pragma unroll
    for (int i = 0; i < NS; i++) O[i] = (v4f){0.f, 0.f, 0.f, 0.f};
    float m_run = -INFINITY, l_run = 0.f;

    // this thread's pieces of a block: piece id = i * 256 + tid -> row id / PPR, 16-byte column id % PPR;
    // rows past the last key repeat it (their scores are masked, their probabilities 0)
    v4i kreg[PP], vreg[PP];
    float vsreg[PP], ksreg = 0.f;  // quantised cache: the V row scale of each piece, one K row scale (threads 0..31)
    auto fetch = [&](uint32_t key0) {
#pragma unroll
        for (int i = 0; i < PP; i++) {
            const uint32_t id = i * 256 + tid;
            if (PIECES % 256 == 0 || id < (uint32_t)PIECES) {
                const uint32_t col = id % PPR;
                const size_t row = row_of(min(key0 + id / PPR, kv_len - 1));
                kreg[i] = *reinterpret_cast<const v4i*>(reinterpret_cast<const uint8_t*>(K + row * HD) + col * 16);
                vreg[i] = *reinterpret_cast<const v4i*>(reinterpret_cast<const uint8_t*>(V + row * HD) + col * 16);
                if constexpr (QC) vsreg[i] = Vsc[row];
            }
        }
        if constexpr (QC)
            if (tid < 32) ksreg = Ksc[row_of(min(key0 + tid, kv_len - 1))];
    };
    auto stash = [&](int buf) {
#pragma unroll
        for (int i = 0; i < PP; i++) {
            const uint32_t id = i * 256 + tid;
            if (PIECES % 256 == 0 || id < (uint32_t)PIECES) {
                if constexpr (QC) {
                    uint32_t kd[8], vd[8];
                    kv_dec4<KVM>((uint32_t)kreg[i].x, kd[0], kd[1]);
                    kv_dec4<KVM>((uint32_t)kreg[i].y, kd[2], kd[3]);
                    kv_dec4<KVM>((uint32_t)kreg[i].z, kd[4], kd[5]);
                    kv_dec4<KVM>((uint32_t)kreg[i].w, kd[6], kd[7]);
                    kv_dec4<KVM>((uint32_t)vreg[i].x, vd[0], vd[1]);
                    kv_dec4<KVM>((uint32_t)vreg[i].y, vd[2], vd[3]);
                    kv_dec4<KVM>((uint32_t)vreg[i].z, vd[4], vd[5]);
                    kv_dec4<KVM>((uint32_t)vreg[i].w, vd[6], vd[7]);
                    // V leaves for LDS as code * scale in fp16 (the probabilities it meets are fp16 as well)
                    const _Float16 sc = (_Float16)vsreg[i];
                    const kvh2_t sc2 = {sc, sc};
#pragma unroll
                    for (int e = 0; e < 8; e++) vd[e] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(kvh2_t, vd[e]) * sc2);
                    _Float16* kd_ = &ks[buf][(id / PPR) * STR + (id % PPR) * 16];
                    _Float16* vd_ = &vs[buf][(id / PPR) * STR + (id % PPR) * 16];
                    *reinterpret_cast<v4i*>(kd_) = (v4i){(int)kd[0], (int)kd[1], (int)kd[2], (int)kd[3]};
                    *reinterpret_cast<v4i*>(kd_ + 8) = (v4i){(int)kd[4], (int)kd[5], (int)kd[6], (int)kd[7]};
                    *reinterpret_cast<v4i*>(vd_) = (v4i){(int)vd[0], (int)vd[1], (int)vd[2], (int)vd[3]};
                    *reinterpret_cast<v4i*>(vd_ + 8) = (v4i){(int)vd[4], (int)vd[5], (int)vd[6], (int)vd[7]};
                } else {
                    *reinterpret_cast<v4i*>(&ks[buf][(id / PPR) * STR + (id % PPR) * 8]) = kreg[i];
                    *reinterpret_cast<v4i*>(&vs[buf][(id / PPR) * STR + (id % PPR) * 8]) = vreg[i];
                }
            }
        }
        if constexpr (QC)
            if (tid < 32) kscale[buf][tid] = ksreg;
    };
    fetch(0);
    stash(0);
    if (next_block(0) < kv_len) fetch(next_block(0));
    __syncthreads();

    int buf = 0;
    for (uint32_t key0 = 0; key0 < kv_len;) {
        const uint32_t key1 = next_block(key0), key2 = next_block(key1);
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
        if constexpr (QC) {
            const float4 a = *reinterpret_cast<const float4*>(&kscale[buf][4 * g]), b = *reinterpret_cast<const float4*>(&kscale[buf][16 + 4 * g]);
            s0[0] *= a.x, s0[1] *= a.y, s0[2] *= a.z, s0[3] *= a.w;
            s1[0] *= b.x, s1[1] *= b.y, s1[2] *= b.z, s1[3] *= b.w;
        }
        float sv[8];
        float mx = -INFINITY;
#pragma unroll
        for (int v = 0; v < 4; v++) {
            const uint32_t ka = key0 + 4 * g + v, kb_ = ka + 16;
            const bool va = ka <= qpos && (!window || ka < p.sinks || qpos - ka < budget);
            const bool vb_ = kb_ <= qpos && (!window || kb_ < p.sinks || qpos - kb_ < budget);
            sv[v] = va ? s0[v] : -INFINITY;
            sv[4 + v] = vb_ ? s1[v] : -INFINITY;
            mx = fmaxf(mx, fmaxf(sv[v], sv[4 + v]));
        }
        mx = max_rows4(mx);
        // without a window key 0 is visible to every query, so the maximum is finite from the first block on; with
        // one, a query may see nothing yet: it keeps its empty state (all probabilities 0)
        const float m_new = fmaxf(m_run, mx);
        const float m_ref = m_new == -INFINITY ? 0.f : m_new;
        const float alpha = __expf(m_run - m_ref);  // 0 for the first block
        float sum = 0.f;
        v8h pb;
#pragma unroll
        for (int e = 0; e < 8; e++) {
            const float pe = __expf(sv[e] - m_ref);
            sum += pe;
            pb[e] = (_Float16)pe;
        }
        sum = sum_rows4(sum);
        l_run = l_run * alpha + sum;
        m_run = m_new;
#pragma unroll
        for (int sl = 0; sl < NS; sl++) {
            // a[e] = V[4 g + e][16 sl + qi], a[4 + e] = V[16 + 4 g + e][16 sl + qi]: two transposing reads
            const _Float16* tile = vb + (4 * g + (qi >> 2)) * STR + 16 * sl + 4 * (qi & 3u);
            const v4h_t t0 = lds_read_tr16(tile), t1 = lds_read_tr16(tile + 16 * STR);
            const v8h a = {t0[0], t0[1], t0[2], t0[3], t1[0], t1[1], t1[2], t1[3]};
#pragma unroll
            for (int v = 0; v < 4; v++) O[sl][v] *= alpha;
            O[sl] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, pb, O[sl], 0, 0, 0);
        }
        // the next block goes into the other buffer (last read one block ago, before the previous barrier);
        // the block after it is requested now
        if (key1 < kv_len) {
            stash(buf ^ 1);
            if (key2 < kv_len) fetch(key2);
        }
        __syncthreads();
        buf ^= 1;
        key0 = key1;
    }
    if (active && qt * 16 + qi < p.M) {
        const float inv = l_run > 0.f ? 1.0f / l_run : 0.f;
        float* o = p.out + ((size_t)(qt * 16 + qi) * p.nq + head) * HD + 4 * g;
#pragma unroll
        for (int sl = 0; sl < NS; sl++)
            *reinterpret_cast<float4*>(o + 16 * sl) = make_float4(O[sl][0] * inv, O[sl][1] * inv, O[sl][2] * inv, O[sl][3] * inv);
    }
}

hipError_t oxb_launch_attn_prefill(const OxbPrefillAttnParams& p, hipStream_t st) {
    if (p.M == 0 || p.nq == 0 || p.nkv == 0 || p.nq % p.nkv || !p.qkv || !p.q_norm || !p.cos_t || !p.sin_t || p.pos_start + p.M > p.max_seq || p.kv_mode > OXB_KV_FP8_E4M3 ||
        (p.kv_mode != OXB_KV_F16 && (!p.k_scale || !p.v_scale)) || (p.kv.page_table && (p.kv.page_shift < 4 || p.kv.page_shift > 7)))
        return hipErrorInvalidValue;
    const uint32_t G = p.nq / p.nkv, hpw = G % 4u == 0 ? 4u : (G % 2u == 0 ? 2u : 1u), tpw = 4u / hpw;
    const uint32_t n_qt = (p.M + 15u) / 16u, grid = ((n_qt + tpw - 1) / tpw) * (p.nq / hpw);
    const bool opt = p.window != 0 || p.kv.page_table != nullptr;
    switch (p.hd) {
#define OXB_PF_LAUNCH(HD_, KVM_)                                                                                     \
    if (opt) hipLaunchKernelGGL((attn_prefill_kernel<HD_, KVM_, true>), dim3(grid), dim3(256), 0, st, p, hpw);        \
    else hipLaunchKernelGGL((attn_prefill_kernel<HD_, KVM_, false>), dim3(grid), dim3(256), 0, st, p, hpw);
#define OXB_PF_CASE(HD_)                                           \
    case HD_:                                                      \
        if (p.kv_mode == OXB_KV_I8) {                              \
            OXB_PF_LAUNCH(HD_, OXB_KV_I8)                          \
        } else if (p.kv_mode == OXB_KV_FP8_E4M3) {                 \
            OXB_PF_LAUNCH(HD_, OXB_KV_FP8_E4M3)                    \
        } else {                                                   \
            OXB_PF_LAUNCH(HD_, OXB_KV_F16)                         \
        }                                                          \
        break;
        OXB_PF_CASE(32)
        OXB_PF_CASE(64)
        OXB_PF_CASE(128)
        OXB_PF_CASE(256)
#undef OXB_PF_LAUNCH
#undef OXB_PF_CASE
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}
