// gemm_kernels.hip — prefill GEMM for Q1_0_g128 / TQ2_0_g128 weights on gfx950:
//     Y[m][n] = sum_k W[n][k] * X[m][k]      (X: M token rows, W: the resident quantised matrix)
// (reference semantics: crates/oxibonsai-kernels/src/gemm.rs:19-87, gemm_ternary.rs:35-69; the CUDA tier's
// scalar-FMA kernels gemm_q1_g128_v7 / gemm_tq2_g128_v7, gpu_backend/cuda_prefill_kernels.rs:74-140, 457-551).
//
// Arithmetic.  Weights +-d / 0 are exact in fp16 and so is every product with an fp16 activation in the fp32
// accumulator of v_mfma_f32_16x16x32_f16; the only rounding beyond fp32 summation is the activation's
// conversion to fp16 (relative 2^-11 per element), after scaling each token row by a power of two so the
// result does not depend on the row's magnitude.
//
// Data flow.  The weight side never touches LDS: the resident layout (layout.h) already hands lane (r, g) of a
// wave the code bits of row r, k-group g, which is the MFMA A-operand position, so each lane expands its own
// bits to fp16 +-d in registers.  Because the k order inside an MFMA is free as long as A and B agree, the
// expansion pairs weights whose codes lie 16 bits apart in a code dword (one shift + one mask builds two fp16
// values) and the activation packer writes X in exactly that order:
//   xh[(blk * 16 + 4g + s) * M_pad + m]  = 16 bytes = the 8 fp16 that lane (token m, k-group g) feeds to MFMA
//   step s of block blk;  element 2p+h  <->  k = 128 blk + 32 g + 4 s + p + 16 h            (Q1)
//                                             k = 128 blk + 32 g + 16 (s/2) + 4 (s%2) + p + 8 h   (TQ2)
// One workgroup = 4 waves stacked along the weight rows; they share one token tile of X that is staged per
// 128-weight block through double-buffered LDS.  Wave w owns up to RT row tiles (16 rows each) and CT token
// tiles (16 tokens each): RT*CT accumulator tiles, RT decoded A operands reused over CT B operands.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "device_utils.h"
#include "gemm_kernels.h"
#include "layout.h"

typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef _Float16 v2h __attribute__((ext_vector_type(2)));

#define OXB_GEMM_THREADS 256

// ---------------------------------------------------------------------------
// Activation packer.  One workgroup = 16 token rows; grid.y workgroups share the blocks of those rows.
// ---------------------------------------------------------------------------
__device__ __forceinline__ uint32_t pack_h2(float a, float b) {
    const v2h h = {(_Float16)a, (_Float16)b};
    return __builtin_bit_cast(uint32_t, h);
}

template <int FMT>
__global__ __launch_bounds__(256) void xh_pack_kernel(const float* __restrict__ x, uint32_t ldx, uint32_t k, uint32_t M,
                                                       uint32_t M_pad, uint32_t nblk_pad, uint4* __restrict__ xh,
                                                       int32_t* __restrict__ xsh) {
    __shared__ int sh_shift[16];
    const uint32_t tid = threadIdx.x, m0 = blockIdx.x * 16;
    {  // row maxima: 16 lanes per row
        const uint32_t j = tid >> 4, i = tid & 15u, m = m0 + j;
        float mx = 0.0f;
        int bad = 0;
        if (m < M) {
            const float* xr = x + (size_t)m * ldx;
            for (uint32_t kk = i * 4; kk < k; kk += 64) {
                const float4 v = *reinterpret_cast<const float4*>(xr + kk);
                bad |= !(fabsf(v.x) <= 3.402823466e38f) | !(fabsf(v.y) <= 3.402823466e38f) |
                       !(fabsf(v.z) <= 3.402823466e38f) | !(fabsf(v.w) <= 3.402823466e38f);
                mx = fmaxf(fmaxf(mx, fmaxf(fabsf(v.x), fabsf(v.y))), fmaxf(fabsf(v.z), fabsf(v.w)));
            }
        }
#pragma unroll
        for (int o = 8; o > 0; o >>= 1) {
            mx = fmaxf(mx, __shfl_xor(mx, o, 16));
            bad |= __shfl_xor(bad, o, 16);
        }
        if (i == 0) {
            int E = 0;
            if (mx > 0.0f) (void)frexpf(mx, &E);  // mx = f * 2^E, f in [0.5, 1)
            const int shift = mx > 0.0f ? 15 - E : 0;
            sh_shift[j] = bad ? INT32_MIN : shift;
            if (blockIdx.y == 0 && m < M) xsh[m] = bad ? INT32_MIN : -shift;
        }
    }
    __syncthreads();
    const uint32_t j = tid & 15u, c = tid >> 4, g = c >> 2, s = c & 3u, m = m0 + j;
    const int shift = sh_shift[j];
    const bool live = m < M && shift != INT32_MIN;
    const uint32_t k0 = FMT == OXB_FMT_Q1 ? 32 * g + 4 * s : 32 * g + 16 * (s >> 1) + 4 * (s & 1u);
    const uint32_t k1 = k0 + (FMT == OXB_FMT_Q1 ? 16 : 8);
    for (uint32_t blk = blockIdx.y; blk < nblk_pad; blk += gridDim.y) {
        uint4 o = make_uint4(0, 0, 0, 0);
        if (live && blk * 128 < k) {
            const float* xb = x + (size_t)m * ldx + blk * 128;
            const float4 a = *reinterpret_cast<const float4*>(xb + k0);
            const float4 b = *reinterpret_cast<const float4*>(xb + k1);
            o.x = pack_h2(ldexpf(a.x, shift), ldexpf(b.x, shift));
            o.y = pack_h2(ldexpf(a.y, shift), ldexpf(b.y, shift));
            o.z = pack_h2(ldexpf(a.z, shift), ldexpf(b.z, shift));
            o.w = pack_h2(ldexpf(a.w, shift), ldexpf(b.w, shift));
        }
        xh[(size_t)(blk * 16 + c) * M_pad + m] = o;
    }
}

// ---------------------------------------------------------------------------
// GEMM.
// ---------------------------------------------------------------------------
template <int FMT, int RT>
struct WeightRegs {
    v4i c[RT][FMT == OXB_FMT_Q1 ? 1 : 2];  // one superblock of codes per row tile
    uint32_t d[RT][4];                     // fp16 scale bits of this lane's row, blocks 0..3 of the superblock
};

template <int FMT, int RT>
__device__ __forceinline__ void load_weights(WeightRegs<FMT, RT>& W, __amdgpu_buffer_rsrc_t rc, __amdgpu_buffer_rsrc_t rs,
                                             uint32_t t0, uint32_t n_valid, uint32_t n_sb, uint32_t sb, uint32_t lane) {
    constexpr uint32_t UNIT = FMT == OXB_FMT_Q1 ? 1024u : 2048u;
    const uint32_t r = lane & 15u;
#pragma unroll
    for (int rt = 0; rt < RT; rt++) {
        const bool ok = (uint32_t)rt < n_valid && sb < n_sb;
        const uint32_t unit = (t0 + rt) * n_sb + sb;
        const uint32_t cv = ok ? lane * 16u : OXB_OOB;
        W.c[rt][0] = buf_load_b128(rc, cv, unit * UNIT);
        if (FMT != OXB_FMT_Q1) W.c[rt][FMT == OXB_FMT_Q1 ? 0 : 1] = buf_load_b128(rc, ok ? lane * 16u + 1024u : OXB_OOB, unit * UNIT);
        const uint32_t sv = ok ? ((r >> 2) * 16u + (r & 3u)) * 2u : OXB_OOB;
#pragma unroll
        for (int q = 0; q < 4; q++)
            W.d[rt][q] = (uint32_t)__builtin_amdgcn_raw_buffer_load_b16(rs, (int)(ok ? sv + q * 8u : OXB_OOB), (int)(unit * 128u), 0);
    }
}

// Per (row tile, block) state prepared once and used by the four MFMA steps of the block.
template <int FMT>
struct BlockDec {
    uint32_t w0, w1;  // Q1: w0 = inverted sign bits (xor the scale's sign); TQ2: fields of halves m = 0, 1 as value+1
    uint32_t d2;      // Q1: |d| in both halves; TQ2: d in both halves
};

template <int FMT>
__device__ __forceinline__ BlockDec<FMT> prepare_block(const v4i (&c)[FMT == OXB_FMT_Q1 ? 1 : 2], uint32_t dbits, int q) {
    BlockDec<FMT> B;
    const uint32_t dd = (dbits & 0xFFFFu) * 0x00010001u;
    if (FMT == OXB_FMT_Q1) {
        // weight = bit ? d : -d  ->  sign bit = ~bit ^ sign(d)
        const uint32_t flip = (uint32_t)((int32_t)(dbits << 16) >> 31);
        B.w0 = ~(uint32_t)c[0][q] ^ flip;
        B.w1 = 0;
        B.d2 = dd & 0x7FFF7FFFu;
    } else {
        // fields at in-byte position 3 are 2-bit two's complement (3, 0, 1 for -1, 0, +1): adding 1 modulo 4
        // turns them into value+1 like the others
        const int half = q >> 1, e = q & 1;
        const uint32_t a = (uint32_t)c[half][2 * e], b = (uint32_t)c[half][2 * e + 1];
        B.w0 = (a & 0x3F3F3F3Fu) | (((a & 0xC0C0C0C0u) + 0x40404040u) & 0xC0C0C0C0u);
        B.w1 = (b & 0x3F3F3F3Fu) | (((b & 0xC0C0C0C0u) + 0x40404040u) & 0xC0C0C0C0u);
        B.d2 = dd;
    }
    return B;
}

// The A operand of MFMA step s (0..3) of the block.
template <int FMT>
__device__ __forceinline__ v8h decode_step(const BlockDec<FMT>& B, int s) {
    uint32_t o[4];
    if (FMT == OXB_FMT_Q1) {
#pragma unroll
        for (int p = 0; p < 4; p++) o[p] = ((B.w0 << (15 - (4 * s + p))) & 0x80008000u) | B.d2;
    } else {
        const uint32_t w = (s >> 1) ? B.w1 : B.w0;
        const v2h dd = __builtin_bit_cast(v2h, B.d2);
        const v2h bias = {(_Float16)1025.0f, (_Float16)1025.0f};
#pragma unroll
        for (int p = 0; p < 4; p++) {
            // 0x6400 | field is the fp16 number 1024 + field; both steps below are exact
            const uint32_t t = ((w >> (2 * (4 * (s & 1) + p))) & 0x00030003u) | 0x64006400u;
            const v2h v = (__builtin_bit_cast(v2h, t) - bias) * dd;
            o[p] = __builtin_bit_cast(uint32_t, v);
        }
    }
    const v4u u = {o[0], o[1], o[2], o[3]};
    return __builtin_bit_cast(v8h, u);
}

template <int FMT, int RT, int CT>
__global__ __launch_bounds__(OXB_GEMM_THREADS) void gemm_mfma_kernel(const OxbGemmParams p) {
    constexpr int BM = 16 * CT;
    __shared__ __attribute__((aligned(16))) uint4 xs[2][16 * BM];
    const uint32_t tid = threadIdx.x, lane = tid & 63u, wave = tid >> 6, r = lane & 15u, g = lane >> 4;
    const uint32_t m_t = blockIdx.x % p.n_mt, n_g = blockIdx.x / p.n_mt;
    const uint32_t m0 = m_t * BM;
    // row tiles: the workgroup's [wg_t0, wg_t1), split evenly over the four waves
    const uint32_t wg_t0 = n_g * p.tpw, wg_t1 = min(wg_t0 + p.tpw, p.n_tiles);
    const uint32_t per = (p.tpw + 3u) / 4u;  // <= RT
    const uint32_t t0 = wg_t0 + wave * per;
    const uint32_t t1 = min(t0 + per, wg_t1);
    const uint32_t n_valid = t1 > t0 ? t1 - t0 : 0u;

    const __amdgpu_buffer_rsrc_t rc = make_rsrc(p.codes, p.codes_bytes), rs = make_rsrc(p.scales, p.scales_bytes);
    const __amdgpu_buffer_rsrc_t rx = make_rsrc(p.xh, p.xh_bytes);

    v4f acc[RT][CT];
#pragma unroll
    for (int rt = 0; rt < RT; rt++)
#pragma unroll
        for (int ct = 0; ct < CT; ct++) acc[rt][ct] = (v4f){0.f, 0.f, 0.f, 0.f};

    // this thread's share of an X stage: CT items of 16 bytes; item id = it*256 + tid -> chunk id / BM, token id % BM
    uint32_t xoff[CT];
#pragma unroll
    for (int it = 0; it < CT; it++) {
        const uint32_t id = it * OXB_GEMM_THREADS + tid, c = id / BM, j = id % BM;
        xoff[it] = m0 + j < p.M_pad ? (c * p.M_pad + m0 + j) * 16u : OXB_OOB;
    }
    const uint32_t blk_stride = 16u * p.M_pad * 16u;  // bytes of xh per block
    const uint32_t nblk = p.n_sb * 4u;

    v4i xr[CT];
#pragma unroll
    for (int it = 0; it < CT; it++) xr[it] = buf_load_b128(rx, xoff[it], 0);
    WeightRegs<FMT, RT> Wn;
    load_weights<FMT, RT>(Wn, rc, rs, t0, n_valid, p.n_sb, 0, lane);
#pragma unroll
    for (int it = 0; it < CT; it++) reinterpret_cast<v4i*>(xs[0])[it * OXB_GEMM_THREADS + tid] = xr[it];
    lds_barrier();

    for (uint32_t sb = 0; sb < p.n_sb; sb++) {
        WeightRegs<FMT, RT> W = Wn;
        load_weights<FMT, RT>(Wn, rc, rs, t0, n_valid, p.n_sb, sb + 1, lane);
#pragma unroll
        for (int q = 0; q < 4; q++) {
            const uint32_t blk = sb * 4 + q;
            const int buf = q & 1;
            const bool more = blk + 1 < nblk;
            if (more) {
#pragma unroll
                for (int it = 0; it < CT; it++) xr[it] = buf_load_b128(rx, xoff[it], (blk + 1) * blk_stride);
            }
            BlockDec<FMT> bd[RT];
#pragma unroll
            for (int rt = 0; rt < RT; rt++) bd[rt] = prepare_block<FMT>(W.c[rt], W.d[rt][q], q);
            const v8h* xsb = reinterpret_cast<const v8h*>(xs[buf]);
#pragma unroll
            for (int s = 0; s < 4; s++) {
                v8h A[RT];
#pragma unroll
                for (int rt = 0; rt < RT; rt++) A[rt] = decode_step<FMT>(bd[rt], s);
#pragma unroll
                for (int ct = 0; ct < CT; ct++) {
                    const v8h B = xsb[(g * 4 + s) * BM + ct * 16 + r];
#pragma unroll
                    for (int rt = 0; rt < RT; rt++)  // row tiles past the range hold zero weights
                        acc[rt][ct] = __builtin_amdgcn_mfma_f32_16x16x32_f16(A[rt], B, acc[rt][ct], 0, 0, 0);
                }
            }
            if (more) {
#pragma unroll
                for (int it = 0; it < CT; it++) reinterpret_cast<v4i*>(xs[buf ^ 1])[it * OXB_GEMM_THREADS + tid] = xr[it];
            }
            lds_barrier();
        }
    }

    // epilogue: lane holds rows 4g..4g+3 of the row tile for token 16ct + r
    const bool vec_ok = (p.ldy & 3u) == 0;
#pragma unroll
    for (int ct = 0; ct < CT; ct++) {
        const uint32_t m = m0 + ct * 16 + r;
        if (m >= p.M) continue;
        const int e = p.xsh[m];
        float* yr = p.y + (size_t)m * p.ldy;
        const float* rr = p.mode == OXB_GEMM_RESIDUAL ? p.residual + (size_t)m * p.ldy : nullptr;
#pragma unroll
        for (int rt = 0; rt < RT; rt++) {
            if ((uint32_t)rt >= n_valid) continue;
            const uint32_t n = (t0 + rt) * 16 + 4 * g;
            float o[4];
#pragma unroll
            for (int v = 0; v < 4; v++) o[v] = e == INT32_MIN ? __int_as_float(0x7FC00000) : ldexpf(acc[rt][ct][v], e);
            if (vec_ok && n + 3 < p.n_rows) {
                if (rr) {
                    const float4 q4 = *reinterpret_cast<const float4*>(rr + n);
                    o[0] += q4.x, o[1] += q4.y, o[2] += q4.z, o[3] += q4.w;
                }
                *reinterpret_cast<float4*>(yr + n) = make_float4(o[0], o[1], o[2], o[3]);
            } else {
#pragma unroll
                for (int v = 0; v < 4; v++)
                    if (n + v < p.n_rows) yr[n + v] = rr ? rr[n + v] + o[v] : o[v];
            }
        }
    }
}

// ---------------------------------------------------------------------------
// Host-side launchers.
// ---------------------------------------------------------------------------
size_t oxb_xh_bytes(uint32_t k, uint32_t M) {
    const size_t nblk_pad = ((k + 511u) / 512u) * 4u, M_pad = (M + 15u) / 16u * 16u;
    return nblk_pad * 16 * M_pad * 16;
}

hipError_t oxb_launch_xh_pack(int fmt, const float* d_x, uint32_t ldx, uint32_t k, uint32_t M, uint32_t* d_xh,
                              int32_t* d_xsh, hipStream_t st) {
    if (M == 0 || k == 0 || (k % OXB_QK) != 0 || (ldx & 3u) != 0) return hipErrorInvalidValue;
    const uint32_t nblk_pad = ((k + 511u) / 512u) * 4u, M_pad = (M + 15u) / 16u * 16u;
    if (oxb_xh_bytes(k, M) >= 0xFFFFFFF0ull) return hipErrorInvalidValue;
    uint32_t split = nblk_pad < 16 ? nblk_pad : 16;
    const dim3 grid(M_pad / 16, split);
    if (fmt == OXB_FMT_Q1)
        hipLaunchKernelGGL(xh_pack_kernel<OXB_FMT_Q1>, grid, dim3(256), 0, st, d_x, ldx, k, M, M_pad, nblk_pad,
                           reinterpret_cast<uint4*>(d_xh), d_xsh);
    else
        hipLaunchKernelGGL(xh_pack_kernel<OXB_FMT_TQ2>, grid, dim3(256), 0, st, d_x, ldx, k, M, M_pad, nblk_pad,
                           reinterpret_cast<uint4*>(d_xh), d_xsh);
    return hipGetLastError();
}

template <int FMT, int RT, int CT>
static hipError_t launch_gemm_case(const OxbGemmParams& p, uint32_t grid, hipStream_t st) {
    hipLaunchKernelGGL((gemm_mfma_kernel<FMT, RT, CT>), dim3(grid), dim3(OXB_GEMM_THREADS), 0, st, p);
    return hipGetLastError();
}

hipError_t oxb_launch_gemm(int fmt, OxbGemmParams p, uint32_t n_cus, hipStream_t st) {
    if (p.M == 0 || p.n_rows == 0) return hipSuccess;
    if (p.n_sb == 0 || (uint64_t)p.n_tiles * p.n_sb * 2048ull >= 0xFFFFFFF0ull) return hipErrorInvalidValue;
    constexpr uint32_t CT = 8, BM = 16 * CT;
    p.M_pad = (p.M + 15u) / 16u * 16u;
    p.n_mt = (p.M + BM - 1) / BM;
    // Row tiles per workgroup: minimise (rounds of workgroups over the CUs) x (row tiles per wave).
    static const uint32_t rts[] = {1, 2, 3, 4, 5};
    uint32_t best_rt = 0, best_tpw = 0;
    uint64_t best_cost = ~0ull;
    for (uint32_t rt : rts) {
        for (uint32_t tpw = 4 * rt; tpw > 4 * rt - 4; tpw--) {
            const uint32_t groups = (p.n_tiles + tpw - 1) / tpw;
            const uint64_t wgs = (uint64_t)groups * p.n_mt;
            const uint64_t cost = ((wgs + n_cus - 1) / n_cus) * rt * 64 + rt;  // ties: fewer tiles per wave
            if (cost < best_cost) best_cost = cost, best_rt = rt, best_tpw = tpw;
        }
    }
    p.tpw = best_tpw;
    const uint32_t grid = ((p.n_tiles + p.tpw - 1) / p.tpw) * p.n_mt;
#define OXB_GEMM_CASE(F, R) \
    if (fmt == F && best_rt == R) return launch_gemm_case<F, R, CT>(p, grid, st);
    OXB_GEMM_CASE(OXB_FMT_Q1, 1)
    OXB_GEMM_CASE(OXB_FMT_Q1, 2)
    OXB_GEMM_CASE(OXB_FMT_Q1, 3)
    OXB_GEMM_CASE(OXB_FMT_Q1, 4)
    OXB_GEMM_CASE(OXB_FMT_Q1, 5)
    OXB_GEMM_CASE(OXB_FMT_TQ2, 1)
    OXB_GEMM_CASE(OXB_FMT_TQ2, 2)
    OXB_GEMM_CASE(OXB_FMT_TQ2, 3)
    OXB_GEMM_CASE(OXB_FMT_TQ2, 4)
    OXB_GEMM_CASE(OXB_FMT_TQ2, 5)
#undef OXB_GEMM_CASE
    return hipErrorInvalidValue;
}
