// quant_device.h — device-side activation quantiser shared by every kernel that feeds a GEMV.
//
// A GEMV input x[k] (fp32) becomes, per vector n of the pass (NC = 8 * vectors columns,
// column c = 8n + digit):
//   xq  [((blk*2+m)*4+g)*NC + c][jj]  one dword = 4 int8 (bb = 0..3), the MFMA B operand of
//        lane (c,g), register jj, of MFMA m of block blk;
//        Q1 : element bb is digit(c%8) of  s_j * 2*r(k),  k = 128blk+32g+8bb+j, j = 4m+jj,
//             r(k) = rint(x[k] * 2^(P-E-j)),  s_j = -1 for j = 7 (0x80 is -128 as int8)
//        TQ2: element bb is digit(c%8) of  r(k) = rint(x[k] * 2^(P-E-2jj)), k = 128blk+32g+16m+4bb+jj
//   cneg[blk][c][0..3]  four copies of -C, C = the part of the block sum that the biased
//        encodings add (Q1: sum_k 2^j digit(r); TQ2: sum_{jj<3} 4^jj digit(r)), used as the
//        MFMA accumulator's start value;
//   xexp[n]  E - P, or INT_MIN when the vector holds a NaN or an infinity,
// where 2^E > max|x| >= 2^(E-1) and P = 53: every element within 2^22 of the largest keeps all
// 24 mantissa bits, so the integer block sums are exact for practical inputs.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "device_utils.h"
#include "layout.h"

#define OXB_XQ_P 53  // |x * 2^(P-E)| < 2^53, doubled values stay below 2^54
#define OXB_XQ_DIGITS 8

__device__ __forceinline__ int oxb_not_finite(float v) { return !(fabsf(v) <= 3.402823466e38f); }

// rint(v * 2^shift) as a 64-bit integer, using fp32 operations only.  Scaling by a power of
// two is exact, rintf is exact, and the split at 2^27 leaves two parts that fit an int32.
__device__ __forceinline__ long long scaled_rint_i64(float v, int shift) {
    const float r = rintf(ldexpf(v, shift));              // |r| < 2^54, an integer
    const float hi = truncf(r * 7.450580596923828e-09f);  // r / 2^27
    const float lo = r - hi * 134217728.0f;               // exact: |lo| < 2^27
    return ((long long)(int)hi << 27) + (long long)(int)lo;
}

// Transpose a 4 x 4 byte matrix held in four dwords: o[d] = { t[0].byte d, t[1].byte d, t[2].byte d, t[3].byte d }.
__device__ __forceinline__ void transpose_bytes4(const uint32_t t[4], uint32_t o[4]) {
    const uint32_t p01l = __builtin_amdgcn_perm(t[1], t[0], 0x05010400u), p01h = __builtin_amdgcn_perm(t[1], t[0], 0x07030602u);
    const uint32_t p23l = __builtin_amdgcn_perm(t[3], t[2], 0x05010400u), p23h = __builtin_amdgcn_perm(t[3], t[2], 0x07030602u);
    o[0] = __builtin_amdgcn_perm(p23l, p01l, 0x05040100u);
    o[1] = __builtin_amdgcn_perm(p23l, p01l, 0x07060302u);
    o[2] = __builtin_amdgcn_perm(p23h, p01h, 0x05040100u);
    o[3] = __builtin_amdgcn_perm(p23h, p01h, 0x07060302u);
}

// Balanced base-256 digits of four 64-bit integers, digit-major: dig[d] = one dword holding digit d of
// v[0..3] as int8.  Adding 0x80 to every byte below the top one and flipping that bit back turns
// the two's-complement bytes into signed digits in [-128, 127] with the carries propagated.
__device__ __forceinline__ void digits_of4(const long long v[4], uint32_t dig[8]) {
    const unsigned long long bias = 0x0080808080808080ull;
    uint32_t lo[4], hi[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const unsigned long long t = ((unsigned long long)v[i] + bias) ^ bias;
        lo[i] = (uint32_t)t;
        hi[i] = (uint32_t)(t >> 32);
    }
    transpose_bytes4(lo, dig);
    transpose_bytes4(hi, dig + 4);
}

// Quantise the 16 activations that one lane group (blk, m, g) of the MFMA B operand holds and
// store their eight digit planes; cs[d] returns this group's share of the block's correction sums.
template <int FMT>
__device__ __forceinline__ void quant_unit(const float* __restrict__ xn, uint32_t blk, uint32_t m, uint32_t g,
                                           int base_shift, bool live, uint32_t NC, uint32_t n,
                                           uint32_t* __restrict__ xq, int cs[8]) {
    uint32_t out[8][4];
#pragma unroll
    for (int d = 0; d < 8; d++) {
        cs[d] = 0;
        out[d][0] = out[d][1] = out[d][2] = out[d][3] = 0;
    }
    if (live) {
        const float* xb = xn + blk * 128 + 32 * g;
        float vv[4][4];  // [bb][jj]
#pragma unroll
        for (uint32_t bb = 0; bb < 4; bb++) {
            // Q1: k = 8bb + 4m + jj;  TQ2: k = 16m + 4bb + jj   (jj = 0..3 contiguous)
            const float4 v4 = *reinterpret_cast<const float4*>(xb + (FMT == OXB_FMT_Q1 ? 8 * bb + 4 * m : 16 * m + 4 * bb));
            vv[bb][0] = v4.x;
            vv[bb][1] = v4.y;
            vv[bb][2] = v4.z;
            vv[bb][3] = v4.w;
        }
#pragma unroll
        for (uint32_t jj = 0; jj < 4; jj++) {
            long long xi[4], cr[4];
            uint32_t dig[8], cdig[8];
            if (FMT == OXB_FMT_Q1) {
                const uint32_t j = 4 * m + jj;
#pragma unroll
                for (int bb = 0; bb < 4; bb++) {
                    cr[bb] = scaled_rint_i64(vv[bb][jj], base_shift - (int)j);
                    xi[bb] = (j == 7) ? -2 * cr[bb] : 2 * cr[bb];
                }
                digits_of4(xi, dig);
                digits_of4(cr, cdig);
#pragma unroll
                for (int d = 0; d < 8; d++) cs[d] += __builtin_amdgcn_sdot4((int)cdig[d], 0x01010101, 0, false) << j;
            } else {
#pragma unroll
                for (int bb = 0; bb < 4; bb++) xi[bb] = scaled_rint_i64(vv[bb][jj], base_shift - 2 * (int)jj);
                digits_of4(xi, dig);
                if (jj < 3) {
#pragma unroll
                    for (int d = 0; d < 8; d++) cs[d] += __builtin_amdgcn_sdot4((int)dig[d], 0x01010101, 0, false) << (2 * jj);
                }
            }
#pragma unroll
            for (int d = 0; d < 8; d++) out[d][jj] = dig[d];
        }
    }
    uint4* dst = reinterpret_cast<uint4*>(xq) + (size_t)((blk * 2 + m) * 4 + g) * NC + 8 * n;
#pragma unroll
    for (int d = 0; d < 8; d++) dst[d] = make_uint4(out[d][0], out[d][1], out[d][2], out[d][3]);
}

// Workgroup-wide maximum of |x| and a "not finite" flag; `red` holds blockDim.x / 64 floats.
// Every thread gets the results.  Contains two barriers.
__device__ __forceinline__ float block_absmax(float mx, int bad, float* red, int* bad_flag, bool* any_bad) {
    const uint32_t tid = threadIdx.x, nw = blockDim.x >> 6;
    if (tid == 0) *bad_flag = 0;
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
    if ((tid & 63u) == 0) red[tid >> 6] = mx;
    __syncthreads();
    if (bad) *bad_flag = 1;
    mx = red[0];
    for (uint32_t i = 1; i < nw; i++) mx = fmaxf(mx, red[i]);
    __syncthreads();
    *any_bad = *bad_flag != 0;
    return mx;
}

// Quantise vector n (values at xn[0..k), any address space) given its absolute maximum.
// All threads of the workgroup call it; blockDim.x must be a multiple of 64.  Workgroup
// (part of parts) takes an equal share of the 64-unit groups, so several workgroups can split
// one vector after each has found the same maximum.
template <int FMT>
__device__ __forceinline__ void quantise_vector(const float* __restrict__ xn, uint32_t k, uint32_t nblk_pad,
                                                uint32_t NC, uint32_t n, float mx, bool any_bad,
                                                uint32_t* __restrict__ xq, int32_t* __restrict__ cneg,
                                                int32_t* __restrict__ xexp, uint32_t part = 0, uint32_t parts = 1) {
    int E = 0;
    if (mx > 0.0f) (void)frexpf(mx, &E);  // mx = f * 2^E, f in [0.5, 1)
    const int base_shift = OXB_XQ_P - E;
    const uint32_t nblk = k / OXB_QK;
    const bool ok = mx > 0.0f && !any_bad;
    // unit u = (blk, m, g): eight consecutive lanes cover one block
    const uint32_t n_units = nblk_pad * 8, per = (((n_units + 63) / 64 + parts - 1) / parts) * 64;  // n_units % 32 == 0
    const uint32_t u_end = (part + 1) * per < n_units ? (part + 1) * per : n_units;
    for (uint32_t u = part * per + threadIdx.x; u < u_end; u += blockDim.x) {
        const uint32_t blk = u >> 3, m = (u >> 2) & 1u, g = u & 3u;
        int cs[8];
        quant_unit<FMT>(xn, blk, m, g, base_shift, ok && blk < nblk, NC, n, xq, cs);
        // sum the correction over the block's eight lanes: i <-> 7-i, then within quads
#pragma unroll
        for (int d = 0; d < 8; d++) {
            int v = cs[d];
            v += dpp_i32<0x141>(v);  // row_half_mirror
            v += dpp_i32<0xB1>(v);   // quad_perm [1,0,3,2]
            v += dpp_i32<0x4E>(v);   // quad_perm [2,3,0,1]
            cs[d] = v;
        }
        // lane j of the eight writes digit j (four copies: the MFMA takes it as a 4-register operand)
        int mine = cs[0];
#pragma unroll
        for (int d = 1; d < 8; d++) mine = ((u & 7u) == (uint32_t)d) ? cs[d] : mine;
        *reinterpret_cast<int4*>(cneg + ((size_t)blk * NC + 8 * n + (u & 7u)) * 4) = make_int4(-mine, -mine, -mine, -mine);
    }
    if (threadIdx.x == 0 && part == 0) xexp[n] = any_bad ? INT32_MIN : (mx > 0.0f ? E - OXB_XQ_P : 0);
}

// Workgroups that share one vector: one per 64 units (1024 activations), at most 16.
__host__ __device__ inline uint32_t oxb_quant_parts(uint32_t k) {
    const uint32_t p = (((k + 511u) / 512u) * 32u + 63u) / 64u;
    return p < 1 ? 1 : (p > 16 ? 16 : p);
}

__host__ __device__ inline uint32_t oxb_nblk_pad(uint32_t k) { return ((k + 511u) / 512u) * 4u; }
