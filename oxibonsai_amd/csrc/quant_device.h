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
//   xexp[n][group]  E - P of the exponent group, or INT_MIN when the group holds a NaN or an infinity,
// where 2^E > max|x| >= 2^(E-1) over the group and P = 53: every element within 2^22 of the group's
// largest keeps all 24 mantissa bits, so the integer block sums are exact for practical inputs.
// An exponent group is the K slice one GEMV wave owns (oxb_xq_gsb superblocks of 512 activations): its
// exponent needs no information from the rest of the vector, so a producer of activations can quantise the
// slice it has just computed, and the GEMV applies the exponent when it adds the waves' partial sums.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "device_utils.h"
#include "layout.h"

#define OXB_XQ_P 53  // |x * 2^(P-E)| < 2^53, doubled values stay below 2^54
#define OXB_XQ_DIGITS 8

__host__ __device__ inline uint32_t oxb_nblk_pad(uint32_t k) { return ((k + 511u) / 512u) * 4u; }

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

// Offset (in floats, from the start of the block's 32-weight group g) of the four consecutive activations
// jj = 0..3 that byte position bb of MFMA m pairs with:  Q1: k = 8bb + 4m + jj;  TQ2: k = 16m + 4bb + jj.
template <int FMT>
__device__ __forceinline__ uint32_t unit_val_offset(uint32_t m, uint32_t bb) {
    return FMT == OXB_FMT_Q1 ? 8 * bb + 4 * m : 16 * m + 4 * bb;
}

// One lane's share of the quantiser: the four activations v[bb] that register jj of lane group (blk, m, g) of the
// MFMA B operand packs into one dword.  dig[d] = that dword of digit plane d; cs[d] = this lane's share of the
// block's correction sums.  Zeros in give zeros out.
template <int FMT>
__device__ __forceinline__ void quant_quarter(const float (&v)[4], uint32_t m, uint32_t jj, int base_shift,
                                              uint32_t (&dig)[8], int (&cs)[8]) {
    long long xi[4];
    if (FMT == OXB_FMT_Q1) {
        const uint32_t j = 4 * m + jj;
        long long cr[4];
        uint32_t cdig[8];
#pragma unroll
        for (int bb = 0; bb < 4; bb++) {
            cr[bb] = scaled_rint_i64(v[bb], base_shift - (int)j);
            xi[bb] = (j == 7) ? -2 * cr[bb] : 2 * cr[bb];
        }
        digits_of4(xi, dig);
        digits_of4(cr, cdig);
#pragma unroll
        for (int d = 0; d < 8; d++) cs[d] = __builtin_amdgcn_sdot4((int)cdig[d], 0x01010101, 0, false) << j;
    } else {
#pragma unroll
        for (int bb = 0; bb < 4; bb++) xi[bb] = scaled_rint_i64(v[bb], base_shift - 2 * (int)jj);
        digits_of4(xi, dig);
#pragma unroll
        for (int d = 0; d < 8; d++) cs[d] = jj < 3 ? __builtin_amdgcn_sdot4((int)dig[d], 0x01010101, 0, false) << (2 * jj) : 0;
    }
}

// Sum the correction shares over the 32 lanes of a block (consecutive lanes starting at a multiple of 32) with a
// halving exchange: every step a lane keeps half of its digits and receives the partner's share of those.
// Returns, in every lane, the block's sum of digit 4 * bit0 + 2 * bit1 + bit2 of the lane index.
__device__ __forceinline__ int block_correction32(const int (&cs)[8], uint32_t lane_in_block) {
    const bool b0 = lane_in_block & 1u, b1 = lane_in_block & 2u, b2 = lane_in_block & 4u;
    int r[4], s[2];
#pragma unroll
    for (int d = 0; d < 4; d++) r[d] = (b0 ? cs[d + 4] : cs[d]) + dpp_i32<0xB1>(b0 ? cs[d] : cs[d + 4]);  // quad_perm [1,0,3,2]
#pragma unroll
    for (int d = 0; d < 2; d++) s[d] = (b1 ? r[d + 2] : r[d]) + dpp_i32<0x4E>(b1 ? r[d] : r[d + 2]);      // quad_perm [2,3,0,1]
    int t = (b2 ? s[1] : s[0]) + __shfl_xor(b2 ? s[0] : s[1], 4, 64);
    t += __shfl_xor(t, 8, 64);
    t += __shfl_xor(t, 16, 64);
    return t;
}

// Superblocks per exponent group and groups per vector of n_sb superblocks: the K slice of one GEMV wave
// (eight waves share up to 24 superblocks; longer vectors take several launches of 3-superblock slices).
__host__ __device__ inline uint32_t oxb_xq_gsb(uint32_t n_sb) {
    const uint32_t g = (n_sb + 7u) / 8u;
    return g < 1 ? 1 : (g > 3 ? 3 : g);
}
__host__ __device__ inline uint32_t oxb_xq_groups(uint32_t n_sb) {
    const uint32_t gsb = oxb_xq_gsb(n_sb);
    return n_sb ? (n_sb + gsb - 1) / gsb : 1;
}
#define OXB_XQ_MAX_GROUPS 64  // vectors up to 64 * 3 * 512 = 98304 activations

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

// Group statistics kept in LDS by a quantising workgroup: gstat[2 * i] = bit pattern of the largest |x| of
// its i-th group (non-negative floats order like their bit patterns), gstat[2 * i + 1] = "not finite" flag.
__device__ __forceinline__ void gstat_clear(uint32_t* gstat, uint32_t n_groups_here) {
    for (uint32_t i = threadIdx.x; i < 2 * n_groups_here; i += blockDim.x) gstat[i] = 0;
}
// Every lane of a wave passes values of the same group (a wave covers 256 consecutive activations at a
// 256-aligned index, and groups are multiples of 512).
__device__ __forceinline__ void gstat_update_wave(uint32_t* gstat, uint32_t local_group, float mx, int bad) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        mx = fmaxf(mx, __shfl_xor(mx, o, 64));
        bad |= __shfl_xor(bad, o, 64);
    }
    if ((threadIdx.x & 63u) == 0) {
        atomicMax(&gstat[2 * local_group], __float_as_uint(mx));
        if (bad) atomicOr(&gstat[2 * local_group + 1], 1u);
    }
}

// Maxima of groups [g_begin, g_end) of the values xn[0..k) (any address space) into gstat.  All threads of
// the workgroup call it; blockDim.x is a multiple of 64.  Ends with a barrier.
__device__ __forceinline__ void gstat_scan(const float* __restrict__ xn, uint32_t k, uint32_t gsb, uint32_t g_begin,
                                           uint32_t g_end, uint32_t* gstat) {
    gstat_clear(gstat, g_end - g_begin);
    __syncthreads();
    const uint32_t gel = gsb * 512u, e0 = g_begin * gel, e1 = g_end * gel < k ? g_end * gel : k;
    for (uint32_t base = e0 + (threadIdx.x >> 6) * 256u; base < e1; base += (blockDim.x >> 6) * 256u) {
        const uint32_t i = base + (threadIdx.x & 63u) * 4u;
        float mx = 0.f;
        int bad = 0;
        if (i < e1) {  // k is a multiple of 128
            const float4 v = *reinterpret_cast<const float4*>(xn + i);
            bad = oxb_not_finite(v.x) | oxb_not_finite(v.y) | oxb_not_finite(v.z) | oxb_not_finite(v.w);
            mx = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
        }
        gstat_update_wave(gstat, base / gel - g_begin, mx, bad);
    }
    __syncthreads();
}

// Quantise groups [g_begin, g_end) of vector n (values at xn[0..k), any address space) given their statistics
// in gstat (published by a barrier).  All threads of the workgroup call it.
template <int FMT>
__device__ __forceinline__ void quantise_groups(const float* __restrict__ xn, uint32_t k, uint32_t NC, uint32_t n,
                                                uint32_t gsb, uint32_t n_groups, uint32_t g_begin, uint32_t g_end,
                                                const uint32_t* gstat, uint32_t* __restrict__ xq,
                                                int32_t* __restrict__ cneg, int32_t* __restrict__ xexp) {
    const uint32_t nblk = k / OXB_QK, nblk_pad = oxb_nblk_pad(k);
    // Lane q = (unit u = (blk, m, g), register jj): 32 consecutive lanes cover one block; a group holds gsb * 32
    // units.  Group and padding boundaries are multiples of 32 lanes, so the lanes of a block leave the loop together.
    const uint32_t upg = gsb * 32u, u0 = g_begin * upg;
    const uint32_t u1 = g_end * upg < nblk_pad * 8u ? g_end * upg : nblk_pad * 8u;
    for (uint32_t q = u0 * 4u + threadIdx.x; q < u1 * 4u; q += blockDim.x) {
        const uint32_t u = q >> 2, jj = q & 3u;
        const uint32_t blk = u >> 3, m = (u >> 2) & 1u, g = u & 3u, lg = u / upg - g_begin;
        const float mx = __uint_as_float(gstat[2 * lg]);
        const bool live = mx > 0.0f && gstat[2 * lg + 1] == 0 && blk < nblk;
        int E = 0;
        if (mx > 0.0f) (void)frexpf(mx, &E);  // mx = f * 2^E, f in [0.5, 1)
        float v[4];
#pragma unroll
        for (uint32_t bb = 0; bb < 4; bb++) v[bb] = live ? xn[blk * 128 + 32 * g + unit_val_offset<FMT>(m, bb) + jj] : 0.f;
        uint32_t dig[8];
        int cs[8];
        quant_quarter<FMT>(v, m, jj, OXB_XQ_P - E, dig, cs);
        uint32_t* dst = xq + ((size_t)((blk * 2 + m) * 4 + g) * NC + 8 * n) * 4 + jj;
#pragma unroll
        for (int d = 0; d < 8; d++) dst[4 * d] = dig[d];
        // the first eight lanes of the block write one digit's correction each (four copies: the MFMA takes it
        // as a 4-register operand)
        const int mine = block_correction32(cs, q & 31u);
        if ((q & 24u) == 0) {
            const uint32_t d = ((q & 1u) << 2) | (q & 2u) | ((q >> 2) & 1u);
            *reinterpret_cast<int4*>(cneg + ((size_t)blk * NC + 8 * n + d) * 4) = make_int4(-mine, -mine, -mine, -mine);
        }
    }
    for (uint32_t gi = g_begin + threadIdx.x; gi < g_end; gi += blockDim.x) {
        const float mx = __uint_as_float(gstat[2 * (gi - g_begin)]);
        int E = 0;
        if (mx > 0.0f) (void)frexpf(mx, &E);
        xexp[n * n_groups + gi] = gstat[2 * (gi - g_begin) + 1] ? INT32_MIN : (mx > 0.0f ? E - OXB_XQ_P : 0);
    }
}

