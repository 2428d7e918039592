// gemv_pack_device.h - what the packed GEMV route's quantiser and its users share: the fixed point of the quantised
// activations, the packed layout, and the device function that turns the 512 activations of one superblock of one
// vector - eight per lane of one wave - into the GEMV's int8 MFMA operands.  gemv_pack_kernel (gemv_kernels.hip) calls
// it with values loaded from a vector in memory; the decode attention kernel (layer_kernels.hip) with the output it has
// just merged for a kv head, where that is exactly one superblock of the O projection's input.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "device_utils.h"
#include "layout.h"

// 4 x 4 byte transpose: o[d] = { t[0].byte d, t[1].byte d, t[2].byte d, t[3].byte d }.
__device__ __forceinline__ void transpose_bytes4(const uint32_t t[4], uint32_t o[4]) {
    const uint32_t p01l = __builtin_amdgcn_perm(t[1], t[0], 0x05010400u), p01h = __builtin_amdgcn_perm(t[1], t[0], 0x07030602u);
    const uint32_t p23l = __builtin_amdgcn_perm(t[3], t[2], 0x05010400u), p23h = __builtin_amdgcn_perm(t[3], t[2], 0x07030602u);
    o[0] = __builtin_amdgcn_perm(p23l, p01l, 0x05040100u);
    o[1] = __builtin_amdgcn_perm(p23l, p01l, 0x07060302u);
    o[2] = __builtin_amdgcn_perm(p23h, p01h, 0x05040100u);
    o[3] = __builtin_amdgcn_perm(p23h, p01h, 0x07060302u);
}

// Unsigned maximum over the 64 lanes of a wave (in every lane) and integer sum over the 32 lanes of a half wave
// (lanes 0-31, 32-63).  Zero is the identity of both, so the DPP moves (which hand 0 to a lane without a source) fold
// into the arithmetic; the rows of the maximum meet through the lane-swap instructions, not through LDS.
__device__ __forceinline__ uint32_t wave_umax(uint32_t v) {
    v = max(v, dpp_u32<0xB1>(v));    // quad_perm [1,0,3,2]
    v = max(v, dpp_u32<0x4E>(v));    // quad_perm [2,3,0,1]
    v = max(v, dpp_u32<0x141>(v));   // row_half_mirror
    v = max(v, dpp_u32<0x140>(v));   // row_mirror
    const auto a = __builtin_amdgcn_permlane16_swap(v, v, false, false);
    v = max(a[0], a[1]);
    const auto b = __builtin_amdgcn_permlane32_swap(v, v, false, false);
    return max(b[0], b[1]);
}
__device__ __forceinline__ int half_isum(int v) {
    v += dpp_i32<0xB1>(v);
    v += dpp_i32<0x4E>(v);
    v += dpp_i32<0x141>(v);
    v += dpp_i32<0x140>(v);
    return v + __builtin_amdgcn_ds_swizzle(v, 0x401F);
}

// Fixed point of the quantised activations.  2^E > max |x| of a wave's K slice, r = rint(x * 2^(P - E - s)) with s the
// power of two the weight's operand byte carries (Q1: bit j of a code byte is worth 2^(j & 3), the high nibble being
// masked after a shift by 4; TQ2: field jj is worth 4^jj).  Q1 operands hold 2 r (weights are 2 b - 1), so
// |operand| < 2^30 needs P = 29; TQ2 P = 30.
template <int FMT>
struct Fix {
    static constexpr int P = (FMT == OXB_FMT_Q1) ? 29 : 30;
    __device__ static __forceinline__ int shift_of(uint32_t j) { return FMT == OXB_FMT_Q1 ? (int)(j & 3u) : 2 * (int)(j & 3u); }
};

// Packed layout, dwords, for n_sb superblocks and nvg groups of four vectors, unit = vg * n_sb + sb:
//   A   [unit][q * 2 + m][lane][4]      C4 [unit][q][v][4]      EX [unit][v]      SS [unit][v]      CL [unit][q][v][2]
// (A = the operands of the eight MFMAs of a superblock, lane l's 16 bytes at l * 16; C4 = accumulator start values; EX =
// the superblock's power of two; SS = sum of squares; CL = the start values folded as the kernel joins the digit sums,
// d0 + 256 d1 and d2 + 256 d3).  An all-zero buffer is the packed form of zero vectors.
#define OXB_GEMV_EX_BAD 0x7FFFFFFF  // exponent entry of a (superblock, vector) that holds an infinity or a NaN

__host__ __device__ inline size_t oxb_gemv_pack_dwords(uint32_t n_sb, uint32_t nvg) {
    return (size_t)nvg * n_sb * (2048 + 64 + 4 + 4 + 32);
}

// Lane l of the packing wave holds, as xe[pass][bb], the activation at this element of the superblock (0 .. 511):
// block 2 pass + (l >> 5); within it group gg = (l >> 3) & 3 of 32 and j = l & 7: Q1 32 gg + j + 8 bb,
// TQ2 32 gg + 16 (j >> 2) + (j & 3) + 4 bb.
template <int FMT>
__device__ __forceinline__ uint32_t gemv_pack_elem(uint32_t lane, int pass, int bb) {
    const uint32_t j = lane & 7u, gg = (lane >> 3) & 3u, blh = lane >> 5;
    const uint32_t in_block = FMT == OXB_FMT_Q1 ? 32 * gg + j + 8u * bb : 32 * gg + 16 * (j >> 2) + (j & 3u) + 4u * bb;
    return (pass * 2 + blh) * 128u + in_block;
}

// One wave: quantises the superblock's activations xe (norm weights already multiplied in; ss = the wave's sum of the
// squares of the raw values for the RMSNorm prologue, else 0) and writes the operands of (superblock sb, vector vec)
// into the packed buffer `out` of n_sb superblocks and nvg vector groups.
template <int FMT>
__device__ __forceinline__ void gemv_pack_write(float (&xe)[2][4], float ss, uint32_t lane, uint32_t sb, uint32_t vec, uint32_t n_sb,
                                                uint32_t nvg, uint32_t* __restrict__ out) {
    const uint32_t vg = vec >> 2, v = vec & 3u;
    const uint32_t unit = vg * n_sb + sb, units = nvg * n_sb;
    uint32_t* A = out + (size_t)unit * 2048;
    int* C4 = (int*)(out + (size_t)units * 2048 + (size_t)unit * 64);
    int* EXo = (int*)(out + (size_t)units * (2048 + 64) + (size_t)unit * 4);
    float* SSo = (float*)(out + (size_t)units * (2048 + 64 + 4) + (size_t)unit * 4);
    int* CL = (int*)(out + (size_t)units * (2048 + 64 + 4 + 4) + (size_t)unit * 32);
    const uint32_t j = lane & 7u, gg = (lane >> 3) & 3u, blh = lane >> 5;
    const int js = Fix<FMT>::shift_of(j);
    uint32_t mxb = 0;
#pragma unroll
    for (int pass = 0; pass < 2; pass++)
#pragma unroll
        for (int bb = 0; bb < 4; bb++) mxb = max(mxb, __float_as_uint(xe[pass][bb]) & 0x7FFFFFFFu);
    mxb = (uint32_t)__builtin_amdgcn_readfirstlane((int)wave_umax(mxb));
    const bool bad = mxb >= 0x7F800000u;
    const uint32_t be = mxb >> 23;
    const int E = (int)(be ? be : 1u) - 126;  // 2^E > max |x| (subnormal maxima share the smallest E)
    const int sh = Fix<FMT>::P - E - js;
#pragma unroll
    for (int pass = 0; pass < 2; pass++) {
        const uint32_t bl = pass * 2 + blh;
        int r[4];
#pragma unroll
        for (int bb = 0; bb < 4; bb++) r[bb] = bad ? 0 : (int)rintf(ldexpf(xe[pass][bb], sh));
        uint32_t tb[4];
        int cl = (r[0] & 0x7FFF) + (r[1] & 0x7FFF) + (r[2] & 0x7FFF) + (r[3] & 0x7FFF);
        int ch = (r[0] >> 15) + (r[1] >> 15) + (r[2] >> 15) + (r[3] >> 15);
        if (FMT == OXB_FMT_Q1) {
#pragma unroll
            for (int bb = 0; bb < 4; bb++) tb[bb] = (((uint32_t)r[bb] << 1) + 0x00808080u) ^ 0x00808080u;
        } else {
#pragma unroll
            for (int bb = 0; bb < 4; bb++) tb[bb] = ((uint32_t)r[bb] + 0x00808080u) ^ 0x00808080u;
            if ((j & 3u) == 3u) cl = 0, ch = 0;  // field 3 is two's complement: no bias
        }
        cl = half_isum(cl << js), ch = half_isum(ch << js);
        uint32_t D[4];
        transpose_bytes4(tb, D);
        const uint32_t m = j >> 2, jj = j & 3u;
#pragma unroll
        for (int d = 0; d < 4; d++) A[(((bl * 2 + m) * 64 + gg * 16 + 4 * v + d) << 2) + jj] = D[d];
        if ((lane & 31u) == 0) {
            const long long nc = -(((long long)ch << 15) + cl);  // as three balanced digits and a remainder
            const unsigned long long t = ((unsigned long long)nc + 0x808080ull) ^ 0x808080ull;
            const v4i c4 = {(int)(signed char)(t & 0xFF), (int)(signed char)((t >> 8) & 0xFF), (int)(signed char)((t >> 16) & 0xFF),
                            (int)((long long)t >> 24)};
            *reinterpret_cast<v4i*>(C4 + (bl * 4 + v) * 4) = c4;
            CL[(bl * 4 + v) * 2] = c4[0] + (int)((uint32_t)c4[1] << 8);
            CL[(bl * 4 + v) * 2 + 1] = c4[2] + (int)((uint32_t)c4[3] << 8);
        }
    }
    if (lane == 0) {
        EXo[v] = bad ? OXB_GEMV_EX_BAD : (mxb ? E - Fix<FMT>::P : 0);
        SSo[v] = ss;
    }
}
