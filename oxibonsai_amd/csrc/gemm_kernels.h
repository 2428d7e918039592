// gemm_kernels.h — launch interface of the prefill GEMM (fp16 MFMA) and its activation packer.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "layout.h"

// STORE: y = W a;  RESIDUAL: y = residual + W a;  SWIGLU: W = gate || up (n_rows = 2 * inter, a multiple of 32),
// y[m][i] = silu(gate_i . a) * (up_i . a) for i < inter, ldy >= inter.
enum { OXB_GEMM_STORE = 0, OXB_GEMM_RESIDUAL = 2, OXB_GEMM_SWIGLU = 3 };
#define OXB_GEMM_NARROW_MAX_M 32  // up to this many token rows the narrow kernel (K split over waves) is used

struct OxbGemmParams {
    const uint32_t* codes;   // resident codes section
    const uint16_t* scales;  // resident scales section
    const uint32_t* xh;      // packed fp16 activations (oxb_launch_xh_pack)
    const int32_t* xsh;      // [M] exponent that undoes the row scaling, INT32_MIN for a non-finite row
    float* y;                // [M][ldy]
    const float* residual;   // [M][ldy], mode RESIDUAL only
    uint32_t n_rows, n_tiles, n_sb;
    uint32_t M, M_pad;       // token rows, and that count rounded up to 16
    uint32_t ldy;
    uint32_t tpw;            // row tiles per workgroup   (filled by the launcher)
    uint32_t n_mt;           // token tiles of the launch (filled by the launcher)
    uint32_t n_ng;           // row groups of the launch  (filled by the launcher)
    uint32_t ksplit, sb_per_split;  // K slices and superblocks per slice (filled by the launcher)
    float* part;             // [ksplit][M][ldy] partial sums, needed when oxb_gemm_ksplit(...) > 1
    uint32_t codes_bytes, scales_bytes, xh_bytes;  // buffer extents (loads beyond them read 0)
    int mode;
};

// Bytes of the packed activation buffer for M token rows of length k.
size_t oxb_xh_bytes(uint32_t k, uint32_t M);

// Activations a[M][k] -> fp16 in MFMA B-operand order, each row scaled by a power of two so that its largest
// element lies in [2^14, 2^15).  The activations are computed on the fly from x[M][ldx] by `op`:
//   IDENT: a = x;  RMSNORM: a = w * x / rms(x) (w = d_w[k]).
// d_rowmul: M floats of scratch (the multiplier applied to every row).
enum { OXB_PACK_IDENT = 0, OXB_PACK_RMSNORM = 1 };
hipError_t oxb_launch_xh_pack(int fmt, int op, const float* d_x, const float* d_w, uint32_t ldx, uint32_t k, float eps,
                              uint32_t M, float* d_rowmul, uint32_t* d_xh, int32_t* d_xsh, hipStream_t st);
// Number of K slices the launcher will use for this shape (1: no workspace needed).
uint32_t oxb_gemm_ksplit(const OxbGemmParams& p, uint32_t n_cus);
hipError_t oxb_launch_gemm(int fmt, OxbGemmParams p, uint32_t n_cus, hipStream_t st);
