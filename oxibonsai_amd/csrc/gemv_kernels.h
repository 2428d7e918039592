// gemv_kernels.h — launch interface of the GEMV / quantiser / dequant kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "layout.h"

#define OXB_GEMV_MAX_BATCH 2  // activation vectors per pass over the weights
#define OXB_GEMV_MAX_SB 24    // superblocks (512 weights of K) one launch covers: 8 waves x 3
enum { OXB_GEMV_STORE = 0, OXB_GEMV_ACCUM = 1, OXB_GEMV_RESIDUAL = 2 };

struct OxbGemvParams {
    const uint32_t* codes;   // resident codes section
    const uint16_t* scales;  // resident scales section
    const uint32_t* xq;      // digit planes   (oxb_launch_quant_x)
    const int32_t* cneg;     // accumulator start values
    const int32_t* xexp;     // [batch][n_groups] exponents of the K slices (exponent groups)
    float* y;                // [batch][ldy]
    const float* residual;   // [batch][ldy], mode RESIDUAL only
    uint32_t n_rows, n_tiles, n_sb;
    uint32_t sb_begin, sb_count;  // K range handled by this launch, in superblocks
    uint32_t NC;                  // 8 * batch, batch <= 2 (eight digit columns per vector)
    uint32_t ldy;
    uint32_t groups;              // filled by the launcher: groups of in-flight tiles per workgroup
    uint32_t n_groups;            // filled by the launcher: exponent groups per input vector
    uint32_t codes_bytes, scales_bytes, xq_bytes, cneg_bytes;  // buffer extents (loads beyond them read 0)
    int mode;
};

size_t oxb_xq_bytes(uint32_t k, uint32_t batch);
size_t oxb_cneg_bytes(uint32_t k, uint32_t batch);
#define OXB_XEXP_BYTES (2 * 64 * sizeof(int32_t))  // exponents of a pass: OXB_GEMV_MAX_BATCH vectors x up to 64 groups

hipError_t oxb_launch_quant_x(int fmt, const float* d_x, uint32_t k, uint32_t batch, uint32_t* d_xq, int32_t* d_cneg,
                              int32_t* d_xexp, hipStream_t st);
hipError_t oxb_launch_gemv(int fmt, OxbGemvParams p, uint32_t n_cus, hipStream_t st);
hipError_t oxb_launch_dequant(const OxbLayout& L, const uint32_t* d_codes, const uint16_t* d_scales, float* d_out,
                              hipStream_t st);
