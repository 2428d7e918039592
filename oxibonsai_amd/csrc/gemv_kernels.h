// gemv_kernels.h — launch interface of the GEMV / dequant kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "layout.h"

#define OXB_GEMV_MAX_BATCH 4         // activation vectors per pass over the weights when the kernel quantises them itself
#define OXB_GEMV_PACKED_MAX_BATCH 8  // ... when oxb_launch_gemv_pack has quantised them (OxbGemvParams::xq)
#define OXB_GEMV_MAX_SB 24    // superblocks (512 weights of K) one launch covers: 8 waves x 3

// What the kernel's prologue does with x before quantising it, and what its epilogue does with the row sums.
enum { OXB_GEMV_PRO_F32 = 0,        // a = x
       OXB_GEMV_PRO_RMSNORM = 1 };  // a = norm_w * x / sqrt(mean(x^2) + eps)        (simd_float_ops.rs:204-215)
enum { OXB_GEMV_STORE = 0,          // y = W a
       OXB_GEMV_ACCUM = 1,          // y += W a
       OXB_GEMV_RESIDUAL = 2,       // y = residual + W a
       OXB_GEMV_SWIGLU = 3 };       // W = gate || up (n_rows = 2 * inter): y[i] = silu(gate_i . a) * (up_i . a), i < inter

struct OxbGemvParams {
    const uint32_t* codes;   // resident codes section
    const uint16_t* scales;  // resident scales section
    const float* x;          // [nvec][ldx] fp32 activations (device); unused when xq is set
    const uint32_t* xq;      // the same vectors as oxb_launch_gemv_pack left them (pro applied there), or nullptr
    uint32_t xq_bytes;       // extent of xq
    uint32_t nvg;            // groups of four vectors in xq: (nvec + 3) / 4
    const float* norm_w;     // [k], OXB_GEMV_PRO_RMSNORM only
    float eps;
    float* y;                // [nvec][ldy]
    const float* residual;   // [nvec][ldy], OXB_GEMV_RESIDUAL only
    uint32_t n_rows, n_tiles, n_sb, k;
    uint32_t sb_begin, sb_count;  // K range handled by this launch, in superblocks
    uint32_t nvec;                // 1 .. OXB_GEMV_MAX_BATCH (OXB_GEMV_PACKED_MAX_BATCH with xq)
    uint32_t ldx, ldy;
    uint32_t tpw;                 // filled by the launcher: tile slots per workgroup
    uint32_t codes_bytes, scales_bytes;  // buffer extents (loads beyond them read 0)
    int pro, epi;
};

// One launch covers at most OXB_GEMV_MAX_SB superblocks of K; the caller splits longer rows (first launch with the
// wanted epilogue, the following ones with OXB_GEMV_ACCUM).  OXB_GEMV_SWIGLU needs the whole K in one launch.
hipError_t oxb_launch_gemv(int fmt, OxbGemvParams p, uint32_t n_cus, hipStream_t st);
// Quantises nvec <= OXB_GEMV_PACKED_MAX_BATCH activation vectors of length k once for oxb_launch_gemv (pro as there:
// with OXB_GEMV_PRO_RMSNORM the norm weights are multiplied in and the sums of squares are left for the GEMV's
// epilogue); d_out needs oxb_gemv_pack_bytes(k, nvec) bytes.  The GEMV launch then takes xq = d_out, the same nvec
// and pro, and any sb_begin / sb_count range.
size_t oxb_gemv_pack_bytes(uint32_t k, uint32_t nvec);
hipError_t oxb_launch_gemv_pack(int fmt, int pro, const float* d_x, uint32_t ldx, uint32_t nvec, uint32_t k, const float* d_norm_w,
                                uint32_t* d_out, hipStream_t st);
// Measurement aid: reads the same codes and scales with the same grid, waves and load ring as oxb_launch_gemv would
// use, and does nothing else - the time below which no kernel that streams these bytes can finish.
hipError_t oxb_launch_gemv_stream_floor(int fmt, OxbGemvParams p, uint32_t n_cus, hipStream_t st);
hipError_t oxb_launch_dequant(const OxbLayout& L, const uint32_t* d_codes, const uint16_t* d_scales, float* d_out,
                              hipStream_t st);
// Block bytes in the reference's order (device copy, 2-byte aligned) -> the resident codes and scales sections, every
// padded entry included: the device twin of oxb_repack_aos_to_tiled.
hipError_t oxb_launch_repack(const OxbLayout& L, const uint8_t* d_aos, uint32_t* d_codes, uint16_t* d_scales, hipStream_t st);
// act[v][i] = silu(gu[v][i]) * gu[v][inter + i] for nvec vectors (rows of 2 * inter floats in, ldo floats out): the
// separate SwiGLU for rows too long for one GEMV launch.
hipError_t oxb_launch_swiglu(const float* d_gu, uint32_t inter, uint32_t nvec, float* d_out, uint32_t ldo, hipStream_t st);
