/*
 * oxb_hip_measure.h — measurement and test hooks of liboxb_hip (same library, same conventions as oxb_hip.h).
 *
 * None of these stands in for an interface of the reference's kernel tier: a `NativeHipBackend` does not bind them.
 * They exist for the benchmark (per-kernel timings with HIP events on the stream the kernel runs on, as the reference
 * times its own kernels under CUDA_PROFILE / OXIBONSAI_PROFILE_GPU, KG/cuda_full_layer/mod.rs:339-344,
 * KG/metal_full_layer/functions.rs:17-35) and for one bit-exactness test of the sampler's in-order sum.
 */
#ifndef OXB_HIP_MEASURE_H
#define OXB_HIP_MEASURE_H

#include "oxb_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Launch the GEMV kernel (which quantises d_x in its prologue) `iters` times, launch i on weight ids[i % n_ids] (same
 * shape and format), bracketed by HIP events on the stream the kernel runs on.  *avg_us = mean time per launch in
 * microseconds.  batch = d_x holds that many vectors [batch][k], d_y [batch][n_rows].
 * _floor launches, in place of the GEMV, a kernel that only reads the same codes and scales with the same grid, waves and
 * load ring: the time below which no kernel that streams these bytes can finish on this GPU. */
int  oxb_hip_profile_gemv(const uint64_t* ids, uint32_t n_ids, const float* d_x, float* d_y,
                          uint32_t n_rows, uint32_t k, uint32_t warmup, uint32_t iters, float* avg_us);
int  oxb_hip_profile_gemv_floor(const uint64_t* ids, uint32_t n_ids, uint32_t n_rows, uint32_t k, uint32_t warmup,
                                uint32_t iters, float* avg_us);
/* Route selection of oxb_hip_gemv / oxb_hip_gemv_dev, for A/B measurements and tests.  On one route the activations
 * are quantised by a launch of their own and up to eight vectors share one pass over the weights; on the other every
 * workgroup quantises them in its prologue (four vectors per pass).  n = 1 (the default): by shape - the first route
 * from five vectors on, and from two where K exceeds 4096; n = 0: never the first route; n >= 2: the first route from
 * n vectors on. */
int  oxb_hip_set_gemv_packed_min_batch(uint32_t n);
/* Packs x once, then times `iters` prefill GEMM launches with events on the library's stream. */
int  oxb_hip_profile_gemm(uint64_t id, const float* d_x, float* d_y, uint32_t m, uint32_t n_rows, uint32_t k,
                          uint32_t warmup, uint32_t iters, float* avg_us);
/* The f32 sum of x[0..n) taken element by element from 0, as the loop `sum += *v` of the reference's softmax does
 * (sampling.rs:126-130); all x >= 0.  The filter-off sampler depends on this order bit for bit; exposed so that it can
 * be checked on its own. */
int  oxb_hip_sum_in_order(const float* x, uint32_t n, float* sum_out);

#ifdef __cplusplus
}
#endif
#endif /* OXB_HIP_MEASURE_H */
