// prefill_kernels.h — launch interface of the prefill attention (see prefill_kernels.hip).
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

#include "kv_quant_device.h"

struct OxbPrefillAttnParams {
    const float* qkv;                 // [M][qkv_stride]: the raw projections, q heads first (QK-norm and RoPE happen in the kernel)
    uint32_t qkv_stride;
    const float* q_norm;              // [hd]
    const float *cos_t, *sin_t;       // [max_seq][hd/2]
    float eps;
    const void *k_cache, *v_cache;    // cache rows of hd values each (fp16 or one-byte codes), placed by `kv`
    const float *k_scale, *v_scale;   // quantised cache: one scale per row
    uint32_t kv_mode;                 // OXB_KV_* (kv_quant_device.h)
    OxbKvLayout kv;
    uint32_t seq, layer;              // whose rows the queries attend to
    uint32_t window, sinks;           // sliding window with attention sinks; window 0 = off
    float* out;                       // [M][nq * hd]
    uint32_t M, pos_start;            // query t sits at position pos_start + t and sees keys 0 .. pos_start + t
    uint32_t nq, nkv, hd, max_seq;
    float scale;                      // 1 / sqrt(hd)
};

hipError_t oxb_launch_attn_prefill(const OxbPrefillAttnParams& p, hipStream_t st);
