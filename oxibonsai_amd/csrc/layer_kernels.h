// layer_kernels.h — launch interface of the layer glue kernels (see layer_kernels.hip).
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

#include "kv_quant_device.h"

struct OxbQkParams {
    const float* qkv;      // [batch][qkv_stride]: q heads | k heads | v heads
    uint32_t qkv_stride;
    const float *q_norm, *k_norm;  // [hd]
    const float *cos_t, *sin_t;    // [max_seq][hd/2]
    const uint32_t* pos;           // [batch], device; null: row b is token pos_base + b of sequence `seq` (prefill)
    uint32_t pos_base, seq;
    float* q_rope;                 // [batch][nq][hd]
    void *k_cache, *v_cache;       // cache rows of hd values each (fp16, or one-byte codes: kv_mode), placed by `kv`
    float *k_scale, *v_scale;      // quantised cache: one scale per row
    uint32_t kv_mode;
    OxbKvLayout kv;
    uint32_t nq, nkv, hd, max_seq, n_layers, layer;
    float eps;
};

struct OxbAttnParams {
    // the attention kernel reads the raw projections and does QK-norm, RoPE and the KV store itself
    const float* qkv;                    // [batch][qkv_stride]: q heads | k heads | v heads
    uint32_t qkv_stride;
    const float *q_norm, *k_norm;        // [hd]
    const float *cos_t, *sin_t;          // [max_seq][hd/2]
    float eps;
    void *k_cache, *v_cache;             // cache rows of hd values each (fp16, or one-byte codes: kv_mode), placed by `kv`
    float *k_scale, *v_scale;            // quantised cache: one scale per row
    uint32_t kv_mode;                    // OXB_KV_* (kv_quant_device.h)
    OxbKvLayout kv;                      // contiguous (row_stride a multiple of the chunk, >= max_seq) or paged (pages of 16..128 positions)
    uint32_t window, sinks;              // sliding window with attention sinks; window 0 = off
    float* part;                         // [batch][nq][n_splits][hd + OXB_ATTN_PART_PAD]: un-normalised output, maximum, sum
    float* out_single;                   // optional, n_splits == 1 only: [batch][nq*hd] receives the finished output (no merge launch)
    float* out_merged;                   // n_splits > 1: [batch][nq*hd], written by the last workgroup of each (sequence, kv head) to finish
    uint32_t* done;                      // n_splits > 1: [batch][nkv] arrival counters, zero before the launch; the kernel leaves them zero
    const uint32_t* pos;                 // [batch], device; seq_len = pos + 1
    uint32_t nq, nkv, hd, max_seq, n_layers, layer, chunk, n_splits;
    float scale;                         // 1 / sqrt(hd)
    // Optional: the workgroup that merges the slots of (sequence b, kv head) also leaves its 512 outputs quantised for
    // the O projection's packed GEMV (gemv_pack_device.h) as superblock `kv head` of vector b - instead of a pack launch
    // between the two kernels.  Only where a kv head's q heads are exactly one superblock (nq / nkv * hd == 512) and the
    // slots are merged in the kernel (n_splits > 1); pack_fmt = the O weight's format.
    uint32_t* pack_out;                  // nullptr = off
    uint32_t pack_fmt, pack_n_sb, pack_nvg;
};

// n_rows rows of n values -> one-byte codes [n_rows][n] and a scale per row (kv_mode: OXB_KV_I8 or OXB_KV_FP8_E4M3).
hipError_t oxb_launch_kv_dequantize_rows(int kv_mode, const uint8_t* d_codes, const float* d_scales, uint32_t n_rows, uint32_t n,
                                         float* d_out, hipStream_t st);
hipError_t oxb_launch_kv_quantize_rows(int kv_mode, const float* d_x, uint32_t n_rows, uint32_t n, uint8_t* d_codes, float* d_scales,
                                       hipStream_t st);
hipError_t oxb_launch_qk_norm_rope_store(const OxbQkParams& p, uint32_t batch, hipStream_t st);
#define OXB_ATTN_CHUNK_POSITIONS 128  // KV positions one attention workgroup covers at a time
#define OXB_ATTN_MAX_SPLITS 64        // slots the KV sequence is split over; slot s walks chunks s, s + n_splits, ...
#define OXB_ATTN_PART_PAD 4           // floats after the hd outputs of a slot: maximum, sum, 2 unused (16-byte rows)
// QK-norm, RoPE, KV store of the new position, split-KV attention (at most 16 q heads per kv head) into p.part and
// the merge of the slots into the fp32 attention output p.out_merged [batch][nq * hd], all in one launch.
hipError_t oxb_launch_attn_decode(const OxbAttnParams& p, uint32_t batch, hipStream_t st);
// out[v] = w * x[v] / sqrt(mean(x[v]^2) + eps) for nvec vectors of n values; d_w == nullptr copies.
hipError_t oxb_launch_rmsnorm(const float* d_x, const float* d_w, uint32_t n, uint32_t nvec, float eps, float* d_out, hipStream_t st);
// d_ws: batch * OXB_ARGMAX_MAX_PARTS * 8 bytes of scratch for the per-span maxima.
#define OXB_ARGMAX_MAX_PARTS 256u
// host_copy_or_null: pinned host memory that receives the token ids too (readable after the stream is synchronised)
hipError_t oxb_launch_argmax(const float* d_logits, uint32_t n, uint32_t batch, uint32_t* d_out, void* d_ws, hipStream_t st,
                             uint32_t* host_copy_or_null = nullptr);
// hidden rows (n_floats, a multiple of 4) and positions from pinned host memory to their device buffers, one launch
hipError_t oxb_launch_stage_in(const float* h_hidden, uint32_t n_floats, const uint32_t* h_pos, uint32_t n_pos, float* d_hidden,
                               uint32_t* d_pos, hipStream_t st);
