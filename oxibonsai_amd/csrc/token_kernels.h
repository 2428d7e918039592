// token_kernels.h — the device steps either side of the forward: token embedding lookup, sampling, token bookkeeping.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

// Token embedding lookup: out[i][0..h) = row ids[i] of the table kept in its stored form (gguf_type 0 F32, 1 F16,
// 41 Q1_0_g128 blocks, 42 TQ2_0_g128 blocks), widened / dequantised as the reference's loader does.  ids are device
// memory; an id >= vocab yields a row of NaN (host-supplied ids are validated before the launch).
hipError_t oxb_launch_embedding_gather(const void* d_table, int gguf_type, uint32_t vocab, uint32_t h, const uint32_t* d_ids,
                                       uint32_t n, float* d_out, hipStream_t st);
// End of one step of the on-device greedy loop: history[b] = tokens[b]; pos[b] += 1.
hipError_t oxb_launch_token_step(const uint32_t* d_tokens, uint32_t* d_history, uint32_t* d_pos, uint32_t batch, hipStream_t st);

// Sampler::sample on the device (crates/oxibonsai-runtime/src/sampling.rs:84-177) for `batch` rows of logits:
// the top_k largest logits in descending order (ties: lower index first; up to OXB_SAMPLE_MAX_TOP_K by selection
// kernels, beyond that by a stable sort of the whole row), v / temperature, softmax, top-p cut and renormalisation,
// one xorshift64 draw per row from d_rng[row] (updated in place), cumulative pick -> d_tokens[row].  top_k = 0 or
// >= n: the filter is off and the row is taken in index order, as the reference does (sampling.rs:111).
// d_ws: oxb_sample_ws_bytes(n, batch) bytes of scratch.
#define OXB_SAMPLE_MAX_TOP_K 128
size_t oxb_sample_ws_bytes(uint32_t n, uint32_t batch);
hipError_t oxb_launch_sample(const float* d_logits, uint32_t n, uint32_t batch, float temperature, uint32_t top_k, float top_p,
                             uint64_t* d_rng, uint32_t* d_tokens, void* d_ws, hipStream_t st);
// d_sum[0] = ((0 + x[0]) + x[1]) + ... in f32, element by element: the softmax denominator as the reference's loop
// forms it (sampling.rs:126-130).  All x >= 0.
hipError_t oxb_launch_sum_in_order(const float* d_x, uint32_t n, float* d_sum, hipStream_t st);
