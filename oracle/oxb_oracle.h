/*
 * oxb_oracle.h — CPU restatement of the reference's scalar sub-2-bit path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the shipped library links, loads or
 * calls this code: it exists so the tests, the smoke check and the bench's
 * cpu_baseline leg can check the HIP path against the reference's arithmetic.
 *
 * Every function names the reference source it follows (paths are relative
 * to the reference checkout).  The scalar kernels keep the reference's exact
 * summation order: per block a 128-term fp32 sum in index order, then
 * `sum += d * block_sum`; the file is built with -ffp-contract=off so no
 * multiply-add is fused, as in the Rust original.
 *
 * Pinning status (what fixes each function without running the reference):
 *   f16<->f32          IEEE-754, all 65 536 patterns vs numpy.float16
 *   dequant_*          closed forms of the reference's unit tests + brute force
 *   gemv_* / gemm_*    reference KATs (+-128 d, 0, sum 0..127, 0x46 canary),
 *                      float64 numpy product of the dequantized matrix,
 *                      linearity / gemm(m=1)=gemv invariants
 *   rms_norm, swiglu, rope, softmax, attention
 *                      reference closed-form KATs + float64 numpy
 *   model forward      float64 numpy restatement on the tiny test geometry
 *                      (no stored logits exist in the reference: end-to-end
 *                      token strings of the real binary are parity unpinned)
 *   sample             the reference's sampler unit tests (greedy, valid index,
 *                      top-k range), the xorshift64 recurrence and the draw formula
 *                      recomputed with Python integers, candidates / probabilities
 *                      against a float64 numpy softmax, draw frequencies.  Parity
 *                      unpinned: the candidate order the reference's partial
 *                      selection leaves when top_p == 1 (implementation-defined)
 *                      and the last place of exp()
 *   fp8 codes, kv rows the reference's encode / decode unit tests (0, -0, NaN, infinities, 448, 2^-9, 1000, ...),
 *                      every byte's value and every representable value's code against torch's float8 types,
 *                      round-to-nearest-even against a float64 search over the code table; INT8 rows against the
 *                      reference's [127, -127, 0] test and a float64 numpy restatement
 *   in_window          the reference's attention_range / is_in_window unit tests (positions listed there)
 */
#ifndef OXB_ORACLE_H
#define OXB_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Error codes mirroring KernelError (crates/oxibonsai-kernels/src/error.rs). */
enum {
    OXB_OK = 0,
    OXB_ERR_NOT_BLOCK_ALIGNED = 1,
    OXB_ERR_DIMENSION_MISMATCH = 2,
    OXB_ERR_BUFFER_TOO_SMALL = 3,
};

#define OXB_QK 128          /* weights per block, both formats              */
#define OXB_Q1_BYTES 18     /* [d: f16 LE][qs: 16 B]                        */
#define OXB_TQ2_BYTES 34    /* [qs: 32 B][d: f16 LE]                        */

void     oxb_oracle_set_threads(int n);  /* row-loop threads of the scalar kernels; 0 = all cores */
float    oxb_f16_to_f32(uint16_t h);
uint16_t oxb_f32_to_f16(float f);  /* round-to-nearest-even, as half::f16::from_f32 */

int oxb_dequant_q1(const uint8_t* blocks, size_t n_blocks, float* out, size_t out_len);
int oxb_dequant_tq2(const uint8_t* blocks, size_t n_blocks, float* out, size_t out_len);

/* Lengths are element counts of the caller's buffers, checked as the reference checks them. */
int oxb_gemv_q1(const uint8_t* blocks, size_t n_blocks, const float* x, size_t x_len,
                float* y, size_t y_len, size_t n_rows, size_t k);
int oxb_gemv_tq2(const uint8_t* blocks, size_t n_blocks, const float* x, size_t x_len,
                 float* y, size_t y_len, size_t n_rows, size_t k);
int oxb_gemm_q1(const uint8_t* blocks, size_t n_blocks, const float* x, size_t x_len,
                float* y, size_t y_len, size_t m, size_t n_rows, size_t k);
int oxb_gemm_tq2(const uint8_t* blocks, size_t n_blocks, const float* x, size_t x_len,
                 float* y, size_t y_len, size_t m, size_t n_rows, size_t k);

void  oxb_rms_norm(const float* in, const float* w, float* out, size_t n, float eps);
float oxb_silu(float x);
void  oxb_swiglu(const float* gate, const float* up, float* out, size_t n);
void  oxb_softmax(float* v, size_t n);
void  oxb_rope_table(float* cos_t, float* sin_t, size_t head_dim, size_t max_seq, float freq_base);
void  oxb_rope_apply(const float* in, float* out, const float* cos_row, const float* sin_row, size_t half_dim);
void  oxb_attention_head(const float* q, const float* keys, const float* values, float* out,
                         size_t seq_len, size_t head_dim);
/* Sliding window with attention sinks (model/src/layers/sliding_window.rs); window == 0 in the attention call: off. */
int   oxb_in_window(size_t key, size_t query, size_t window, size_t sinks);
void  oxb_attention_head_windowed(const float* q, const float* keys, const float* values, float* out,
                                  size_t seq_len, size_t head_dim, size_t window, size_t sinks);

/* How a KV cache keeps its rows. */
enum { OXB_KV_F32 = 0, OXB_KV_F16 = 1, OXB_KV_I8 = 2, OXB_KV_FP8_E4M3 = 3, OXB_KV_FP8_E5M2 = 4 };
uint8_t oxb_fp8_e4m3_encode(float x);
uint8_t oxb_fp8_e5m2_encode(float x);
float   oxb_fp8_e4m3_decode(uint8_t b);
float   oxb_fp8_e5m2_decode(uint8_t b);
/* One row of head_dim values -> codes (i8 as its byte, or FP8) and the row scale; and back (code * scale). */
int oxb_kv_quantize_row(int mode, const float* row, size_t n, uint8_t* codes, float* scale_out);
int oxb_kv_dequantize_row(int mode, const uint8_t* codes, size_t n, float scale, float* out);
uint32_t oxb_argmax_last(const float* v, size_t n);   /* Sampler greedy: last max on ties */
uint32_t oxb_argmax_first(const float* v, size_t n);  /* GPU argmax_f32: first max        */
/* Sampler::sample (runtime/src/sampling.rs:84-177); see the definition for the candidate order it fixes. */
uint32_t oxb_sample(const float* logits, size_t n, float temperature, size_t top_k, float top_p, uint64_t* rng_state,
                    uint32_t* cand_idx, float* cand_p, size_t cap, size_t* n_cand, float* r_out);

/* One linear layer in the reference's AoS block format. fmt: 0 = Q1_0_g128, 1 = TQ2_0_g128. */
typedef struct {
    const uint8_t* blocks;
    size_t n_rows, k;
} oxb_linear;

typedef struct {
    const float* attn_norm;   /* [h]  */
    const float* q_norm;      /* [hd] */
    const float* k_norm;      /* [hd] */
    const float* ffn_norm;    /* [h]  */
    oxb_linear q, k, v, o, gate, up, down;
} oxb_layer;

typedef struct {
    int fmt;                  /* 0 / 1 as above; 2 / 3: the same formats with every linear layer summed in double;
                                 4 / 5: the same formats with the linear layers on the CPU SIMD tier (oxb_simd.cpp) */
    size_t n_layers, h, inter, nq, nkv, hd, vocab, max_seq;
    float eps, rope_theta;
    const oxb_layer* layers;
    const float* final_norm;  /* [h] */
    oxb_linear lm_head;       /* vocab x h */
    int kv_mode;              /* OXB_KV_*: F16 rounds K/V through f16 as the reference's GPU cache does; I8 / FP8 store
                                 codes + a scale per (position, kv head) as model/src/kv_cache_quant.rs does */
    size_t window, sinks;     /* sliding-window attention; window == 0: every earlier position is visible */
} oxb_model;

typedef struct oxb_state oxb_state;   /* KV cache + scratch */
oxb_state* oxb_state_new(const oxb_model* m);
void       oxb_state_free(oxb_state* s);
/* which: 0 / 1 K / V as attention reads them (f32 [L][nkv][max_seq][hd]); 2 / 3 their codes (u8, same shape) and
 * 4 / 5 their scales (f32 [L][nkv][max_seq]) when the cache is quantised, else NULL. */
const void* oxb_state_cache(const oxb_state* s, int which);
/* Test aid: give the cache rows of one (layer, kv head) as attention shall read them; while frozen, a forward stores
 * nothing (its attention then runs over exactly the given rows). */
void oxb_state_load_rows(const oxb_model* m, oxb_state* s, size_t layer, size_t kv_head, size_t pos0, size_t n,
                         const float* k_rows, const float* v_rows);
void oxb_state_freeze(oxb_state* s, int frozen);
/* One decode step: hidden[h] (embedding row) at position pos -> logits[vocab]. */
int oxb_forward(const oxb_model* m, oxb_state* s, const float* hidden_in, size_t pos, float* logits);
/* Same but also returns the hidden state after the final norm (may be NULL). */
int oxb_forward_ex(const oxb_model* m, oxb_state* s, const float* hidden_in, size_t pos,
                   float* logits, float* normed_out);

/* A run of n consecutive positions pos_start .. pos_start + n - 1 of one sequence, layer by layer (every operation
 * is per token, so the values are those of n calls of oxb_forward_ex in a row; the linear layers go through the
 * batched products).  hidden_in [n][h]; logits / normed_out (either may be NULL) receive the last position's. */
int oxb_forward_batch(const oxb_model* m, oxb_state* s, const float* hidden_in, size_t pos_start, size_t n,
                      float* logits, float* normed_out);

/* CPU SIMD tier (oxb_simd.cpp): the model forward uses it for its linear layers when oxb_model.fmt is 4 / 5. */
int oxb_simd_gemv(int fmt, const uint8_t* blocks, size_t n_blocks, const float* x, size_t x_len,
                  float* y, size_t y_len, size_t n_rows, size_t k);
int oxb_simd_gemm_x4(int fmt, const uint8_t* blocks, size_t n_blocks, const float* x, size_t x_len,
                     float* y, size_t y_len, size_t m, size_t n_rows, size_t k);

#ifdef __cplusplus
}
#endif
#endif
