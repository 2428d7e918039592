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
    int fmt;                  /* 0 / 1 as above; 2 / 3: the same formats with every linear layer summed in double */
    size_t n_layers, h, inter, nq, nkv, hd, vocab, max_seq;
    float eps, rope_theta;
    const oxb_layer* layers;
    const float* final_norm;  /* [h] */
    oxb_linear lm_head;       /* vocab x h */
    int kv_f16;               /* 1: round K/V through f16 as the reference's GPU cache does */
} oxb_model;

typedef struct oxb_state oxb_state;   /* KV cache + scratch */
oxb_state* oxb_state_new(const oxb_model* m);
void       oxb_state_free(oxb_state* s);
/* One decode step: hidden[h] (embedding row) at position pos -> logits[vocab]. */
int oxb_forward(const oxb_model* m, oxb_state* s, const float* hidden_in, size_t pos, float* logits);
/* Same but also returns the hidden state after the final norm (may be NULL). */
int oxb_forward_ex(const oxb_model* m, oxb_state* s, const float* hidden_in, size_t pos,
                   float* logits, float* normed_out);

#ifdef __cplusplus
}
#endif
#endif
