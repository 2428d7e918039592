/*
 * oxb_oracle.c — scalar CPU restatement of the reference's sub-2-bit path.
 * TEST INFRASTRUCTURE ONLY (see oxb_oracle.h).  Build: -O2 -ffp-contract=off.
 */
#include "oxb_oracle.h"

#include <float.h>
#include <math.h>
#include <stdlib.h>
#ifdef _OPENMP
#include <omp.h>
#endif
#include <string.h>

/* ------------------------------------------------------------------------- */
/* binary16 <-> binary32.  The reference uses half::f16::{to_f32,from_f32}     */
/* (half 2.7.1; call sites kernels/src/gemv.rs:65, gemv_ternary.rs:87,        */
/* core/src/tensor.rs:70): IEEE-754 widening is exact, narrowing is RNE.      */
/* ------------------------------------------------------------------------- */
float oxb_f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else { /* subnormal: normalise */
            int e = -1;
            do { man <<= 1; e++; } while (!(man & 0x400u));
            man &= 0x3FFu;
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7F800000u | (man << 13);
    } else {
        bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

uint16_t oxb_f32_to_f16(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    uint32_t abs = x & 0x7FFFFFFFu;
    if (abs >= 0x7F800000u) { /* inf / nan */
        return (uint16_t)(sign | 0x7C00u | (abs > 0x7F800000u ? (0x200u | ((abs >> 13) & 0x3FFu)) : 0));
    }
    if (abs >= 0x477FF000u) { /* rounds to >= 65520 -> inf */
        return (uint16_t)(sign | 0x7C00u);
    }
    if (abs < 0x33000001u) { /* < 2^-25 (or == 2^-25 tie -> even 0) */
        return sign;
    }
    int32_t e = (int32_t)(abs >> 23) - 127;
    uint32_t man = (abs & 0x7FFFFFu) | 0x800000u;
    uint32_t shift, half_man;
    if (e < -14) { /* subnormal result */
        shift = (uint32_t)(13 + (-14 - e));
        half_man = man >> shift;
        uint32_t rem = man & ((1u << shift) - 1u);
        uint32_t halfway = 1u << (shift - 1);
        if (rem > halfway || (rem == halfway && (half_man & 1u))) half_man++;
        return (uint16_t)(sign | half_man);
    }
    shift = 13;
    half_man = man >> shift; /* includes the implicit bit at 0x400 */
    uint32_t rem = man & 0x1FFFu;
    uint32_t out = ((uint32_t)(e + 15) << 10) + (half_man - 0x400u);
    if (rem > 0x1000u || (rem == 0x1000u && (out & 1u))) out++;
    return (uint16_t)(sign | out);
}

static inline float q1_scale(const uint8_t* b) { /* [d LE][qs16]: core/src/tensor.rs:25-32 */
    return oxb_f16_to_f32((uint16_t)(b[0] | (b[1] << 8)));
}
static inline float tq2_scale(const uint8_t* b) { /* [qs32][d LE]: core/src/quant_ternary.rs:64-71 */
    return oxb_f16_to_f32((uint16_t)(b[32] | (b[33] << 8)));
}
/* core/src/quant_ternary.rs:191-200, kernels/src/gemv_ternary.rs:19-27 */
static inline float tq2_code(uint8_t byte, unsigned lane) {
    switch ((byte >> (lane * 2)) & 3u) {
        case 0: return -1.0f;
        case 1: return 0.0f;
        case 2: return 1.0f;
        default: return 0.0f;
    }
}

/* kernels/src/dequant.rs:15-37 */
int oxb_dequant_q1(const uint8_t* blocks, size_t n_blocks, float* out, size_t out_len) {
    if (out_len < n_blocks * OXB_QK) return OXB_ERR_BUFFER_TOO_SMALL;
    for (size_t i = 0; i < n_blocks; i++) {
        const uint8_t* b = blocks + i * OXB_Q1_BYTES;
        float d = q1_scale(b);
        for (size_t j = 0; j < OXB_QK; j++) {
            unsigned bit = (b[2 + j / 8] >> (j % 8)) & 1u;
            out[i * OXB_QK + j] = bit ? d : -d;
        }
    }
    return OXB_OK;
}

/* kernels/src/dequant_ternary.rs:42-64 */
int oxb_dequant_tq2(const uint8_t* blocks, size_t n_blocks, float* out, size_t out_len) {
    if (out_len < n_blocks * OXB_QK) return OXB_ERR_BUFFER_TOO_SMALL;
    for (size_t i = 0; i < n_blocks; i++) {
        const uint8_t* b = blocks + i * OXB_TQ2_BYTES;
        float d = tq2_scale(b);
        for (size_t byte = 0; byte < 32; byte++)
            for (unsigned lane = 0; lane < 4; lane++)
                out[i * OXB_QK + byte * 4 + lane] = d * tq2_code(b[byte], lane);
    }
    return OXB_OK;
}

/* kernels/src/gemv.rs:60-84 — inner loop of one row. */
static float q1_row_dot(const uint8_t* row_blocks, size_t blocks_per_row, const float* x) {
    float sum = 0.0f;
    for (size_t bi = 0; bi < blocks_per_row; bi++) {
        const uint8_t* b = row_blocks + bi * OXB_Q1_BYTES;
        float d = q1_scale(b);
        const float* xb = x + bi * OXB_QK;
        float block_sum = 0.0f;
        for (size_t j = 0; j < OXB_QK; j++) {
            float sign = ((b[2 + j / 8] >> (j % 8)) & 1u) ? 1.0f : -1.0f;
            block_sum += sign * xb[j];
        }
        sum += d * block_sum;
    }
    return sum;
}

/* kernels/src/gemv_ternary.rs:83-102 — inner loop of one row. */
static float tq2_row_dot(const uint8_t* row_blocks, size_t blocks_per_row, const float* x) {
    float sum = 0.0f;
    for (size_t bi = 0; bi < blocks_per_row; bi++) {
        const uint8_t* b = row_blocks + bi * OXB_TQ2_BYTES;
        float d = tq2_scale(b);
        const float* xb = x + bi * OXB_QK;
        float block_sum = 0.0f;
        for (size_t byte = 0; byte < 32; byte++)
            for (unsigned lane = 0; lane < 4; lane++)
                block_sum += tq2_code(b[byte], lane) * xb[byte * 4 + lane];
        sum += d * block_sum;
    }
    return sum;
}

/* Threads the row loops of the scalar kernels may use (rows are independent, so the results do not depend on it);
 * 1 gives the single-thread time of the reference's scalar tier. */
void oxb_oracle_set_threads(int n) {
#ifdef _OPENMP
    omp_set_num_threads(n > 0 ? n : omp_get_num_procs());
#else
    (void)n;
#endif
}

/* kernels/src/gemv.rs:25-87 (validation order :32-58) */
int oxb_gemv_q1(const uint8_t* blocks, size_t n_blocks, const float* x, size_t x_len,
                float* y, size_t y_len, size_t n_rows, size_t k) {
    if (k % OXB_QK != 0) return OXB_ERR_NOT_BLOCK_ALIGNED;
    if (x_len < k) return OXB_ERR_DIMENSION_MISMATCH;
    if (y_len < n_rows) return OXB_ERR_BUFFER_TOO_SMALL;
    size_t bpr = k / OXB_QK;
    if (n_blocks < n_rows * bpr) return OXB_ERR_BUFFER_TOO_SMALL;
#pragma omp parallel for schedule(static) if (n_rows * bpr > 4096)  /* rows are independent: same bits, less waiting */
    for (size_t r = 0; r < n_rows; r++)
        y[r] = q1_row_dot(blocks + r * bpr * OXB_Q1_BYTES, bpr, x);
    return OXB_OK;
}

/* kernels/src/gemv_ternary.rs:48-105 (short block slice is DimensionMismatch, :76-81) */
int oxb_gemv_tq2(const uint8_t* blocks, size_t n_blocks, const float* x, size_t x_len,
                 float* y, size_t y_len, size_t n_rows, size_t k) {
    if (k % OXB_QK != 0) return OXB_ERR_NOT_BLOCK_ALIGNED;
    if (x_len < k) return OXB_ERR_DIMENSION_MISMATCH;
    if (y_len < n_rows) return OXB_ERR_BUFFER_TOO_SMALL;
    size_t bpr = k / OXB_QK;
    if (n_blocks < n_rows * bpr) return OXB_ERR_DIMENSION_MISMATCH;
#pragma omp parallel for schedule(static) if (n_rows * bpr > 4096)
    for (size_t r = 0; r < n_rows; r++)
        y[r] = tq2_row_dot(blocks + r * bpr * OXB_TQ2_BYTES, bpr, x);
    return OXB_OK;
}

/* kernels/src/gemm.rs:19-87: Y[mi][ni] = dot(W[ni,:], X[mi,:]) */
int oxb_gemm_q1(const uint8_t* blocks, size_t n_blocks, const float* x, size_t x_len,
                float* y, size_t y_len, size_t m, size_t n_rows, size_t k) {
    if (k % OXB_QK != 0) return OXB_ERR_NOT_BLOCK_ALIGNED;
    if (x_len < m * k) return OXB_ERR_DIMENSION_MISMATCH;
    if (y_len < m * n_rows) return OXB_ERR_BUFFER_TOO_SMALL;
    size_t bpr = k / OXB_QK;
    if (n_blocks < n_rows * bpr) return OXB_ERR_BUFFER_TOO_SMALL;
    for (size_t mi = 0; mi < m; mi++)
        for (size_t ni = 0; ni < n_rows; ni++)
            y[mi * n_rows + ni] = q1_row_dot(blocks + ni * bpr * OXB_Q1_BYTES, bpr, x + mi * k);
    return OXB_OK;
}

/* kernels/src/gemm_ternary.rs:35-69: a GEMV per batch row. */
int oxb_gemm_tq2(const uint8_t* blocks, size_t n_blocks, const float* x, size_t x_len,
                 float* y, size_t y_len, size_t m, size_t n_rows, size_t k) {
    if (k % OXB_QK != 0) return OXB_ERR_NOT_BLOCK_ALIGNED;
    if (x_len < m * k) return OXB_ERR_DIMENSION_MISMATCH;
    if (y_len < m * n_rows) return OXB_ERR_BUFFER_TOO_SMALL;
    for (size_t mi = 0; mi < m; mi++) {
        int rc = oxb_gemv_tq2(blocks, n_blocks, x + mi * k, k, y + mi * n_rows, n_rows, n_rows, k);
        if (rc) return rc;
    }
    return OXB_OK;
}

/* kernels/src/simd_float_ops.rs:204-215 */
void oxb_rms_norm(const float* in, const float* w, float* out, size_t n, float eps) {
    float sum_sq = 0.0f;
    for (size_t i = 0; i < n; i++) sum_sq += in[i] * in[i];
    float rms = sqrtf(sum_sq / (float)n + eps);
    float inv_rms = 1.0f / rms;
    for (size_t i = 0; i < n; i++) out[i] = w[i] * in[i] * inv_rms;
}

/* kernels/src/simd_float_ops.rs:217-220; model/src/layers/swiglu.rs:9-12 */
float oxb_silu(float x) { return x / (1.0f + expf(-x)); }

/* kernels/src/simd_float_ops.rs:232-236 */
void oxb_swiglu(const float* gate, const float* up, float* out, size_t n) {
    for (size_t i = 0; i < n; i++) out[i] = oxb_silu(gate[i]) * up[i];
}

/* kernels/src/simd_float_ops.rs:187-201 */
void oxb_softmax(float* v, size_t n) {
    float mx = -INFINITY;
    for (size_t i = 0; i < n; i++) mx = fmaxf(mx, v[i]);
    float sum = 0.0f;
    for (size_t i = 0; i < n; i++) { v[i] = expf(v[i] - mx); sum += v[i]; }
    if (sum > 0.0f) {
        float inv = 1.0f / sum;
        for (size_t i = 0; i < n; i++) v[i] *= inv;
    }
}

/* model/src/layers/rope.rs:27-48: all arithmetic in f32 (powf, cos, sin). */
void oxb_rope_table(float* cos_t, float* sin_t, size_t head_dim, size_t max_seq, float freq_base) {
    size_t half = head_dim / 2;
    for (size_t pos = 0; pos < max_seq; pos++)
        for (size_t i = 0; i < half; i++) {
            float freq = 1.0f / powf(freq_base, 2.0f * (float)i / (float)head_dim);
            float angle = (float)pos * freq;
            cos_t[pos * half + i] = cosf(angle);
            sin_t[pos * half + i] = sinf(angle);
        }
}

/* kernels/src/simd_float_ops.rs:240-253: half-split pairs (i, i + half). */
void oxb_rope_apply(const float* in, float* out, const float* c, const float* s, size_t half) {
    for (size_t i = 0; i < half; i++) {
        float x0 = in[i], x1 = in[half + i];
        out[i] = x0 * c[i] - x1 * s[i];
        out[half + i] = x0 * s[i] + x1 * c[i];
    }
}

/* model/src/layers/sliding_window.rs:173-189 (is_in_window; attention_range :53-98 lists the same positions):
 * the first `sinks` keys are always visible, the others while query - key < window - sinks. */
int oxb_in_window(size_t key, size_t query, size_t window, size_t sinks) {
    if (window == 0) return 0;
    if (key < sinks) return 1;
    if (query < key) return 0;
    const size_t budget = window > sinks ? window - sinks : 0;
    return query - key < budget;
}

/* model/src/layers/attention_fused.rs:166-226 (online softmax state) and :329-400
 * (contiguous K/V walk).  The reference's dot product is AVX dual-accumulator on
 * x86 (:139-164); the plain index-order sum is used here, the difference being a
 * summation order the tolerances cover.  window > 0 restricts the keys of the query at
 * position seq_len - 1 to those oxb_in_window admits (masked keys get weight 0, which
 * is what apply_sliding_window_mask's -inf scores amount to, sliding_window.rs:109-135). */
void oxb_attention_head_windowed(const float* q, const float* keys, const float* values, float* out,
                                 size_t seq_len, size_t hd, size_t window, size_t sinks) {
    for (size_t d = 0; d < hd; d++) out[d] = 0.0f;
    if (seq_len == 0) return;
    float scale = 1.0f / sqrtf((float)hd);
    float max_val = -INFINITY, sum_exp = 0.0f;
    for (size_t t = 0; t < seq_len; t++) {
        if (window && !oxb_in_window(t, seq_len - 1, window, sinks)) continue;
        const float* kt = keys + t * hd;
        float dot = 0.0f;
        for (size_t d = 0; d < hd; d++) dot += q[d] * kt[d];
        float score = dot * scale;
        if (score > max_val) {
            float rescale = (max_val == -INFINITY) ? 0.0f : expf(max_val - score);
            sum_exp *= rescale;
            for (size_t d = 0; d < hd; d++) out[d] *= rescale;
            max_val = score;
        }
        float e = expf(score - max_val);
        sum_exp += e;
        const float* vt = values + t * hd;
        for (size_t d = 0; d < hd; d++) out[d] += e * vt[d];
    }
    if (sum_exp > 0.0f) {
        float inv = 1.0f / sum_exp;
        for (size_t d = 0; d < hd; d++) out[d] *= inv;
    }
}

void oxb_attention_head(const float* q, const float* keys, const float* values, float* out,
                        size_t seq_len, size_t hd) {
    oxb_attention_head_windowed(q, keys, values, out, seq_len, hd, 0, 0);
}

/* ------------------------------------------------------------------------- */
/* Quantised KV rows.                                                         */
/* FP8 codes: core/src/quant_fp8.rs:47-160 (E4M3FN: s eeee mmm, bias 7, no infinity, NaN = 0x7f, |x| >= 448
 * saturates to 0x7e) and :208-301 (E5M2: s eeeee mm, bias 15, |x| > 57344 becomes infinity 0x7c, NaN = 0x7e);
 * both round to nearest, ties to even, including into and inside the subnormal range.  One routine covers both:
 * man_bits / bias / the code of the largest finite value / what lies beyond it. */
static uint8_t fp8_encode(float x, int man_bits, int bias, float max_finite, int at_max_saturates,
                          uint8_t code_max, uint8_t code_over, uint8_t code_nan) {
    uint32_t bits;
    memcpy(&bits, &x, 4);
    const uint8_t sign = (uint8_t)((bits >> 31) << 7);
    const uint32_t mag = bits & 0x7FFFFFFFu;
    if (mag > 0x7F800000u) return code_nan;             /* NaN: canonical, positive */
    if (mag == 0x7F800000u) return sign | code_over;
    if (mag == 0) return sign;
    float a;
    memcpy(&a, &mag, 4);
    if (at_max_saturates ? a >= max_finite : a > max_finite) return sign | (at_max_saturates ? code_max : code_over);
    const int e = (int)(mag >> 23) - 127 + bias;        /* biased exponent in the target format */
    uint32_t code;
    if (e >= 1) {
        const int shift = 23 - man_bits;
        const uint32_t man = mag & 0x7FFFFFu, rem = man & ((1u << shift) - 1u), halfway = 1u << (shift - 1);
        code = ((uint32_t)e << man_bits) | (man >> shift);
        if (rem > halfway || (rem == halfway && (code & 1u))) code++;   /* a carry runs into the exponent field */
        if (code > code_max) code = at_max_saturates ? code_max : code_over;
    } else {
        /* subnormal target: multiples of 2^(1 - bias - man_bits); the product is exact, rintf rounds to even,
         * and 2^man_bits is the code of the smallest normal value */
        code = (uint32_t)rintf(ldexpf(a, bias - 1 + man_bits));
    }
    return sign | (uint8_t)code;
}

static float fp8_decode(uint8_t b, int man_bits, int bias, int has_inf) {
    const int exp_bits = 7 - man_bits;
    const uint32_t e = (b >> man_bits) & ((1u << exp_bits) - 1u), m = b & ((1u << man_bits) - 1u);
    const float sgn = (b & 0x80) ? -1.0f : 1.0f;
    if (e == (1u << exp_bits) - 1u) {
        if (has_inf) return m == 0 ? sgn * INFINITY : NAN;
        if (m == (1u << man_bits) - 1u) return NAN;
    }
    if (e == 0) return sgn * ldexpf((float)m, 1 - bias - man_bits);
    return sgn * ldexpf((float)((1u << man_bits) | m), (int)e - bias - man_bits);
}

uint8_t oxb_fp8_e4m3_encode(float x) { return fp8_encode(x, 3, 7, 448.0f, 1, 0x7e, 0x7e, 0x7f); }
uint8_t oxb_fp8_e5m2_encode(float x) { return fp8_encode(x, 2, 15, 57344.0f, 0, 0x7b, 0x7c, 0x7e); }
float oxb_fp8_e4m3_decode(uint8_t b) { return fp8_decode(b, 3, 7, 0); }
float oxb_fp8_e5m2_decode(uint8_t b) { return fp8_decode(b, 2, 15, 1); }

/* One row (one position of one kv head) -> codes + scale.
 * INT8: model/src/kv_cache_quant.rs:46-62  scale = max(max|x| / 127, f32::EPSILON), q = round(x / scale) (half away
 *       from zero) clamped to +-127.
 * FP8:  model/src/kv_cache_quant.rs:519-540  scale = max(max|x| / FP8_MAX, f32::EPSILON), code = encode(x / scale).
 * Dequantisation (:69-71, :545-556) is code * scale in f32. */
int oxb_kv_quantize_row(int mode, const float* row, size_t n, uint8_t* codes, float* scale_out) {
    if (mode != OXB_KV_I8 && mode != OXB_KV_FP8_E4M3 && mode != OXB_KV_FP8_E5M2) return OXB_ERR_DIMENSION_MISMATCH;
    float max_abs = 0.0f;
    for (size_t i = 0; i < n; i++) max_abs = fmaxf(max_abs, fabsf(row[i]));
    const float top = mode == OXB_KV_I8 ? 127.0f : mode == OXB_KV_FP8_E4M3 ? 448.0f : 57344.0f;
    float scale = max_abs / top;
    if (!(scale >= FLT_EPSILON)) scale = FLT_EPSILON;
    for (size_t i = 0; i < n; i++) {
        const float t = row[i] / scale;
        if (mode == OXB_KV_I8) {
            float r = roundf(t);
            r = r < -127.0f ? -127.0f : r > 127.0f ? 127.0f : r;
            codes[i] = (uint8_t)(int8_t)r;
        } else {
            codes[i] = mode == OXB_KV_FP8_E4M3 ? oxb_fp8_e4m3_encode(t) : oxb_fp8_e5m2_encode(t);
        }
    }
    *scale_out = scale;
    return OXB_OK;
}

int oxb_kv_dequantize_row(int mode, const uint8_t* codes, size_t n, float scale, float* out) {
    for (size_t i = 0; i < n; i++) {
        switch (mode) {
            case OXB_KV_I8: out[i] = (float)(int8_t)codes[i] * scale; break;
            case OXB_KV_FP8_E4M3: out[i] = oxb_fp8_e4m3_decode(codes[i]) * scale; break;
            case OXB_KV_FP8_E5M2: out[i] = oxb_fp8_e5m2_decode(codes[i]) * scale; break;
            default: return OXB_ERR_DIMENSION_MISMATCH;
        }
    }
    return OXB_OK;
}

/* runtime/src/sampling.rs:84-91,182-189: Iterator::max_by keeps the LAST maximum. */
uint32_t oxb_argmax_last(const float* v, size_t n) {
    size_t best = 0;
    for (size_t i = 1; i < n; i++) if (v[i] >= v[best]) best = i;
    return (uint32_t)best;
}
/* kernels/src/gpu_backend/cuda_kernels.rs:407-436: strict '>' keeps the FIRST maximum. */
uint32_t oxb_argmax_first(const float* v, size_t n) {
    size_t best = 0;
    for (size_t i = 1; i < n; i++) if (v[i] > v[best]) best = i;
    return (uint32_t)best;
}

/* ------------------------------------------------------------------------- */
/* Sampler::sample, crates/oxibonsai-runtime/src/sampling.rs:84-177 (xorshift64 next_u64 :73-80).
 * temperature < 1e-6: greedy, the LAST maximum (Iterator::max_by).  Otherwise: v / temperature; keep the top_k
 * largest (top_k == 0 or >= n: all); softmax over the kept values; if top_p < 1: sort by probability descending,
 * keep the shortest prefix whose cumulative sum exceeds top_p (all but none if it never does), renormalise;
 * draw r = (next_u64 / u64::MAX) as f32 and return the first candidate whose cumulative probability reaches r
 * (the first candidate if none does).
 * The reference leaves the candidates in the order select_nth_unstable_by happens to produce when top_p == 1 and
 * sums the softmax in that order; this restatement always works in descending order of value, ties by ascending
 * index (a stable sort of the index-ordered buffer).  cand_idx / cand_p (capacity cap, may be NULL) receive the
 * final candidate list, *n_cand its length, *r_out the random draw. */
static uint64_t xorshift64(uint64_t* state) {
    uint64_t x = *state;
    x ^= x << 13;
    x ^= x >> 7;
    x ^= x << 17;
    *state = x;
    return x;
}

uint32_t oxb_sample(const float* logits, size_t n, float temperature, size_t top_k, float top_p, uint64_t* rng_state,
                    uint32_t* cand_idx, float* cand_p, size_t cap, size_t* n_cand, float* r_out) {
    if (n_cand) *n_cand = 0;
    if (n == 0) return 0;
    if (temperature < 1e-6f) return oxb_argmax_last(logits, n);
    const int filtered = top_k > 0 && top_k < n;
    size_t k = filtered ? top_k : n;
    uint32_t* idx = (uint32_t*)malloc(k * sizeof(uint32_t));
    float* p = (float*)malloc(k * sizeof(float));
    float max_val = -INFINITY;
    if (filtered) {
        /* sampling.rs:111-118 keeps the k largest in the order select_nth_unstable_by leaves them, which is
         * implementation-defined; here: descending, ties by ascending index (selection; n * k compares) */
        unsigned char* taken = (unsigned char*)calloc(n, 1);
        for (size_t j = 0; j < k; j++) {
            size_t best = n;
            float bv = 0.0f;
            for (size_t i = 0; i < n; i++) {
                if (taken[i]) continue;
                const float v = logits[i] / temperature;
                if (best == n || v > bv) best = i, bv = v;
            }
            taken[best] = 1;
            idx[j] = (uint32_t)best;
            p[j] = bv;
        }
        free(taken);
    } else {
        /* top-k off (or k >= n): the buffer stays in index order (sampling.rs:98-104) */
        for (size_t i = 0; i < n; i++) idx[i] = (uint32_t)i, p[i] = logits[i] / temperature;
    }
    for (size_t j = 0; j < k; j++) max_val = fmaxf(max_val, p[j]);  /* fold(NEG_INFINITY, f32::max), :121-125 */
    float sum = 0.0f;
    for (size_t j = 0; j < k; j++) {
        p[j] = expf(p[j] - max_val);
        sum += p[j];
    }
    for (size_t j = 0; j < k; j++) p[j] /= sum;
    if (top_p < 1.0f) {
        if (!filtered) {
            /* sort_by(|a, b| b.1.partial_cmp(&a.1)) is a stable sort (:136-137): descending probability, equal
             * probabilities keep index order.  Bottom-up merge sort. */
            uint32_t* ti = (uint32_t*)malloc(k * sizeof(uint32_t));
            float* tp = (float*)malloc(k * sizeof(float));
            for (size_t w = 1; w < k; w *= 2) {
                for (size_t lo = 0; lo < k; lo += 2 * w) {
                    const size_t mid = lo + w < k ? lo + w : k, hi = lo + 2 * w < k ? lo + 2 * w : k;
                    size_t a = lo, b = mid, o = lo;
                    while (a < mid && b < hi) {
                        if (p[b] > p[a]) tp[o] = p[b], ti[o++] = idx[b++];
                        else tp[o] = p[a], ti[o++] = idx[a++];
                    }
                    while (a < mid) tp[o] = p[a], ti[o++] = idx[a++];
                    while (b < hi) tp[o] = p[b], ti[o++] = idx[b++];
                }
                float* sp = p; p = tp; tp = sp;
                uint32_t* si = idx; idx = ti; ti = si;
            }
            free(ti);
            free(tp);
        }
        float cum = 0.0f;
        size_t cutoff = k ? k - 1 : 0;
        for (size_t j = 0; j < k; j++) {
            cum += p[j];
            if (cum > top_p) {
                cutoff = j;
                break;
            }
        }
        k = cutoff + 1;
        float s2 = 0.0f;
        for (size_t j = 0; j < k; j++) s2 += p[j];
        for (size_t j = 0; j < k; j++) p[j] /= s2;
    }
    const float r = (float)((double)xorshift64(rng_state) / (double)UINT64_MAX);
    if (r_out) *r_out = r;
    if (n_cand) *n_cand = k;
    for (size_t j = 0; j < k && j < cap; j++) {
        if (cand_idx) cand_idx[j] = idx[j];
        if (cand_p) cand_p[j] = p[j];
    }
    uint32_t tok = idx[0];
    float cum = 0.0f;
    for (size_t j = 0; j < k; j++) {
        cum += p[j];
        if (r <= cum) {
            tok = idx[j];
            break;
        }
    }
    free(idx);
    free(p);
    return tok;
}

/* Whole-model decode step: model/src/model/types/mod.rs:633-934 (embedding   */
/* row -> blocks -> output_norm -> LM head) around                            */
/* model/src/block/types/forward.rs:92-408 (one transformer block).           */
/* KV layout: model/src/kv_cache.rs:118-120  [layer][kv_head][pos][d].        */
/* ------------------------------------------------------------------------- */
struct oxb_state {
    float *k_cache, *v_cache;     /* [L][nkv][max_seq][hd], as attention reads them (after the cache's rounding) */
    int frozen;                   /* 1: the cache rows are given (oxb_state_load_rows); a forward stores nothing */
    uint8_t *k_codes, *v_codes;   /* quantised caches only: codes [L][nkv][max_seq][hd], scales [L][nkv][max_seq] */
    float *k_scale, *v_scale;
    float *cos_t, *sin_t;         /* [max_seq][hd/2] */
    float *hidden, *normed, *q, *k, *v, *qn, *kn, *qr, *kr, *attn, *proj, *gate, *up, *act, *down;
};

/* The same row products with every sum kept in double (block sums and the row total), rounded to float once:
 * not the reference's arithmetic but a check on it - with 24 more bits the order of the additions no longer
 * matters, so this is what any correct tier converges to. */
static void linear_fwd_f64(int fmt, const oxb_linear* l, const float* x, float* y) {
    const size_t bpr = l->k / OXB_QK, bb = fmt == 0 ? OXB_Q1_BYTES : OXB_TQ2_BYTES;
#pragma omp parallel for schedule(static) if (l->n_rows * bpr > 4096)
    for (size_t r = 0; r < l->n_rows; r++) {
        const uint8_t* row = l->blocks + r * bpr * bb;
        double sum = 0.0;
        for (size_t bi = 0; bi < bpr; bi++) {
            const uint8_t* b = row + bi * bb;
            const float* xb = x + bi * OXB_QK;
            double bs = 0.0;
            if (fmt == 0) {
                for (size_t j = 0; j < OXB_QK; j++) bs += ((b[2 + j / 8] >> (j % 8)) & 1u) ? (double)xb[j] : -(double)xb[j];
                sum += (double)q1_scale(b) * bs;
            } else {
                for (size_t byte = 0; byte < 32; byte++)
                    for (unsigned lane = 0; lane < 4; lane++) bs += (double)tq2_code(b[byte], lane) * (double)xb[byte * 4 + lane];
                sum += (double)tq2_scale(b) * bs;
            }
        }
        y[r] = (float)sum;
    }
}

static int linear_fwd(int fmt, const oxb_linear* l, const float* x, float* y) {
    if (fmt >= 4) /* the SIMD tier, itself held to the scalar kernels by the tests */
        return oxb_simd_gemv(fmt - 4, l->blocks, l->n_rows * (l->k / OXB_QK), x, l->k, y, l->n_rows, l->n_rows, l->k);
    if (fmt >= 2) {
        linear_fwd_f64(fmt - 2, l, x, y);
        return OXB_OK;
    }
    size_t nb = l->n_rows * (l->k / OXB_QK);
    return fmt == 0 ? oxb_gemv_q1(l->blocks, nb, x, l->k, y, l->n_rows, l->n_rows, l->k)
                    : oxb_gemv_tq2(l->blocks, nb, x, l->k, y, l->n_rows, l->n_rows, l->k);
}

oxb_state* oxb_state_new(const oxb_model* m) {
    oxb_state* s = (oxb_state*)calloc(1, sizeof(*s));
    if (!s) return NULL;
    size_t kv = m->n_layers * m->nkv * m->max_seq * m->hd;
    size_t qd = m->nq * m->hd, kd = m->nkv * m->hd;
    s->k_cache = (float*)calloc(kv, 4);
    s->v_cache = (float*)calloc(kv, 4);
    if (m->kv_mode >= OXB_KV_I8) {
        s->k_codes = (uint8_t*)calloc(kv, 1);
        s->v_codes = (uint8_t*)calloc(kv, 1);
        s->k_scale = (float*)calloc(kv / m->hd, 4);
        s->v_scale = (float*)calloc(kv / m->hd, 4);
    }
    s->cos_t = (float*)malloc(m->max_seq * (m->hd / 2) * 4);
    s->sin_t = (float*)malloc(m->max_seq * (m->hd / 2) * 4);
    oxb_rope_table(s->cos_t, s->sin_t, m->hd, m->max_seq, m->rope_theta);
    s->hidden = (float*)malloc(m->h * 4);
    s->normed = (float*)malloc(m->h * 4);
    s->q = (float*)malloc(qd * 4);  s->qn = (float*)malloc(qd * 4);  s->qr = (float*)malloc(qd * 4);
    s->k = (float*)malloc(kd * 4);  s->kn = (float*)malloc(kd * 4);  s->kr = (float*)malloc(kd * 4);
    s->v = (float*)malloc(kd * 4);
    s->attn = (float*)malloc(qd * 4);
    s->proj = (float*)malloc(m->h * 4);
    s->gate = (float*)malloc(m->inter * 4);
    s->up = (float*)malloc(m->inter * 4);
    s->act = (float*)malloc(m->inter * 4);
    s->down = (float*)malloc(m->h * 4);
    return s;
}

void oxb_state_free(oxb_state* s) {
    if (!s) return;
    free(s->k_cache); free(s->v_cache); free(s->cos_t); free(s->sin_t);
    free(s->k_codes); free(s->v_codes); free(s->k_scale); free(s->v_scale);
    free(s->hidden); free(s->normed); free(s->q); free(s->qn); free(s->qr);
    free(s->k); free(s->kn); free(s->kr); free(s->v); free(s->attn); free(s->proj);
    free(s->gate); free(s->up); free(s->act); free(s->down);
    free(s);
}

int oxb_forward_ex(const oxb_model* m, oxb_state* s, const float* hidden_in, size_t pos,
                   float* logits, float* normed_out) {
    if (pos >= m->max_seq) return OXB_ERR_DIMENSION_MISMATCH;
    const size_t h = m->h, hd = m->hd, half = hd / 2, nq = m->nq, nkv = m->nkv;
    const size_t group = nq / nkv;
    memcpy(s->hidden, hidden_in, h * 4);
    const float* c = s->cos_t + pos * half;
    const float* sn = s->sin_t + pos * half;
    for (size_t L = 0; L < m->n_layers; L++) {
        const oxb_layer* ly = &m->layers[L];
        int rc;
        oxb_rms_norm(s->hidden, ly->attn_norm, s->normed, h, m->eps);            /* forward.rs:94 */
        if ((rc = linear_fwd(m->fmt, &ly->q, s->normed, s->q))) return rc;       /* :172-174 */
        if ((rc = linear_fwd(m->fmt, &ly->k, s->normed, s->k))) return rc;
        if ((rc = linear_fwd(m->fmt, &ly->v, s->normed, s->v))) return rc;
        for (size_t hh = 0; hh < nq; hh++) {                                      /* :179-206 */
            oxb_rms_norm(s->q + hh * hd, ly->q_norm, s->qn + hh * hd, hd, m->eps);
            oxb_rope_apply(s->qn + hh * hd, s->qr + hh * hd, c, sn, half);
        }
        for (size_t hh = 0; hh < nkv; hh++) {
            oxb_rms_norm(s->k + hh * hd, ly->k_norm, s->kn + hh * hd, hd, m->eps);
            oxb_rope_apply(s->kn + hh * hd, s->kr + hh * hd, c, sn, half);
        }
        for (size_t hh = 0; hh < nkv && !s->frozen; hh++) {                       /* :209-213 */
            size_t off = ((L * nkv + hh) * m->max_seq + pos) * hd;
            if (m->kv_mode >= OXB_KV_I8) { /* a quantised cache: attention reads back code * scale */
                const size_t row = (L * nkv + hh) * m->max_seq + pos;
                oxb_kv_quantize_row(m->kv_mode, s->kr + hh * hd, hd, s->k_codes + off, &s->k_scale[row]);
                oxb_kv_quantize_row(m->kv_mode, s->v + hh * hd, hd, s->v_codes + off, &s->v_scale[row]);
                oxb_kv_dequantize_row(m->kv_mode, s->k_codes + off, hd, s->k_scale[row], s->k_cache + off);
                oxb_kv_dequantize_row(m->kv_mode, s->v_codes + off, hd, s->v_scale[row], s->v_cache + off);
                continue;
            }
            for (size_t d = 0; d < hd; d++) {
                float kv = s->kr[hh * hd + d], vv = s->v[hh * hd + d];
                if (m->kv_mode == OXB_KV_F16) { /* cuda_attn_kernels.rs:228-251 rounds to f16 on store */
                    kv = oxb_f16_to_f32(oxb_f32_to_f16(kv));
                    vv = oxb_f16_to_f32(oxb_f32_to_f16(vv));
                }
                s->k_cache[off + d] = kv;
                s->v_cache[off + d] = vv;
            }
        }
        for (size_t qh = 0; qh < nq; qh++) {                                      /* block/functions.rs:78-127 */
            size_t kvh = qh / group;
            size_t base = (L * nkv + kvh) * m->max_seq * hd;
            oxb_attention_head_windowed(s->qr + qh * hd, s->k_cache + base, s->v_cache + base,
                                        s->attn + qh * hd, pos + 1, hd, m->window, m->sinks);
        }
        if ((rc = linear_fwd(m->fmt, &ly->o, s->attn, s->proj))) return rc;      /* :389-392 */
        for (size_t i = 0; i < h; i++) s->hidden[i] += s->proj[i];
        oxb_rms_norm(s->hidden, ly->ffn_norm, s->normed, h, m->eps);             /* :393 */
        if ((rc = linear_fwd(m->fmt, &ly->gate, s->normed, s->gate))) return rc; /* :394-403 */
        if ((rc = linear_fwd(m->fmt, &ly->up, s->normed, s->up))) return rc;
        oxb_swiglu(s->gate, s->up, s->act, m->inter);                            /* :404 */
        if ((rc = linear_fwd(m->fmt, &ly->down, s->act, s->down))) return rc;    /* :405-408 */
        for (size_t i = 0; i < h; i++) s->hidden[i] += s->down[i];
    }
    oxb_rms_norm(s->hidden, m->final_norm, s->normed, h, m->eps);                /* mod.rs:869-870 */
    if (normed_out) memcpy(normed_out, s->normed, h * 4);
    if (logits) return linear_fwd(m->fmt, &m->lm_head, s->normed, logits);       /* mod.rs:874-880 */
    return OXB_OK;
}

/* n tokens through one linear layer: x [n][k] -> y [n][n_rows]. */
static int linear_batch(int fmt, const oxb_linear* l, const float* x, float* y, size_t n) {
    if (fmt >= 4)
        return oxb_simd_gemm_x4(fmt - 4, l->blocks, l->n_rows * (l->k / OXB_QK), x, n * l->k, y, n * l->n_rows, n, l->n_rows, l->k);
    for (size_t t = 0; t < n; t++) {
        int rc = linear_fwd(fmt, l, x + t * l->k, y + t * l->n_rows);
        if (rc) return rc;
    }
    return OXB_OK;
}

/* The reference's batched prefill has no arithmetic of its own: its parity test holds it to the token-by-token
 * forward (model/tests/metal_prefill_ternary_parity_tests.rs:226-366), and so does this - the operations of
 * oxb_forward_ex, applied to all n tokens one layer at a time. */
int oxb_forward_batch(const oxb_model* m, oxb_state* s, const float* hidden_in, size_t pos_start, size_t n,
                      float* logits, float* normed_out) {
    if (n == 0 || pos_start + n > m->max_seq || s->frozen || m->hd > 512) return OXB_ERR_DIMENSION_MISMATCH;
    const size_t h = m->h, hd = m->hd, half = hd / 2, nq = m->nq, nkv = m->nkv, inter = m->inter;
    const size_t group = nq / nkv, qd = nq * hd, kd = nkv * hd;
    float* hid = (float*)malloc(n * h * 4);
    float* nrm = (float*)malloc(n * h * 4);
    float* q = (float*)malloc(n * qd * 4);
    float* k = (float*)malloc(n * kd * 4);
    float* v = (float*)malloc(n * kd * 4);
    float* att = (float*)malloc(n * qd * 4);
    float* gate = (float*)malloc(n * inter * 4);
    float* up = (float*)malloc(n * inter * 4);
    int rc = OXB_OK;
    if (!hid || !nrm || !q || !k || !v || !att || !gate || !up) { rc = OXB_ERR_BUFFER_TOO_SMALL; goto out; }
    memcpy(hid, hidden_in, n * h * 4);
    for (size_t L = 0; L < m->n_layers && !rc; L++) {
        const oxb_layer* ly = &m->layers[L];
#pragma omp parallel for schedule(static)
        for (size_t t = 0; t < n; t++) oxb_rms_norm(hid + t * h, ly->attn_norm, nrm + t * h, h, m->eps);
        if ((rc = linear_batch(m->fmt, &ly->q, nrm, q, n))) break;
        if ((rc = linear_batch(m->fmt, &ly->k, nrm, k, n))) break;
        if ((rc = linear_batch(m->fmt, &ly->v, nrm, v, n))) break;
#pragma omp parallel for schedule(static)
        for (size_t t = 0; t < n; t++) {
            const size_t pos = pos_start + t;
            const float* c = s->cos_t + pos * half;
            const float* sn = s->sin_t + pos * half;
            float tmp[512];
            for (size_t hh = 0; hh < nq; hh++) {
                oxb_rms_norm(q + t * qd + hh * hd, ly->q_norm, tmp, hd, m->eps);
                oxb_rope_apply(tmp, q + t * qd + hh * hd, c, sn, half);
            }
            for (size_t hh = 0; hh < nkv; hh++) {
                float kr[512];
                oxb_rms_norm(k + t * kd + hh * hd, ly->k_norm, tmp, hd, m->eps);
                oxb_rope_apply(tmp, kr, c, sn, half);
                const size_t row = (L * nkv + hh) * m->max_seq + pos, off = row * hd;
                if (m->kv_mode >= OXB_KV_I8) {
                    oxb_kv_quantize_row(m->kv_mode, kr, hd, s->k_codes + off, &s->k_scale[row]);
                    oxb_kv_quantize_row(m->kv_mode, v + t * kd + hh * hd, hd, s->v_codes + off, &s->v_scale[row]);
                    oxb_kv_dequantize_row(m->kv_mode, s->k_codes + off, hd, s->k_scale[row], s->k_cache + off);
                    oxb_kv_dequantize_row(m->kv_mode, s->v_codes + off, hd, s->v_scale[row], s->v_cache + off);
                    continue;
                }
                for (size_t d = 0; d < hd; d++) {
                    float kv = kr[d], vv = v[t * kd + hh * hd + d];
                    if (m->kv_mode == OXB_KV_F16) {
                        kv = oxb_f16_to_f32(oxb_f32_to_f16(kv));
                        vv = oxb_f16_to_f32(oxb_f32_to_f16(vv));
                    }
                    s->k_cache[off + d] = kv;
                    s->v_cache[off + d] = vv;
                }
            }
        }
        /* every row of the run is in the cache now; token t reads positions 0 .. pos_start + t only */
#pragma omp parallel for schedule(dynamic, 1) collapse(2)
        for (size_t t = 0; t < n; t++)
            for (size_t qh = 0; qh < nq; qh++) {
                const size_t base = (L * nkv + qh / group) * m->max_seq * hd;
                oxb_attention_head_windowed(q + t * qd + qh * hd, s->k_cache + base, s->v_cache + base,
                                            att + t * qd + qh * hd, pos_start + t + 1, hd, m->window, m->sinks);
            }
        if ((rc = linear_batch(m->fmt, &ly->o, att, nrm, n))) break;
#pragma omp parallel for schedule(static)
        for (size_t t = 0; t < n; t++) {
            for (size_t i = 0; i < h; i++) hid[t * h + i] += nrm[t * h + i];
            oxb_rms_norm(hid + t * h, ly->ffn_norm, nrm + t * h, h, m->eps);
        }
        if ((rc = linear_batch(m->fmt, &ly->gate, nrm, gate, n))) break;
        if ((rc = linear_batch(m->fmt, &ly->up, nrm, up, n))) break;
#pragma omp parallel for schedule(static)
        for (size_t t = 0; t < n; t++) oxb_swiglu(gate + t * inter, up + t * inter, gate + t * inter, inter);
        if ((rc = linear_batch(m->fmt, &ly->down, gate, nrm, n))) break;
#pragma omp parallel for schedule(static)
        for (size_t t = 0; t < n; t++)
            for (size_t i = 0; i < h; i++) hid[t * h + i] += nrm[t * h + i];
    }
    if (!rc) {
        oxb_rms_norm(hid + (n - 1) * h, m->final_norm, s->normed, h, m->eps);
        if (normed_out) memcpy(normed_out, s->normed, h * 4);
        if (logits) rc = linear_fwd(m->fmt, &m->lm_head, s->normed, logits);
    }
out:
    free(hid); free(nrm); free(q); free(k); free(v); free(att); free(gate); free(up);
    return rc;
}

/* Test aid: rows pos0 .. pos0 + n - 1 of one (layer, kv head) as attention shall read them, e.g. the rows another
 * implementation stored; with oxb_state_freeze(s, 1) the forward then leaves the cache alone, so that its attention
 * runs over exactly those rows (its own K and V of the current position included). */
void oxb_state_load_rows(const oxb_model* m, oxb_state* s, size_t layer, size_t kv_head, size_t pos0, size_t n,
                         const float* k_rows, const float* v_rows) {
    const size_t off = ((layer * m->nkv + kv_head) * m->max_seq + pos0) * m->hd;
    memcpy(s->k_cache + off, k_rows, n * m->hd * 4);
    memcpy(s->v_cache + off, v_rows, n * m->hd * 4);
}
void oxb_state_freeze(oxb_state* s, int frozen) { s->frozen = frozen; }

const void* oxb_state_cache(const oxb_state* s, int which) {
    switch (which) {
        case 0: return s->k_cache;
        case 1: return s->v_cache;
        case 2: return s->k_codes;
        case 3: return s->v_codes;
        case 4: return s->k_scale;
        case 5: return s->v_scale;
        default: return NULL;
    }
}

int oxb_forward(const oxb_model* m, oxb_state* s, const float* hidden_in, size_t pos, float* logits) {
    return oxb_forward_ex(m, s, hidden_in, pos, logits, NULL);
}
