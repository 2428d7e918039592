/*
 * oxb_simd.cpp — C++ restatement of the reference's best x86 CPU tier, the
 * "CPU baseline" timed beside the GPU path.  TEST / BENCH INFRASTRUCTURE ONLY:
 * nothing in the shipped library links or calls it.
 *
 * Follows (structure, not text):
 *   tier selection   crates/oxibonsai-kernels/src/dispatch.rs:143-175
 *                    (AVX-512 f+bw+vl > AVX2+FMA > scalar, decided by CPUID at run time)
 *   Q1  GEMV AVX-512 crates/oxibonsai-kernels/src/simd_avx512.rs:573-654 (sign mask-blend :42-48)
 *   TQ2 GEMV AVX-512 crates/oxibonsai-kernels/src/simd_avx512.rs:138-225 (2-bit decode :66-85)
 *   Q1  GEMV AVX2    crates/oxibonsai-kernels/src/simd_avx2.rs:295-412
 *   TQ2 GEMV AVX2    crates/oxibonsai-kernels/src/simd_avx2.rs:420-497
 *   threading        crates/oxibonsai-kernels/src/parallel_tiled.rs:22-31,120-186,273-322
 *                    crates/oxibonsai-kernels/src/parallel.rs:161-222
 *                    (n_rows <= 32 direct; Q1 > 256 rows: tasks of 256 rows; TQ2: row tasks;
 *                     a std::thread pool with a shared work counter stands in for rayon)
 * The exact last-ulp summation order of the Rust SIMD tiers is parity unpinned
 * (it can only be fixed by running the Rust build); the tests hold this file to
 * the scalar oracle within the reference's own SIMD-vs-scalar tolerance.
 */
#include "oxb_oracle.h"

#include <immintrin.h>

#include <algorithm>
#include <atomic>
#include <condition_variable>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <mutex>
#include <thread>
#include <vector>

namespace {

enum Tier { TIER_SCALAR = 0, TIER_AVX2 = 1, TIER_AVX512 = 2 };

Tier detect_tier() {
    __builtin_cpu_init();
    if (__builtin_cpu_supports("avx512f") && __builtin_cpu_supports("avx512bw") &&
        __builtin_cpu_supports("avx512vl"))
        return TIER_AVX512;
    if (__builtin_cpu_supports("avx2") && __builtin_cpu_supports("fma")) return TIER_AVX2;
    return TIER_SCALAR;
}

inline float f16_bits_to_f32(const uint8_t* p) { return oxb_f16_to_f32((uint16_t)(p[0] | (p[1] << 8))); }

/* ------------------------------- AVX-512 -------------------------------- */
__attribute__((target("avx512f,avx512bw,avx512vl")))
void q1_rows_avx512(const uint8_t* blocks, const float* x, float* y, size_t row0, size_t row1, size_t bpr) {
    const __m512 neg1 = _mm512_set1_ps(-1.0f), pos1 = _mm512_set1_ps(1.0f);
    for (size_t r = row0; r < row1; r++) {
        const uint8_t* rb = blocks + r * bpr * OXB_Q1_BYTES;
        _mm_prefetch((const char*)(rb + bpr * OXB_Q1_BYTES), _MM_HINT_T0);
        __m512 acc0 = _mm512_setzero_ps(), acc1 = _mm512_setzero_ps();
        for (size_t bi = 0; bi < bpr; bi++) {
            const uint8_t* b = rb + bi * OXB_Q1_BYTES;
            _mm_prefetch((const char*)(b + OXB_Q1_BYTES), _MM_HINT_T0);
            const __m512 scale = _mm512_set1_ps(f16_bits_to_f32(b));
            const float* xb = x + bi * OXB_QK;
            for (int c = 0; c < 8; c++) {
                __mmask16 m = (__mmask16)(b[2 + 2 * c] | (b[3 + 2 * c] << 8));
                __m512 sgn = _mm512_mask_blend_ps(m, neg1, pos1);
                __m512 sx = _mm512_mul_ps(sgn, _mm512_loadu_ps(xb + 16 * c));
                if (c & 1) acc1 = _mm512_fmadd_ps(scale, sx, acc1);
                else       acc0 = _mm512_fmadd_ps(scale, sx, acc0);
            }
        }
        y[r] = _mm512_reduce_add_ps(_mm512_add_ps(acc0, acc1));
    }
}

__attribute__((target("avx512f,avx512bw,avx512vl")))
inline __m512 tq2_decode16_avx512(uint32_t packed) {
    const __m512i shifts = _mm512_setr_epi32(0, 2, 4, 6, 8, 10, 12, 14, 16, 18, 20, 22, 24, 26, 28, 30);
    const __m512i one = _mm512_set1_epi32(1), three = _mm512_set1_epi32(3);
    __m512i idx = _mm512_and_si512(_mm512_srlv_epi32(_mm512_set1_epi32((int)packed), shifts), three);
    __m512i val = _mm512_sub_epi32(_mm512_srli_epi32(idx, 1),
                                   _mm512_sub_epi32(one, _mm512_min_epu32(idx, one)));
    __mmask16 reserved = _mm512_cmpeq_epi32_mask(idx, three);
    return _mm512_cvtepi32_ps(_mm512_mask_mov_epi32(val, reserved, _mm512_setzero_si512()));
}

__attribute__((target("avx512f,avx512bw,avx512vl")))
void tq2_rows_avx512(const uint8_t* blocks, const float* x, float* y, size_t row0, size_t row1, size_t bpr) {
    for (size_t r = row0; r < row1; r++) {
        const uint8_t* rb = blocks + r * bpr * OXB_TQ2_BYTES;
        _mm_prefetch((const char*)(rb + bpr * OXB_TQ2_BYTES), _MM_HINT_T0);
        float row_sum = 0.0f;
        for (size_t bi = 0; bi < bpr; bi++) {
            const uint8_t* b = rb + bi * OXB_TQ2_BYTES;
            _mm_prefetch((const char*)(b + OXB_TQ2_BYTES), _MM_HINT_T0);
            const float* xb = x + bi * OXB_QK;
            __m512 acc0 = _mm512_setzero_ps(), acc1 = _mm512_setzero_ps();
            for (int g = 0; g < 4; g++) {
                uint32_t p0, p1;
                std::memcpy(&p0, b + 8 * g, 4);
                std::memcpy(&p1, b + 8 * g + 4, 4);
                acc0 = _mm512_fmadd_ps(tq2_decode16_avx512(p0), _mm512_loadu_ps(xb + 32 * g), acc0);
                acc1 = _mm512_fmadd_ps(tq2_decode16_avx512(p1), _mm512_loadu_ps(xb + 32 * g + 16), acc1);
            }
            row_sum += f16_bits_to_f32(b + 32) * _mm512_reduce_add_ps(_mm512_add_ps(acc0, acc1));
        }
        y[r] = row_sum;
    }
}

/* Four token rows at a time over the same weight rows: every (token, weight row) sum is formed by exactly the
 * operations of the single-token kernels above, in the same order, so the results are the same bits; what is
 * shared is the decoded sign / code vector of a chunk, and four independent accumulator chains keep the FMA units
 * busy.  A test aid for prompts of thousands of tokens (oxb_simd_gemm_x4), not one of the reference's tiers. */
__attribute__((target("avx512f,avx512bw,avx512vl")))
void q1_rows_avx512_x4(const uint8_t* blocks, const float* x, size_t ldx, float* y, size_t ldy, size_t row0, size_t row1,
                       size_t bpr) {
    /* two weight rows per pass, so that each activation chunk is loaded once for both */
    for (size_t r = row0; r < row1; r += 2) {
        const bool two = r + 1 < row1;
        const uint8_t* rb0 = blocks + r * bpr * OXB_Q1_BYTES;
        const uint8_t* rb1 = two ? rb0 + bpr * OXB_Q1_BYTES : rb0;
        __m512 a0[4], a1[4], b0[4], b1[4];   /* a: row r, b: row r + 1; 0 / 1: even / odd chunks */
        for (int t = 0; t < 4; t++) a0[t] = a1[t] = b0[t] = b1[t] = _mm512_setzero_ps();
        for (size_t bi = 0; bi < bpr; bi++) {
            const uint8_t* pa = rb0 + bi * OXB_Q1_BYTES;
            const uint8_t* pb = rb1 + bi * OXB_Q1_BYTES;
            const float da = f16_bits_to_f32(pa), db = f16_bits_to_f32(pb);
            const __m512 sa = _mm512_set1_ps(da), na = _mm512_set1_ps(-da), sb = _mm512_set1_ps(db), nb = _mm512_set1_ps(-db);
            const float* xb = x + bi * OXB_QK;
            for (int c = 0; c < 8; c++) {
                uint16_t ua, ub;   /* little-endian host: the two mask bytes as they lie */
                std::memcpy(&ua, pa + 2 + 2 * c, 2);
                std::memcpy(&ub, pb + 2 + 2 * c, 2);
                const __mmask16 ma = (__mmask16)ua, mb = (__mmask16)ub;
                /* fma(d, +-x, acc) and fma(+-d, x, acc) round the same exact value: the sign goes to the scale once */
                const __m512 wa = _mm512_mask_blend_ps(ma, na, sa), wb = _mm512_mask_blend_ps(mb, nb, sb);
                for (int t = 0; t < 4; t++) {
                    const __m512 xv = _mm512_loadu_ps(xb + t * ldx + 16 * c);
                    if (c & 1) { a1[t] = _mm512_fmadd_ps(wa, xv, a1[t]); b1[t] = _mm512_fmadd_ps(wb, xv, b1[t]); }
                    else       { a0[t] = _mm512_fmadd_ps(wa, xv, a0[t]); b0[t] = _mm512_fmadd_ps(wb, xv, b0[t]); }
                }
            }
        }
        for (int t = 0; t < 4; t++) {
            y[t * ldy + r] = _mm512_reduce_add_ps(_mm512_add_ps(a0[t], a1[t]));
            if (two) y[t * ldy + r + 1] = _mm512_reduce_add_ps(_mm512_add_ps(b0[t], b1[t]));
        }
    }
}

__attribute__((target("avx512f,avx512bw,avx512vl")))
void tq2_rows_avx512_x4(const uint8_t* blocks, const float* x, size_t ldx, float* y, size_t ldy, size_t row0, size_t row1,
                        size_t bpr) {
    for (size_t r = row0; r < row1; r++) {
        const uint8_t* rb = blocks + r * bpr * OXB_TQ2_BYTES;
        float row_sum[4] = {0.0f, 0.0f, 0.0f, 0.0f};
        for (size_t bi = 0; bi < bpr; bi++) {
            const uint8_t* b = rb + bi * OXB_TQ2_BYTES;
            const float* xb = x + bi * OXB_QK;
            __m512 acc0[4], acc1[4];
            for (int t = 0; t < 4; t++) acc0[t] = acc1[t] = _mm512_setzero_ps();
            for (int g = 0; g < 4; g++) {
                uint32_t p0, p1;
                std::memcpy(&p0, b + 8 * g, 4);
                std::memcpy(&p1, b + 8 * g + 4, 4);
                const __m512 w0 = tq2_decode16_avx512(p0), w1 = tq2_decode16_avx512(p1);
                for (int t = 0; t < 4; t++) {
                    acc0[t] = _mm512_fmadd_ps(w0, _mm512_loadu_ps(xb + t * ldx + 32 * g), acc0[t]);
                    acc1[t] = _mm512_fmadd_ps(w1, _mm512_loadu_ps(xb + t * ldx + 32 * g + 16), acc1[t]);
                }
            }
            const float d = f16_bits_to_f32(b + 32);
            for (int t = 0; t < 4; t++) row_sum[t] += d * _mm512_reduce_add_ps(_mm512_add_ps(acc0[t], acc1[t]));
        }
        for (int t = 0; t < 4; t++) y[t * ldy + r] = row_sum[t];
    }
}

/* -------------------------------- AVX2 ---------------------------------- */
__attribute__((target("avx2,fma")))
inline float hsum256(__m256 v) {
    __m128 s = _mm_add_ps(_mm256_castps256_ps128(v), _mm256_extractf128_ps(v, 1));
    s = _mm_add_ps(s, _mm_movehdup_ps(s));
    s = _mm_add_ss(s, _mm_movehl_ps(s, s));
    return _mm_cvtss_f32(s);
}

__attribute__((target("avx2,fma")))
inline __m256 q1_signs8_avx2(uint8_t bits) {
    const __m256i sel = _mm256_setr_epi32(1, 2, 4, 8, 16, 32, 64, 128);
    __m256i hit = _mm256_cmpeq_epi32(_mm256_and_si256(_mm256_set1_epi32(bits), sel), _mm256_setzero_si256());
    return _mm256_blendv_ps(_mm256_set1_ps(1.0f), _mm256_set1_ps(-1.0f), _mm256_castsi256_ps(hit));
}

__attribute__((target("avx2,fma")))
inline __m256 q1_block_avx2(const uint8_t* b, const float* xb, __m256 acc) {
    const __m256 scale = _mm256_set1_ps(f16_bits_to_f32(b));
    for (int c = 0; c < 16; c++)
        acc = _mm256_fmadd_ps(scale, _mm256_mul_ps(q1_signs8_avx2(b[2 + c]), _mm256_loadu_ps(xb + 8 * c)), acc);
    return acc;
}

__attribute__((target("avx2,fma")))
void q1_rows_avx2(const uint8_t* blocks, const float* x, float* y, size_t row0, size_t row1, size_t bpr) {
    for (size_t r = row0; r < row1; r++) {
        const uint8_t* rb = blocks + r * bpr * OXB_Q1_BYTES;
        __m256 acc0 = _mm256_setzero_ps(), acc1 = _mm256_setzero_ps();
        size_t bi = 0;
        for (; bi + 1 < bpr; bi += 2) { /* even block -> acc0, odd block -> acc1 */
            acc0 = q1_block_avx2(rb + bi * OXB_Q1_BYTES, x + bi * OXB_QK, acc0);
            acc1 = q1_block_avx2(rb + (bi + 1) * OXB_Q1_BYTES, x + (bi + 1) * OXB_QK, acc1);
        }
        if (bi < bpr) acc0 = q1_block_avx2(rb + bi * OXB_Q1_BYTES, x + bi * OXB_QK, acc0);
        y[r] = hsum256(_mm256_add_ps(acc0, acc1));
    }
}

__attribute__((target("avx2,fma")))
inline __m256 tq2_decode8_avx2(uint32_t packed16) {
    const __m256i shifts = _mm256_setr_epi32(0, 2, 4, 6, 8, 10, 12, 14);
    const __m256i one = _mm256_set1_epi32(1), three = _mm256_set1_epi32(3);
    __m256i idx = _mm256_and_si256(_mm256_srlv_epi32(_mm256_set1_epi32((int)packed16), shifts), three);
    __m256i val = _mm256_sub_epi32(_mm256_srli_epi32(idx, 1), _mm256_sub_epi32(one, _mm256_min_epu32(idx, one)));
    val = _mm256_andnot_si256(_mm256_cmpeq_epi32(idx, three), val);
    return _mm256_cvtepi32_ps(val);
}

__attribute__((target("avx2,fma")))
void tq2_rows_avx2(const uint8_t* blocks, const float* x, float* y, size_t row0, size_t row1, size_t bpr) {
    for (size_t r = row0; r < row1; r++) {
        const uint8_t* rb = blocks + r * bpr * OXB_TQ2_BYTES;
        float row_sum = 0.0f;
        for (size_t bi = 0; bi < bpr; bi++) {
            const uint8_t* b = rb + bi * OXB_TQ2_BYTES;
            const float* xb = x + bi * OXB_QK;
            __m256 acc0 = _mm256_setzero_ps(), acc1 = _mm256_setzero_ps();
            for (int p = 0; p < 8; p++) {
                uint32_t lo = (uint32_t)(b[4 * p] | (b[4 * p + 1] << 8));
                uint32_t hi = (uint32_t)(b[4 * p + 2] | (b[4 * p + 3] << 8));
                acc0 = _mm256_fmadd_ps(tq2_decode8_avx2(lo), _mm256_loadu_ps(xb + 16 * p), acc0);
                acc1 = _mm256_fmadd_ps(tq2_decode8_avx2(hi), _mm256_loadu_ps(xb + 16 * p + 8), acc1);
            }
            row_sum += f16_bits_to_f32(b + 32) * hsum256(_mm256_add_ps(acc0, acc1));
        }
        y[r] = row_sum;
    }
}

/* ------------------------------ dispatch -------------------------------- */
void rows_kernel(int fmt, Tier t, const uint8_t* blocks, const float* x, float* y,
                 size_t row0, size_t row1, size_t bpr) {
    if (t == TIER_AVX512) {
        if (fmt == 0) q1_rows_avx512(blocks, x, y, row0, row1, bpr);
        else          tq2_rows_avx512(blocks, x, y, row0, row1, bpr);
    } else if (t == TIER_AVX2) {
        if (fmt == 0) q1_rows_avx2(blocks, x, y, row0, row1, bpr);
        else          tq2_rows_avx2(blocks, x, y, row0, row1, bpr);
    } else {
        size_t bb = fmt == 0 ? OXB_Q1_BYTES : OXB_TQ2_BYTES;
        size_t n = row1 - row0;
        if (fmt == 0) oxb_gemv_q1(blocks + row0 * bpr * bb, n * bpr, x, bpr * OXB_QK, y + row0, n, n, bpr * OXB_QK);
        else          oxb_gemv_tq2(blocks + row0 * bpr * bb, n * bpr, x, bpr * OXB_QK, y + row0, n, n, bpr * OXB_QK);
    }
}

/* A fixed pool; parallel_for hands out [begin,end) chunks from a shared counter. */
class Pool {
public:
    explicit Pool(unsigned n) : n_(std::max(1u, n)) {
        for (unsigned i = 1; i < n_; i++) workers_.emplace_back([this] { worker(); });
    }
    ~Pool() {
        { std::lock_guard<std::mutex> g(mu_); stop_ = true; gen_++; }
        cv_.notify_all();
        for (auto& t : workers_) t.join();
    }
    unsigned size() const { return n_; }
    void parallel_for(size_t n_tasks, const std::function<void(size_t)>& fn) {
        if (n_ == 1 || n_tasks <= 1) { for (size_t i = 0; i < n_tasks; i++) fn(i); return; }
        {
            std::lock_guard<std::mutex> g(mu_);
            fn_ = &fn; total_ = n_tasks; next_.store(0); pending_ = n_ - 1; gen_++;
        }
        cv_.notify_all();
        drain();
        std::unique_lock<std::mutex> lk(mu_);
        done_cv_.wait(lk, [this] { return pending_ == 0; });
        fn_ = nullptr;
    }
private:
    void drain() {
        for (;;) {
            size_t i = next_.fetch_add(1);
            if (i >= total_) break;
            (*fn_)(i);
        }
    }
    void worker() {
        unsigned long seen = 0;
        for (;;) {
            {
                std::unique_lock<std::mutex> lk(mu_);
                cv_.wait(lk, [&] { return gen_ != seen; });
                seen = gen_;
                if (stop_) return;
            }
            drain();
            { std::lock_guard<std::mutex> g(mu_); if (--pending_ == 0) done_cv_.notify_one(); }
        }
    }
    unsigned n_;
    std::vector<std::thread> workers_;
    std::mutex mu_;
    std::condition_variable cv_, done_cv_;
    const std::function<void(size_t)>* fn_ = nullptr;
    size_t total_ = 0;
    std::atomic<size_t> next_{0};
    unsigned pending_ = 0;
    unsigned long gen_ = 0;
    bool stop_ = false;
};

Pool* g_pool = nullptr;
Tier g_tier = TIER_SCALAR;
std::once_flag g_once;
unsigned g_threads_req = 0;

void ensure_init() {
    std::call_once(g_once, [] {
        g_tier = detect_tier();
        /* OXB_SIMD_TIER=scalar|avx2|avx512 lowers the tier below what the CPU offers (never above it), so that
         * the AVX2 path can be run and checked on an AVX-512 host. */
        if (const char* want = std::getenv("OXB_SIMD_TIER")) {
            Tier t = g_tier;
            if (!std::strcmp(want, "scalar")) t = TIER_SCALAR;
            else if (!std::strcmp(want, "avx2")) t = TIER_AVX2;
            else if (!std::strcmp(want, "avx512")) t = TIER_AVX512;
            if (t < g_tier) g_tier = t;
        }
        unsigned n = g_threads_req ? g_threads_req : std::thread::hardware_concurrency();
        g_pool = new Pool(n ? n : 1);
    });
}

constexpr size_t DIRECT_MAX_ROWS = 32;   /* parallel_tiled.rs:22-31 */
constexpr size_t L2_TILE_ROWS = 256;

int gemv_impl(int fmt, const uint8_t* blocks, size_t n_blocks, const float* x, size_t x_len,
              float* y, size_t y_len, size_t n_rows, size_t k) {
    if (k % OXB_QK) return OXB_ERR_NOT_BLOCK_ALIGNED;
    if (x_len < k) return OXB_ERR_DIMENSION_MISMATCH;
    if (y_len < n_rows) return OXB_ERR_BUFFER_TOO_SMALL;
    size_t bpr = k / OXB_QK;
    if (n_blocks < n_rows * bpr) return OXB_ERR_BUFFER_TOO_SMALL;
    ensure_init();
    if (n_rows <= DIRECT_MAX_ROWS) { rows_kernel(fmt, g_tier, blocks, x, y, 0, n_rows, bpr); return OXB_OK; }
    /* Q1: tasks of 256 rows once n_rows > 256, else row ranges; TQ2: row tasks
     * (rayon would split these adaptively: a chunk of rows per grab stands in). */
    size_t chunk;
    if (fmt == 0 && n_rows > L2_TILE_ROWS) chunk = L2_TILE_ROWS;
    else chunk = std::max<size_t>(1, n_rows / (g_pool->size() * 8));
    size_t n_tasks = (n_rows + chunk - 1) / chunk;
    g_pool->parallel_for(n_tasks, [&](size_t t) {
        size_t r0 = t * chunk, r1 = std::min(n_rows, r0 + chunk);
        rows_kernel(fmt, g_tier, blocks, x, y, r0, r1, bpr);
    });
    return OXB_OK;
}

}  // namespace

extern "C" {

/* 0 scalar, 1 AVX2+FMA, 2 AVX-512 — what dispatch.rs:143-175 would pick on this host. */
int oxb_simd_tier(void) { ensure_init(); return (int)g_tier; }
int oxb_simd_threads(void) { ensure_init(); return (int)g_pool->size(); }
/* Lower the tier at run time (0 scalar, 1 AVX2+FMA, 2 AVX-512); a tier the CPU lacks is refused (-1).
 * Returns the tier now in use.  The reference fixes its tier once per process (dispatch.rs:143-175); this
 * switch exists so that one test process can hold every tier the host offers to the scalar oracle. */
int oxb_simd_set_tier(int tier) {
    ensure_init();
    if (tier < 0 || tier > (int)detect_tier()) return -1;
    g_tier = (Tier)tier;
    return (int)g_tier;
}
/* Must be called before the first kernel call to take effect (0 = all host cores). */
void oxb_simd_set_threads(int n) { g_threads_req = n > 0 ? (unsigned)n : 0; }

int oxb_simd_gemv(int fmt, const uint8_t* blocks, size_t n_blocks, const float* x, size_t x_len,
                  float* y, size_t y_len, size_t n_rows, size_t k) {
    return gemv_impl(fmt, blocks, n_blocks, x, x_len, y, y_len, n_rows, k);
}

/* GEMM: m < 4 sequential over tokens, else token rows in parallel, each a
 * single-thread GEMV over all weight rows (parallel.rs:26,224-288). */
int oxb_simd_gemm(int fmt, const uint8_t* blocks, size_t n_blocks, const float* x, size_t x_len,
                  float* y, size_t y_len, size_t m, size_t n_rows, size_t k) {
    if (k % OXB_QK) return OXB_ERR_NOT_BLOCK_ALIGNED;
    if (x_len < m * k) return OXB_ERR_DIMENSION_MISMATCH;
    if (y_len < m * n_rows) return OXB_ERR_BUFFER_TOO_SMALL;
    size_t bpr = k / OXB_QK;
    if (n_blocks < n_rows * bpr) return OXB_ERR_BUFFER_TOO_SMALL;
    ensure_init();
    if (m < 4) {
        for (size_t mi = 0; mi < m; mi++) rows_kernel(fmt, g_tier, blocks, x + mi * k, y + mi * n_rows, 0, n_rows, bpr);
        return OXB_OK;
    }
    g_pool->parallel_for(m, [&](size_t mi) {
        rows_kernel(fmt, g_tier, blocks, x + mi * k, y + mi * n_rows, 0, n_rows, bpr);
    });
    return OXB_OK;
}

/* The same product as oxb_simd_gemm, bit for bit, for long prompts: on the AVX-512 tier four token rows share each
 * decoded weight chunk (above); tasks are (group of four tokens) x (run of 1024 weight rows).  Other tiers and the
 * last m % 4 token rows take oxb_simd_gemm's route.  Not a restatement of a reference tier: a test aid. */
int oxb_simd_gemm_x4(int fmt, const uint8_t* blocks, size_t n_blocks, const float* x, size_t x_len,
                     float* y, size_t y_len, size_t m, size_t n_rows, size_t k) {
    if (k % OXB_QK) return OXB_ERR_NOT_BLOCK_ALIGNED;
    if (x_len < m * k) return OXB_ERR_DIMENSION_MISMATCH;
    if (y_len < m * n_rows) return OXB_ERR_BUFFER_TOO_SMALL;
    size_t bpr = k / OXB_QK;
    if (n_blocks < n_rows * bpr) return OXB_ERR_BUFFER_TOO_SMALL;
    ensure_init();
    const size_t m4 = g_tier == TIER_AVX512 ? m / 4 : 0;
    if (m4) {
        const size_t chunk = 1024, rc = (n_rows + chunk - 1) / chunk;
        g_pool->parallel_for(m4 * rc, [&](size_t task) {
            const size_t g = task / rc, r0 = (task % rc) * chunk, r1 = std::min(n_rows, r0 + chunk);
            if (fmt == 0) q1_rows_avx512_x4(blocks, x + 4 * g * k, k, y + 4 * g * n_rows, n_rows, r0, r1, bpr);
            else          tq2_rows_avx512_x4(blocks, x + 4 * g * k, k, y + 4 * g * n_rows, n_rows, r0, r1, bpr);
        });
    }
    const size_t done = 4 * m4;
    if (done < m)
        return oxb_simd_gemm(fmt, blocks, n_blocks, x + done * k, x_len - done * k, y + done * n_rows, y_len - done * n_rows,
                             m - done, n_rows, k);
    return OXB_OK;
}


}  // extern "C"
