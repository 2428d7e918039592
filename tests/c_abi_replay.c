/*
 * c_abi_replay.c — the call sequence of a Rust `native-hip` tier, written in plain C against include/oxb_hip.h and
 * linked against the STATIC library liboxb_hip.a (what a Cargo build script links), not the .so the Python tests load.
 *
 *   init -> device info -> upload_weights_raw(bytes) -> gemv_q1_g128_cached(handle, x, n_rows, k)      (KG/mod.rs:445, 457)
 *        -> upload_weights_ternary(blocks) -> gemv_tq2_g128_cached                                     (KG/mod.rs:472, 484)
 *        -> per-layer uploads under caller-chosen handle ids, model create                             (KG/cuda_full_layer/mod.rs:250-268)
 *        -> prefill of 5 positions with the caller's RoPE rows                                         (KG/cuda_prefill/try_apis.rs:42)
 *        -> 3 decode steps, each with the caller's RoPE row, logits + greedy token                     (KG/cuda_full_layer/encode_q1.rs:881)
 *        -> the same weights as a model without LM head: normed hidden state of one step               (encode_q1.rs:813)
 *        -> destroy, shutdown.
 * KG = crates/oxibonsai-kernels/src/gpu_backend of the reference.
 *
 * Inputs come from a splitmix64 byte stream that tests/test_gpu_c_abi.py regenerates; every result is appended to the
 * file named by argv[1] as raw little-endian f32 / u32, where the test holds it to the CPU oracle.  Two known-answer
 * cases are checked here as well (all-ones codes, x = 1: the reference's own smoke values, gemv.rs:101-130).
 * Exit code 0 only if every call succeeded.
 */
#include <math.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "../include/oxb_hip.h"

#define CHECK(call)                                                                          \
    do {                                                                                     \
        int rc_ = (call);                                                                    \
        if (rc_ != OXB_HIP_OK) {                                                             \
            fprintf(stderr, "%s:%d: %s -> %d: %s\n", __FILE__, __LINE__, #call, rc_, oxb_hip_last_error()); \
            return 1;                                                                        \
        }                                                                                    \
    } while (0)

static uint8_t stream_byte(uint64_t seed, uint64_t i) { /* splitmix64 of (seed, i), top byte */
    uint64_t z = seed + (i + 1) * 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    z ^= z >> 31;
    return (uint8_t)(z >> 56);
}

/* n blocks of `bb` bytes; the f16 scale (at byte `d_at`) is forced into [2^-7, 2^-6) */
static uint8_t* make_blocks(uint64_t seed, size_t n, size_t bb, size_t d_at) {
    uint8_t* p = (uint8_t*)malloc(n * bb);
    if (!p) return NULL;
    for (size_t i = 0; i < n * bb; i++) p[i] = stream_byte(seed, i);
    for (size_t b = 0; b < n; b++) p[b * bb + d_at + 1] = (uint8_t)(0x20 | (p[b * bb + d_at + 1] & 0x03));
    return p;
}
static uint8_t* q1_blocks(uint64_t seed, size_t rows, size_t k) { return make_blocks(seed, rows * (k / 128), 18, 0); }
static uint8_t* tq2_blocks(uint64_t seed, size_t rows, size_t k) { return make_blocks(seed, rows * (k / 128), 34, 32); }

static float* make_f32(uint64_t seed, size_t n, float offset, float div) { /* offset + (byte - 128) / div */
    float* p = (float*)malloc(n * sizeof(float));
    if (!p) return NULL;
    for (size_t i = 0; i < n; i++) p[i] = offset + ((float)stream_byte(seed, i) - 128.0f) / div;
    return p;
}

static FILE* g_out;
static void put(const void* p, size_t bytes) { fwrite(p, 1, bytes, g_out); }

enum { N_LAYERS = 2, H = 256, INTER = 512, NQ = 4, NKV = 2, HD = 64, VOCAB = 160, MAX_SEQ = 32, N_PREFILL = 5, N_DECODE = 3 };
#define ROPE_THETA 10000.0f
#define EPS 1e-6f

static void rope_rows(uint32_t pos_start, uint32_t n, float* c, float* s) { /* RopeTable::new, rope.rs:27-48 */
    for (uint32_t p = 0; p < n; p++)
        for (uint32_t i = 0; i < HD / 2; i++) {
            const float freq = 1.0f / powf(ROPE_THETA, 2.0f * (float)i / (float)HD);
            const float angle = (float)(pos_start + p) * freq;
            c[p * (HD / 2) + i] = cosf(angle);
            s[p * (HD / 2) + i] = sinf(angle);
        }
}

static int known_answers(void) {
    /* one row, two blocks of all-ones codes with d = 0.5, x = 1: Q1 -> 2 * 128 * 0.5 = 128; TQ2 code 0b10 (+1) the same */
    uint8_t q1[2 * 18], tq[2 * 34];
    float x[256], y = 0.f;
    for (int i = 0; i < 256; i++) x[i] = 1.0f;
    for (int b = 0; b < 2; b++) {
        q1[b * 18] = 0x00, q1[b * 18 + 1] = 0x38; /* f16 0.5 */
        memset(q1 + b * 18 + 2, 0xFF, 16);
        memset(tq + b * 34, 0xAA, 32);
        tq[b * 34 + 32] = 0x00, tq[b * 34 + 33] = 0x38;
    }
    uint64_t id = 0;
    CHECK(oxb_hip_upload_q1_raw(&id, q1, sizeof q1));
    CHECK(oxb_hip_gemv(id, x, &y, 1, 256, 1));
    CHECK(oxb_hip_free_weight(id));
    if (y != 128.0f) { fprintf(stderr, "Q1 known answer: %g, expected 128\n", y); return 1; }
    id = 0;
    CHECK(oxb_hip_upload_tq2_raw(&id, tq, sizeof tq));
    CHECK(oxb_hip_gemv(id, x, &y, 1, 256, 1));
    CHECK(oxb_hip_free_weight(id));
    if (y != 128.0f) { fprintf(stderr, "TQ2 known answer: %g, expected 128\n", y); return 1; }
    return 0;
}

/* uploads one model's weights under caller-chosen ids (base + layer * 16 + slot) and fills the descriptor */
static int upload_model(int fmt, uint64_t seed, uint64_t base, oxb_layer_ids* ids, uint64_t* final_norm, uint64_t* lm_head, int with_lm) {
    const size_t qd = NQ * HD, kd = NKV * HD;
    for (uint32_t L = 0; L < N_LAYERS; L++) {
        const uint64_t s = seed + 100 * L, b = base + 16 * L;
        struct { uint64_t* id; uint64_t slot; size_t n; } vecs[] = {
            {&ids[L].attn_norm, 0, H}, {&ids[L].q_norm, 2, HD}, {&ids[L].k_norm, 3, HD}, {&ids[L].ffn_norm, 5, H}};
        for (size_t v = 0; v < 4; v++) {
            float* w = make_f32(s + vecs[v].slot, vecs[v].n, 1.0f, 256.0f);
            if (!w) return 1;
            *vecs[v].id = b + vecs[v].slot;
            CHECK(oxb_hip_upload_f32(vecs[v].id, w, vecs[v].n));
            free(w);
        }
        struct { uint64_t* id; uint64_t slot; size_t rows, k; } mats[] = {
            {&ids[L].qkv, 1, qd + 2 * kd, H}, {&ids[L].o, 4, H, qd}, {&ids[L].gate_up, 6, 2 * INTER, H}, {&ids[L].down, 7, H, INTER}};
        for (size_t m = 0; m < 4; m++) {
            uint8_t* a = fmt == OXB_HIP_FMT_Q1 ? q1_blocks(s + mats[m].slot, mats[m].rows, mats[m].k)
                                               : tq2_blocks(s + mats[m].slot, mats[m].rows, mats[m].k);
            if (!a) return 1;
            const size_t bytes = mats[m].rows * (mats[m].k / 128) * (fmt == OXB_HIP_FMT_Q1 ? 18 : 34);
            *mats[m].id = b + mats[m].slot;
            /* bytes only, as upload_weights_raw / upload_weights_ternary have them */
            CHECK(fmt == OXB_HIP_FMT_Q1 ? oxb_hip_upload_q1_raw(mats[m].id, a, bytes) : oxb_hip_upload_tq2_raw(mats[m].id, a, bytes));
            free(a);
        }
    }
    float* fn = make_f32(seed + 900, H, 1.0f, 256.0f);
    if (!fn) return 1;
    *final_norm = base + 900;
    CHECK(oxb_hip_upload_f32(final_norm, fn, H));
    free(fn);
    *lm_head = 0;
    if (with_lm) {
        uint8_t* a = fmt == OXB_HIP_FMT_Q1 ? q1_blocks(seed + 901, VOCAB, H) : tq2_blocks(seed + 901, VOCAB, H);
        if (!a) return 1;
        *lm_head = base + 901;
        const size_t bytes = (size_t)VOCAB * (H / 128) * (fmt == OXB_HIP_FMT_Q1 ? 18 : 34);
        CHECK(fmt == OXB_HIP_FMT_Q1 ? oxb_hip_upload_q1_raw(lm_head, a, bytes) : oxb_hip_upload_tq2_raw(lm_head, a, bytes));
        free(a);
    }
    return 0;
}

static int free_model_weights(const oxb_layer_ids* ids, uint64_t final_norm, uint64_t lm_head) {
    for (uint32_t L = 0; L < N_LAYERS; L++) {
        CHECK(oxb_hip_free_f32(ids[L].attn_norm));
        CHECK(oxb_hip_free_f32(ids[L].q_norm));
        CHECK(oxb_hip_free_f32(ids[L].k_norm));
        CHECK(oxb_hip_free_f32(ids[L].ffn_norm));
        CHECK(oxb_hip_free_weight(ids[L].qkv));
        CHECK(oxb_hip_free_weight(ids[L].o));
        CHECK(oxb_hip_free_weight(ids[L].gate_up));
        CHECK(oxb_hip_free_weight(ids[L].down));
    }
    CHECK(oxb_hip_free_f32(final_norm));
    if (lm_head) CHECK(oxb_hip_free_weight(lm_head));
    return 0;
}

static int run_model(int fmt, uint64_t seed) {
    oxb_layer_ids ids[N_LAYERS];
    uint64_t final_norm = 0, lm_head = 0, model = 0;
    if (upload_model(fmt, seed, 1000000 + 100000 * (uint64_t)fmt, ids, &final_norm, &lm_head, 1)) return 1;
    oxb_model_desc d;
    memset(&d, 0, sizeof d);
    d.fmt = fmt, d.n_layers = N_LAYERS, d.h = H, d.inter = INTER, d.nq = NQ, d.nkv = NKV, d.hd = HD, d.vocab = VOCAB;
    d.max_seq = MAX_SEQ, d.batch = 1, d.eps = EPS;
    d.rope_theta = 3.0f; /* deliberately not the caller's: every position used below gets its rows from the caller */
    d.layers = ids, d.final_norm = final_norm, d.lm_head = lm_head;
    CHECK(oxb_hip_model_create(&d, &model));

    float cs[N_PREFILL * HD / 2], sn[N_PREFILL * HD / 2];
    float* rows = make_f32(seed + 950, (size_t)(N_PREFILL + N_DECODE) * H, 0.0f, 32.0f);
    float* logits = (float*)malloc(VOCAB * sizeof(float));
    if (!rows || !logits) return 1;
    uint32_t token = 0;
    rope_rows(0, N_PREFILL, cs, sn);
    CHECK(oxb_hip_model_set_rope_rows(model, 0, N_PREFILL, cs, sn));
    CHECK(oxb_hip_prefill(model, 0, rows, N_PREFILL, 0, logits, &token));
    put(logits, VOCAB * sizeof(float));
    put(&token, 4);
    for (uint32_t step = 0; step < N_DECODE; step++) {
        const uint32_t pos = N_PREFILL + step;
        rope_rows(pos, 1, cs, sn);
        CHECK(oxb_hip_model_set_rope_rows(model, pos, 1, cs, sn));
        CHECK(oxb_hip_decode(model, rows + (size_t)pos * H, &pos, logits, &token));
        put(logits, VOCAB * sizeof(float));
        put(&token, 4);
    }
    const uint32_t graph = (uint32_t)oxb_hip_model_uses_graph(model);
    put(&graph, 4);
    CHECK(oxb_hip_model_destroy(model));

    /* the same layers without an LM head: one step at position 0 returns the normed hidden state */
    d.lm_head = 0, d.vocab = 0;
    d.rope_theta = ROPE_THETA;
    CHECK(oxb_hip_model_create(&d, &model));
    float normed[H];
    const uint32_t pos0 = 0;
    CHECK(oxb_hip_decode_hidden(model, rows, &pos0, normed));
    put(normed, sizeof normed);
    CHECK(oxb_hip_model_destroy(model));
    free(rows);
    free(logits);
    return free_model_weights(ids, final_norm, lm_head);
}

int main(int argc, char** argv) {
    if (argc < 2) {
        fprintf(stderr, "usage: %s <output file>\n", argv[0]);
        return 2;
    }
    if (oxb_hip_device_count() < 1) {
        fprintf(stderr, "no GPU: %s\n", oxb_hip_last_error());
        return 3;
    }
    CHECK(oxb_hip_init(0));
    char name[128];
    size_t free_b = 0, total_b = 0;
    CHECK(oxb_hip_device_info(name, sizeof name, &free_b, &total_b));
    printf("device: %s, %zu MiB free of %zu\n", name, free_b >> 20, total_b >> 20);
    g_out = fopen(argv[1], "wb");
    if (!g_out) {
        perror(argv[1]);
        return 2;
    }
    if (known_answers()) return 1;

    /* cached GEMV on weights uploaded by bytes: Q1 96 x 640, TQ2 80 x 1152 */
    {
        const uint32_t n = 96, k = 640;
        uint8_t* a = q1_blocks(11, n, k);
        float* x = make_f32(12, k, 0.0f, 64.0f);
        float y[96];
        uint64_t id = 0;
        if (!a || !x) return 1;
        CHECK(oxb_hip_upload_q1_raw(&id, a, (size_t)n * (k / 128) * 18));
        CHECK(oxb_hip_gemv(id, x, y, n, k, 1));
        CHECK(oxb_hip_free_weight(id));
        put(y, sizeof y);
        free(a), free(x);
    }
    {
        const uint32_t n = 80, k = 1152;
        uint8_t* a = tq2_blocks(21, n, k);
        float* x = make_f32(22, k, 0.0f, 64.0f);
        float y[80];
        uint64_t id = 0;
        if (!a || !x) return 1;
        CHECK(oxb_hip_upload_tq2_raw(&id, a, (size_t)n * (k / 128) * 34));
        CHECK(oxb_hip_gemv(id, x, y, n, k, 1));
        CHECK(oxb_hip_free_weight(id));
        put(y, sizeof y);
        free(a), free(x);
    }
    if (run_model(OXB_HIP_FMT_Q1, 3000)) return 1;
    if (run_model(OXB_HIP_FMT_TQ2, 4000)) return 1;
    CHECK(oxb_hip_synchronize());
    oxb_hip_shutdown();
    fclose(g_out);
    printf("c_abi_replay: ok\n");
    return 0;
}
