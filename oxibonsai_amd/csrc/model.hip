// model.hip — fused whole-model decode behind the C ABI.
//
// Stands in for the reference's fused GPU forward
//   try_cuda_full_forward[_ternary]_with_gpu_lm_head   gpu_backend/cuda_full_layer/encode_q1.rs:881, encode_ternary.rs:755
//   encode_layer_device / encode_layer_into_ternary     encode_q1.rs:297-463, encode_ternary.rs:116-291
//   CudaKvCache (FP16, [layer][kv_head][max_seq][hd])   gpu_backend/cuda_full_layer/mod.rs:112-139
//   graph capture / replay of the whole token            encode_q1.rs:569-797
// and for GpuBackendTrait::batch_ffn_phase (gpu_backend/mod.rs:519).
// One decode step is a fixed kernel sequence that reads the token position from device memory,
// so it is captured once into a hipGraph and replayed for every following token.  Logits stay on
// the device; the greedy token id comes from an on-device argmax (the reference's Metal tier does
// the same, metal_full_layer/functions_3.rs:676-720).
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>

#include <cmath>
#include <cstdlib>
#include <cstring>
#include <memory>
#include <vector>

#include "../../include/oxb_hip.h"
#include "../../include/oxb_hip_measure.h"
#include "gemm_kernels.h"
#include "gguf.h"
#include "gemv_kernels.h"
#include "kv_quant_device.h"
#include "layer_kernels.h"
#include "prefill_kernels.h"
#include "runtime_internal.h"
#include "token_kernels.h"

namespace oxb {

struct Model {
    oxb_model_desc d;
    std::vector<oxb_layer_ids> layers;
    // activations
    float *hidden = nullptr, *qkv = nullptr, *attn_part = nullptr, *attn_out = nullptr,
          *gu = nullptr, *act = nullptr, *logits = nullptr;  // gu: [batch][2 inter] gate || up sums, act: [batch][inter] SwiGLU output
    uint32_t *tokens = nullptr, *pos = nullptr;
    // pinned host staging of a decode call's small transfers (embedding rows and positions in, tokens out): copies from
    // and to pageable memory go through the runtime's own staging and cost about 10 us per call more
    float* h_hidden = nullptr;
    uint32_t *h_pos = nullptr, *h_tokens = nullptr;
    uint32_t* attn_done = nullptr;  // [batch][nkv] arrival counters of the attention workgroups, 0 between launches
    void* argmax_ws = nullptr;
    // KV cache: rows of hd fp16 values or one-byte codes, a quantised cache also one f32 scale per row.  Contiguous:
    // [batch][n_layers][nkv][row_stride] rows; paged: a pool [n_pages][n_layers][nkv][2^page_shift] rows and, per
    // sequence, a table of page numbers (kv_quant_device.h: OxbKvLayout)
    void *k_cache = nullptr, *v_cache = nullptr;
    float *k_scale = nullptr, *v_scale = nullptr;
    uint32_t kv_mode = OXB_KV_F16, row_stride = 0, window = 0, sinks = 0;
    uint32_t page_shift = 0, n_pages = 0, table_stride = 0;   // n_pages 0: contiguous
    std::vector<uint32_t> free_pages;                          // stack of free physical pages
    std::vector<std::vector<uint32_t>> seq_pages;              // pages of each sequence slot, in position order
    std::vector<uint32_t> h_table;                             // [batch][table_stride], mirrored in d_table
    uint32_t* d_table = nullptr;
    bool table_dirty = false;
    float *cos_t = nullptr, *sin_t = nullptr;
    uint32_t chunk = 0, n_splits = 0;
    // graph
    hipGraphExec_t graph_exec = nullptr;
    uint64_t checked_gen = 0;  // g_rt.weights_gen when every handle was last looked up
    uint64_t graph_gen = 0;  // g_rt.weights_gen at capture: the graph holds the weights' device pointers of that moment
    bool graph_failed = false;
    bool want_logits_in_graph = true;
    size_t logits_cap = 0;  // floats m.logits holds
    std::vector<void*> allocs;
    // prefill activations for up to pf_cap token rows (allocated on first use)
    uint32_t pf_cap = 0;
    float *pf_hidden = nullptr, *pf_qkv = nullptr, *pf_attn = nullptr, *pf_gu = nullptr;
    std::vector<void*> pf_allocs;
    GemmWorkspace gws;  // GEMM scratch of the captured large-batch decode step: sized at creation, never moved
    DevBuf gpack;       // quantised activation vectors of the captured GEMV-based step (batches of two to eight): likewise
    DevBuf gpack_o;     // the O projection's quantised input where the attention kernel writes it itself; starts as zeros (= zero vectors) and
                        // nothing else writes it, so the slots of a last vector group's absent vectors stay zero vectors
    // a model loaded from a file owns the weights it uploaded
    std::vector<uint64_t> owned_mats, owned_vecs;
    DevBuf tok_hist, tok_ids;  // token history of the on-device generation loop; prompt ids of a token prefill
    DevBuf sample_ws, rng;     // sampler scratch and per-sequence xorshift64 states
};

struct Embedding {  // token embedding table in its stored form
    void* d = nullptr;
    int type = 0;   // GGUF tensor type id: 0 F32, 1 F16, 41 Q1_0_g128, 42 TQ2_0_g128
    uint32_t vocab = 0, h = 0;
    size_t bytes = 0;
};
static std::unordered_map<uint64_t, Embedding> g_embeddings;

static std::unordered_map<uint64_t, std::unique_ptr<Model>> g_models;
static uint64_t g_next_model = 1;

static int dev_alloc(Model& m, void** p, size_t bytes) {
    hipError_t e = hipMalloc(p, bytes ? bytes : 16);
    if (e != hipSuccess)
        return fail(OXB_HIP_OUT_OF_MEMORY, "out of device memory: requested %zu bytes on device %d", bytes, g_rt.device);
    m.allocs.push_back(*p);
    return OXB_HIP_OK;
}

static void free_kv_cache(Model& m) {
    void* bufs[5] = {m.k_cache, m.v_cache, m.k_scale, m.v_scale, m.d_table};
    for (void* p : bufs)
        if (p) (void)hipFree(p);
    m.k_cache = m.v_cache = nullptr;
    m.k_scale = m.v_scale = nullptr;
    m.d_table = nullptr;
    m.n_pages = m.page_shift = m.table_stride = 0;
    m.free_pages.clear();
    m.seq_pages.clear();
    m.h_table.clear();
    m.table_dirty = false;
}

static void free_model(Model& m) {
    if (m.graph_exec) (void)hipGraphExecDestroy(m.graph_exec);
    m.graph_exec = nullptr;
    if (m.h_hidden) (void)hipHostFree(m.h_hidden);
    if (m.h_pos) (void)hipHostFree(m.h_pos);
    m.h_hidden = nullptr;
    m.h_pos = m.h_tokens = nullptr;
    for (void* p : m.allocs) (void)hipFree(p);
    m.allocs.clear();
    for (void* p : m.pf_allocs) (void)hipFree(p);
    m.pf_allocs.clear();
    m.pf_cap = 0;
    m.gws.release();
    m.gpack.release();
    m.gpack_o.release();
    free_kv_cache(m);
    m.tok_hist.release();
    m.tok_ids.release();
    m.sample_ws.release();
    m.rng.release();
}

void shutdown_models() {
    for (auto& kv : g_models) free_model(*kv.second);
    g_models.clear();
    for (auto& kv : g_embeddings) (void)hipFree(kv.second.d);
    g_embeddings.clear();
}

static const float* vec_ptr(uint64_t id, uint32_t n, const char* what, int* rc) {
    auto it = g_rt.vectors.find(id);
    if (it == g_rt.vectors.end()) {
        *rc = fail(OXB_HIP_WEIGHT_NOT_FOUND, "weight handle %llu (%s) not found", (unsigned long long)id, what);
        return nullptr;
    }
    if (it->second.n != n) {
        *rc = fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: %s holds %zu values, %u expected", what, it->second.n, n);
        return nullptr;
    }
    return it->second.d;
}

static const Weight* mat_ptr(uint64_t id, int fmt, uint32_t n_rows, uint32_t k, const char* what, int* rc) {
    Weight* w = find_weight(id);
    if (!w) {
        *rc = fail(OXB_HIP_WEIGHT_NOT_FOUND, "weight handle %llu (%s) not found", (unsigned long long)id, what);
        return nullptr;
    }
    if (w->d_raw && (int)w->L.fmt == fmt) {  // uploaded as bytes alone: the model's dimensions give it its shape
        if ((*rc = bind_shape(*w, n_rows, k))) return nullptr;
    }
    if ((int)w->L.fmt != fmt || w->L.n_rows != n_rows || w->L.k != k) {
        *rc = fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: %s is fmt %u %ux%u, model needs fmt %d %ux%u", what,
                   w->L.fmt, w->L.n_rows, w->L.k, fmt, n_rows, k);
        return nullptr;
    }
    return w;
}

#define OXB_TRY_HIP(expr, what)                               \
    do {                                                      \
        hipError_t e_ = (expr);                               \
        if (e_ != hipSuccess) return hip_fail(e_, what);      \
    } while (0)
#define OXB_TRY(expr)            \
    do {                         \
        int rc_ = (expr);        \
        if (rc_) return rc_;     \
    } while (0)

// nb activation vectors through one projection.  From gemv_packed_min_batch(K) vectors on they are quantised by a launch
// of their own into `pack` (sized by the caller: this runs inside stream captures) and up to eight share the pass.
static int proj(const Weight& w, const float* x, uint32_t ldx, uint32_t nb, float* y, uint32_t ldy, int pro, const float* norm_w,
                float eps, int epi, const float* residual, DevBuf* pack, bool prepacked = false) {
    const bool packed = pack && nb >= gemv_packed_min_batch(w.L.k);
    return gemv_launch(w, x, ldx, nb, y, ldy, pro, norm_w, eps, epi, residual, packed ? pack : nullptr, packed && prepacked);
}

// gate || up with SwiGLU behind it: one launch when K fits one GEMV launch (the epilogue needs whole row sums),
// else the plain product into gu and a separate SwiGLU.
static int gate_up_swiglu(const Weight& gate_up, const float* x, uint32_t ldx, uint32_t nb, const float* norm_w, float eps,
                          float* gu, float* act, uint32_t inter, DevBuf* pack) {
    if (gate_up.L.n_sb <= OXB_GEMV_MAX_SB)
        return proj(gate_up, x, ldx, nb, act, inter, OXB_GEMV_PRO_RMSNORM, norm_w, eps, OXB_GEMV_SWIGLU, nullptr, pack);
    OXB_TRY(proj(gate_up, x, ldx, nb, gu, 2 * inter, OXB_GEMV_PRO_RMSNORM, norm_w, eps, OXB_GEMV_STORE, nullptr, pack));
    OXB_TRY_HIP(oxb_launch_swiglu(gu, inter, nb, act, inter, g_rt.stream), "kernel launch failed: swiglu");
    return OXB_HIP_OK;
}

// The FFN half of a layer on nb <= OXB_GEMV_PACKED_MAX_BATCH vectors: O-proj + residual, RMSNorm -> gate || up -> SwiGLU,
// down + residual: three launches (RMSNorm rides in the gate || up kernel's prologue, SwiGLU in its epilogue), plus
// one pack launch in front of each where the vectors are quantised ahead.
static int encode_ffn(float* hidden, const float* attn_out, const float* ffn_norm, float eps, const Weight& o,
                      const Weight& gate_up, const Weight& down, float* gu, float* act, uint32_t h, uint32_t inter,
                      uint32_t attn_k, uint32_t nb, DevBuf* pack, DevBuf* o_prepacked = nullptr) {
    // (o_prepacked: the attention kernel has left attn_out quantised there)
    OXB_TRY(proj(o, attn_out, attn_k, nb, hidden, h, OXB_GEMV_PRO_F32, nullptr, 0.f, OXB_GEMV_RESIDUAL, hidden, o_prepacked ? o_prepacked : pack,
                 o_prepacked != nullptr));
    OXB_TRY(gate_up_swiglu(gate_up, hidden, h, nb, ffn_norm, eps, gu, act, inter, pack));
    OXB_TRY(proj(down, act, inter, nb, hidden, h, OXB_GEMV_PRO_F32, nullptr, 0.f, OXB_GEMV_RESIDUAL, hidden, pack));
    return OXB_HIP_OK;
}

// Decode batches from this size on run their projections through the prefill GEMM (fp16 activations on the
// matrix cores, one pass over the weights for the whole batch) instead of the fp32-exact GEMV, which streams
// the weights once per eight sequences.
#define OXB_DECODE_GEMM_MIN_BATCH (OXB_GEMV_PACKED_MAX_BATCH + 1)
// Sequences per pass of the GEMV-based step: all of them up to eight.
static uint32_t decode_chunk(uint32_t batch) { return batch <= OXB_GEMV_PACKED_MAX_BATCH ? batch : OXB_GEMV_PACKED_MAX_BATCH; }

// Looks every handle of the model up with the shape the model needs (which also binds a weight that was uploaded
// without one).  Run at creation and again whenever a weight or vector was replaced or freed since, before a decode
// step is captured: inside the capture nothing may allocate.
static int check_model_handles(Model& m) {
    const oxb_model_desc& d = m.d;
    const uint32_t qd = d.nq * d.hd, kd = d.nkv * d.hd, qkv_rows = qd + 2 * kd;
    int rc = OXB_HIP_OK;
    for (uint32_t L = 0; L < d.n_layers && !rc; L++) {
        const oxb_layer_ids& ly = m.layers[L];
        vec_ptr(ly.attn_norm, d.h, "attn_norm", &rc);
        if (!rc) vec_ptr(ly.q_norm, d.hd, "q_norm", &rc);
        if (!rc) vec_ptr(ly.k_norm, d.hd, "k_norm", &rc);
        if (!rc) vec_ptr(ly.ffn_norm, d.h, "ffn_norm", &rc);
        if (!rc) mat_ptr(ly.qkv, d.fmt, qkv_rows, d.h, "qkv", &rc);
        if (!rc) mat_ptr(ly.o, d.fmt, d.h, qd, "o", &rc);
        if (!rc) mat_ptr(ly.gate_up, d.fmt, 2 * d.inter, d.h, "gate_up", &rc);
        if (!rc) mat_ptr(ly.down, d.fmt, d.h, d.inter, "down", &rc);
    }
    if (!rc && d.final_norm) vec_ptr(d.final_norm, d.h, "final_norm", &rc);
    if (!rc && d.lm_head) mat_ptr(d.lm_head, d.fmt, d.vocab, d.h, "lm_head", &rc);
    if (!rc) m.checked_gen = g_rt.weights_gen;
    return rc;
}

// The GEMM-based decode step of a large batch is captured into a graph: its GEMM workspaces are sized here, before any
// capture, for every projection shape of the model (the LM head included when there is one).
static int size_gemm_workspaces(Model& m) {
    const oxb_model_desc& d = m.d;
    if (d.batch >= 2) {  // the pack buffer of the GEMV-based step (also what a larger batch's decode_hidden runs)
        uint32_t kmax = d.h > d.inter ? d.h : d.inter;
        if (d.nq * d.hd > kmax) kmax = d.nq * d.hd;
        int rc = m.gpack.ensure(oxb_gemv_pack_bytes(kmax, decode_chunk(d.batch)));
        if (rc) return rc;
        if (d.batch <= OXB_GEMV_PACKED_MAX_BATCH && !m.gpack_o.ptr) {
            const size_t n = oxb_gemv_pack_bytes(d.nq * d.hd, d.batch);
            if ((rc = m.gpack_o.ensure(n))) return rc;
            OXB_TRY_HIP(hipMemset(m.gpack_o.ptr, 0, n), "pack buffer clear");  // (at creation, like the cache's scales: never inside a capture)
        }
    }
    if (d.batch < OXB_DECODE_GEMM_MIN_BATCH) return OXB_HIP_OK;
    const uint32_t qd = d.nq * d.hd, kd = d.nkv * d.hd, qkv_rows = qd + 2 * kd;
    uint32_t kx = d.h > d.inter ? d.h : d.inter;
    if (qd > kx) kx = qd;
    size_t part_bytes = 0;
    const struct { uint64_t id; uint32_t n, k; } shapes[] = {{m.layers[0].qkv, qkv_rows, d.h}, {m.layers[0].o, d.h, qd},
                                                             {m.layers[0].gate_up, 2 * d.inter, d.h},
                                                             {m.layers[0].down, d.h, d.inter}, {d.lm_head, d.vocab, d.h}};
    for (const auto& sh : shapes) {
        const Weight* w = find_weight(sh.id);
        if (!w) continue;  // a model without an LM head
        OxbGemmParams gp;
        memset(&gp, 0, sizeof gp);
        gp.n_rows = sh.n;
        gp.n_tiles = w->L.n_tiles;
        gp.n_sb = w->L.n_sb;
        gp.M = d.batch;
        gp.ldy = sh.n;
        const size_t b = (size_t)oxb_gemm_ksplit(gp, g_rt.n_cus) * d.batch * sh.n * sizeof(float);
        if (oxb_gemm_ksplit(gp, g_rt.n_cus) > 1 && b > part_bytes) part_bytes = b;
    }
    int rc;
    if ((rc = m.gws.xh.ensure(oxb_xh_bytes(kx, d.batch))) || (rc = m.gws.xsh.ensure(((size_t)d.batch + 16) * 4)) ||
        (rc = m.gws.rowmul.ensure(((size_t)d.batch + 16) * 4)) || (part_bytes && (rc = m.gws.part.ensure(part_bytes))))
        return rc;
    return OXB_HIP_OK;
}

static OxbKvLayout kv_layout(const Model& m) {
    OxbKvLayout L;
    L.page_table = m.n_pages ? m.d_table : nullptr;
    L.page_shift = m.page_shift;
    L.table_stride = m.table_stride;
    L.n_pages = m.n_pages;
    L.n_layers = m.d.n_layers;
    L.nkv = m.d.nkv;
    L.row_stride = m.row_stride;
    return L;
}

// Paged cache: make sure sequence `seq` owns pages for positions 0 .. n_tokens - 1 (PagedKvCache::ensure_capacity,
// crates/oxibonsai-model/src/paged_kv_cache.rs:394-433: pages are taken from the free list one by one; when the pool
// runs dry the pages taken so far stay with the sequence).  A contiguous cache needs nothing.
static int kv_reserve(Model& m, uint32_t seq, uint64_t n_tokens) {
    if (!m.k_cache) return fail(OXB_HIP_OUT_OF_MEMORY, "out of device memory: the model has no KV cache (its last reallocation failed)");
    if (!m.n_pages) return OXB_HIP_OK;
    const size_t need = (size_t)((n_tokens + (1u << m.page_shift) - 1) >> m.page_shift);
    std::vector<uint32_t>& pg = m.seq_pages[seq];
    while (pg.size() < need) {
        if (m.free_pages.empty())
            return fail(OXB_HIP_OUT_OF_MEMORY, "out of memory: no free KV blocks (sequence %u needs %zu pages of %u positions, it holds %zu, pool of %u)",
                        seq, need, 1u << m.page_shift, pg.size(), m.n_pages);
        const uint32_t page = m.free_pages.back();
        m.free_pages.pop_back();
        m.h_table[(size_t)seq * m.table_stride + pg.size()] = page;
        pg.push_back(page);
        m.table_dirty = true;
    }
    return OXB_HIP_OK;
}

static void kv_release(Model& m, uint32_t seq) {  // PagedKvCache::drop_sequence (:362-375): pages go back to the pool
    if (!m.n_pages) return;
    std::vector<uint32_t>& pg = m.seq_pages[seq];
    for (size_t i = pg.size(); i-- > 0;) m.free_pages.push_back(pg[i]);
    pg.clear();
}

// The device copy of the page tables follows the host's before the next launch reads it (never inside a capture).
static int kv_sync_table(Model& m) {
    if (!m.n_pages || !m.table_dirty) return OXB_HIP_OK;
    OXB_TRY_HIP(hipMemcpyAsync(m.d_table, m.h_table.data(), m.h_table.size() * 4, hipMemcpyHostToDevice, g_rt.stream), "page table upload");
    OXB_TRY_HIP(hipStreamSynchronize(g_rt.stream), "page table upload");
    m.table_dirty = false;
    return OXB_HIP_OK;
}

// QK-norm + RoPE + KV store + split-KV attention of one layer for the whole decode batch, one launch; leaves the
// slot results in m.attn_part and the parameters the merge needs in *ap.
// One launch: QK-norm, RoPE, the store of the new rows, attention over the cache and the merge of the KV slots into
// m.attn_out (with a single slot per sequence the kernel writes its output directly).
static int encode_decode_attention(Model& m, uint32_t L, const float* q_norm, const float* k_norm, const Weight* pack_for = nullptr) {
    const oxb_model_desc& d = m.d;
    OxbAttnParams ap;
    ap.qkv = m.qkv;
    ap.qkv_stride = (d.nq + 2 * d.nkv) * d.hd;
    ap.q_norm = q_norm;
    ap.k_norm = k_norm;
    ap.cos_t = m.cos_t;
    ap.sin_t = m.sin_t;
    ap.eps = d.eps;
    ap.k_cache = m.k_cache;
    ap.v_cache = m.v_cache;
    ap.k_scale = m.k_scale;
    ap.v_scale = m.v_scale;
    ap.kv_mode = m.kv_mode;
    ap.kv = kv_layout(m);
    ap.window = m.window;
    ap.sinks = m.sinks;
    ap.part = m.attn_part;
    ap.out_single = m.n_splits == 1 ? m.attn_out : nullptr;
    ap.out_merged = m.attn_out;
    ap.done = m.attn_done;
    ap.pos = m.pos;
    ap.nq = d.nq;
    ap.nkv = d.nkv;
    ap.hd = d.hd;
    ap.max_seq = d.max_seq;
    ap.n_layers = d.n_layers;
    ap.layer = L;
    ap.chunk = m.chunk;
    ap.n_splits = m.n_splits;
    ap.scale = 1.0f / sqrtf((float)d.hd);
    ap.pack_out = pack_for ? (uint32_t*)m.gpack_o.ptr : nullptr;  // the O projection's operands, written by the merging workgroups
    ap.pack_fmt = pack_for ? (uint32_t)pack_for->L.fmt : 0;
    ap.pack_n_sb = pack_for ? pack_for->L.n_sb : 0;
    ap.pack_nvg = (d.batch + 3) / 4;
    OXB_TRY_HIP(oxb_launch_attn_decode(ap, d.batch, g_rt.stream), "kernel launch failed: attention");
    return OXB_HIP_OK;
}


static int encode_decode_step_gemm(Model& m) {
    const oxb_model_desc& d = m.d;
    hipStream_t st = g_rt.stream;
    const uint32_t qd = d.nq * d.hd, kd = d.nkv * d.hd, qkv_rows = qd + 2 * kd, B = d.batch;
    int rc = OXB_HIP_OK;
    for (uint32_t L = 0; L < d.n_layers; L++) {
        const oxb_layer_ids& ly = m.layers[L];
        const float* attn_norm = vec_ptr(ly.attn_norm, d.h, "attn_norm", &rc);
        const float* q_norm = vec_ptr(ly.q_norm, d.hd, "q_norm", &rc);
        const float* k_norm = vec_ptr(ly.k_norm, d.hd, "k_norm", &rc);
        const float* ffn_norm = vec_ptr(ly.ffn_norm, d.h, "ffn_norm", &rc);
        const Weight* wqkv = mat_ptr(ly.qkv, d.fmt, qkv_rows, d.h, "qkv", &rc);
        const Weight* wo = mat_ptr(ly.o, d.fmt, d.h, qd, "o", &rc);
        const Weight* wgu = mat_ptr(ly.gate_up, d.fmt, 2 * d.inter, d.h, "gate_up", &rc);
        const Weight* wdn = mat_ptr(ly.down, d.fmt, d.h, d.inter, "down", &rc);
        if (rc) return rc;
        OXB_TRY(gemm_device(*wqkv, m.hidden, d.h, m.qkv, B, qkv_rows, OXB_GEMM_STORE, nullptr, OXB_PACK_RMSNORM, attn_norm, d.eps, &m.gws));
        OXB_TRY(encode_decode_attention(m, L, q_norm, k_norm));
        OXB_TRY(gemm_device(*wo, m.attn_out, qd, m.hidden, B, d.h, OXB_GEMM_RESIDUAL, m.hidden, OXB_PACK_IDENT, nullptr, 0.f, &m.gws));
        // SwiGLU in the epilogue of the gate || up product
        OXB_TRY(gemm_device(*wgu, m.hidden, d.h, m.gu, B, d.inter, OXB_GEMM_SWIGLU, nullptr, OXB_PACK_RMSNORM, ffn_norm, d.eps, &m.gws));
        OXB_TRY(gemm_device(*wdn, m.gu, d.inter, m.hidden, B, d.h, OXB_GEMM_RESIDUAL, m.hidden, OXB_PACK_IDENT, nullptr, 0.f, &m.gws));
    }
    const float* final_norm = vec_ptr(d.final_norm, d.h, "final_norm", &rc);
    const Weight* lm = mat_ptr(d.lm_head, d.fmt, d.vocab, d.h, "lm_head", &rc);
    if (rc) return rc;
    OXB_TRY(gemm_device(*lm, m.hidden, d.h, m.logits, B, d.vocab, OXB_GEMM_STORE, nullptr, OXB_PACK_RMSNORM, final_norm, d.eps, &m.gws));
    OXB_TRY_HIP(oxb_launch_argmax(m.logits, d.vocab, B, m.tokens, m.argmax_ws, st, m.h_tokens), "kernel launch failed: argmax");
    return OXB_HIP_OK;
}

// Every kernel of one decode step, for all sequences of the batch (no host synchronisation).
static int encode_decode_step(Model& m, bool with_lm_head) {
    if (m.d.batch >= OXB_DECODE_GEMM_MIN_BATCH && with_lm_head) return encode_decode_step_gemm(m);
    const oxb_model_desc& d = m.d;
    hipStream_t st = g_rt.stream;
    const uint32_t qd = d.nq * d.hd, kd = d.nkv * d.hd, qkv_rows = qd + 2 * kd;
    const uint32_t chunk = decode_chunk(d.batch);
    DevBuf* pack = m.gpack.ptr ? &m.gpack : nullptr;
    int rc = OXB_HIP_OK;
    for (uint32_t L = 0; L < d.n_layers; L++) {
        const oxb_layer_ids& ly = m.layers[L];
        const float* attn_norm = vec_ptr(ly.attn_norm, d.h, "attn_norm", &rc);
        const float* q_norm = vec_ptr(ly.q_norm, d.hd, "q_norm", &rc);
        const float* k_norm = vec_ptr(ly.k_norm, d.hd, "k_norm", &rc);
        const float* ffn_norm = vec_ptr(ly.ffn_norm, d.h, "ffn_norm", &rc);
        const Weight* wqkv = mat_ptr(ly.qkv, d.fmt, qkv_rows, d.h, "qkv", &rc);
        const Weight* wo = mat_ptr(ly.o, d.fmt, d.h, qd, "o", &rc);
        const Weight* wgu = mat_ptr(ly.gate_up, d.fmt, 2 * d.inter, d.h, "gate_up", &rc);
        const Weight* wdn = mat_ptr(ly.down, d.fmt, d.h, d.inter, "down", &rc);
        if (rc) return rc;
        // attention input: RMSNorm -> QKV in one launch per pass of `chunk` sequences
        for (uint32_t b0 = 0; b0 < d.batch; b0 += chunk) {
            const uint32_t nb = (d.batch - b0) < chunk ? (d.batch - b0) : chunk;
            OXB_TRY(proj(*wqkv, m.hidden + (size_t)b0 * d.h, d.h, nb, m.qkv + (size_t)b0 * qkv_rows, qkv_rows,
                         OXB_GEMV_PRO_RMSNORM, attn_norm, d.eps, OXB_GEMV_STORE, nullptr, pack));
        }
        // Where the q heads of a kv head are one superblock of the O projection's input and the batch's vectors are
        // quantised ahead of that GEMV, the attention kernel's merging workgroups do the quantising: no pack launch.
        const bool fuse_o = m.gpack_o.ptr && d.batch <= OXB_GEMV_PACKED_MAX_BATCH && d.batch >= gemv_packed_min_batch(qd) &&
                            m.n_splits > 1 && (d.nq / d.nkv) * d.hd == 512u && m.gpack_o.cap >= oxb_gemv_pack_bytes(qd, d.batch);
        OXB_TRY(encode_decode_attention(m, L, q_norm, k_norm, fuse_o ? wo : nullptr));
        for (uint32_t b0 = 0; b0 < d.batch; b0 += chunk) {
            const uint32_t nb = (d.batch - b0) < chunk ? (d.batch - b0) : chunk;
            OXB_TRY(encode_ffn(m.hidden + (size_t)b0 * d.h, m.attn_out + (size_t)b0 * qd, ffn_norm, d.eps, *wo, *wgu, *wdn,
                               m.gu + (size_t)b0 * 2 * d.inter, m.act + (size_t)b0 * d.inter, d.h, d.inter, qd, nb, pack,
                               fuse_o ? &m.gpack_o : nullptr));
        }
    }
    if (with_lm_head) {
        const float* final_norm = vec_ptr(d.final_norm, d.h, "final_norm", &rc);
        const Weight* lm = mat_ptr(d.lm_head, d.fmt, d.vocab, d.h, "lm_head", &rc);
        if (rc) return rc;
        for (uint32_t b0 = 0; b0 < d.batch; b0 += chunk) {
            const uint32_t nb = (d.batch - b0) < chunk ? (d.batch - b0) : chunk;
            OXB_TRY(proj(*lm, m.hidden + (size_t)b0 * d.h, d.h, nb, m.logits + (size_t)b0 * d.vocab, d.vocab,
                         OXB_GEMV_PRO_RMSNORM, final_norm, d.eps, OXB_GEMV_STORE, nullptr, pack));
        }
        OXB_TRY_HIP(oxb_launch_argmax(m.logits, d.vocab, d.batch, m.tokens, m.argmax_ws, st, m.h_tokens), "kernel launch failed: argmax");
    }
    return OXB_HIP_OK;
}

// Prefill buffers for `rows` token rows.
static int ensure_prefill_buffers(Model& m, uint32_t rows) {
    if (rows <= m.pf_cap) return OXB_HIP_OK;
    (void)hipStreamSynchronize(g_rt.stream);
    for (void* p : m.pf_allocs) (void)hipFree(p);
    m.pf_allocs.clear();
    m.pf_cap = 0;
    const oxb_model_desc& d = m.d;
    const size_t R = (rows + 127u) / 128u * 128u, qd = (size_t)d.nq * d.hd, qkv_rows = qd + 2 * (size_t)d.nkv * d.hd;
    struct { float** p; size_t n; } bufs[] = {{&m.pf_hidden, R * d.h}, {&m.pf_qkv, R * qkv_rows},
                                             {&m.pf_attn, R * qd},    {&m.pf_gu, R * d.inter}};
    for (auto& b : bufs) {
        if (hipMalloc((void**)b.p, b.n * sizeof(float)) != hipSuccess) {
            for (void* p : m.pf_allocs) (void)hipFree(p);
            m.pf_allocs.clear();
            return fail(OXB_HIP_OUT_OF_MEMORY, "out of device memory: requested %zu bytes on device %d", b.n * sizeof(float), g_rt.device);
        }
        m.pf_allocs.push_back(*b.p);
    }
    m.pf_cap = (uint32_t)R;
    return OXB_HIP_OK;
}

// All layers for M token rows of sequence `seq` at positions pos_start .. pos_start + M - 1: batched
// projections on the matrix cores (RMSNorm and SwiGLU fused into the fp16 packer of the GEMM that consumes them), one causal attention launch per layer, KV written to the cache; then the
// LM head and the greedy token for the last row.
static int encode_prefill(Model& m, uint32_t seq, uint32_t M, uint32_t pos_start) {
    const oxb_model_desc& d = m.d;
    hipStream_t st = g_rt.stream;
    const uint32_t qd = d.nq * d.hd, kd = d.nkv * d.hd, qkv_rows = qd + 2 * kd;
    int rc = OXB_HIP_OK;
    for (uint32_t L = 0; L < d.n_layers; L++) {
        const oxb_layer_ids& ly = m.layers[L];
        const float* attn_norm = vec_ptr(ly.attn_norm, d.h, "attn_norm", &rc);
        const float* q_norm = vec_ptr(ly.q_norm, d.hd, "q_norm", &rc);
        const float* k_norm = vec_ptr(ly.k_norm, d.hd, "k_norm", &rc);
        const float* ffn_norm = vec_ptr(ly.ffn_norm, d.h, "ffn_norm", &rc);
        const Weight* wqkv = mat_ptr(ly.qkv, d.fmt, qkv_rows, d.h, "qkv", &rc);
        const Weight* wo = mat_ptr(ly.o, d.fmt, d.h, qd, "o", &rc);
        const Weight* wgu = mat_ptr(ly.gate_up, d.fmt, 2 * d.inter, d.h, "gate_up", &rc);
        const Weight* wdn = mat_ptr(ly.down, d.fmt, d.h, d.inter, "down", &rc);
        if (rc) return rc;
        OXB_TRY(gemm_device(*wqkv, m.pf_hidden, d.h, m.pf_qkv, M, qkv_rows, OXB_GEMM_STORE, nullptr, OXB_PACK_RMSNORM, attn_norm, d.eps));
        OxbQkParams qp;
        qp.qkv = m.pf_qkv;
        qp.qkv_stride = qkv_rows;
        qp.q_norm = q_norm;
        qp.k_norm = k_norm;
        qp.cos_t = m.cos_t;
        qp.sin_t = m.sin_t;
        qp.pos = nullptr;
        qp.pos_base = pos_start;
        qp.seq = seq;
        qp.q_rope = nullptr;  // the attention kernel norms and rotates Q itself
        qp.k_cache = m.k_cache;
        qp.v_cache = m.v_cache;
        qp.k_scale = m.k_scale;
        qp.v_scale = m.v_scale;
        qp.kv_mode = m.kv_mode;
        qp.kv = kv_layout(m);
        qp.nq = d.nq;
        qp.nkv = d.nkv;
        qp.hd = d.hd;
        qp.max_seq = d.max_seq;
        qp.n_layers = d.n_layers;
        qp.layer = L;
        qp.eps = d.eps;
        OXB_TRY_HIP(oxb_launch_qk_norm_rope_store(qp, M, st), "kernel launch failed: qk_norm_rope_store");
        OxbPrefillAttnParams ap;
        ap.qkv = m.pf_qkv;
        ap.qkv_stride = qkv_rows;
        ap.q_norm = q_norm;
        ap.cos_t = m.cos_t;
        ap.sin_t = m.sin_t;
        ap.eps = d.eps;
        ap.k_cache = m.k_cache;
        ap.v_cache = m.v_cache;
        ap.k_scale = m.k_scale;
        ap.v_scale = m.v_scale;
        ap.kv_mode = m.kv_mode;
        ap.kv = kv_layout(m);
        ap.seq = seq;
        ap.layer = L;
        ap.window = m.window;
        ap.sinks = m.sinks;
        ap.out = m.pf_attn;
        ap.M = M;
        ap.pos_start = pos_start;
        ap.nq = d.nq;
        ap.nkv = d.nkv;
        ap.hd = d.hd;
        ap.max_seq = d.max_seq;
        ap.scale = 1.0f / sqrtf((float)d.hd);
        OXB_TRY_HIP(oxb_launch_attn_prefill(ap, st), "kernel launch failed: attn_prefill");
        OXB_TRY(gemm_device(*wo, m.pf_attn, qd, m.pf_hidden, M, d.h, OXB_GEMM_RESIDUAL, m.pf_hidden, OXB_PACK_IDENT, nullptr, 0.f));
        // SwiGLU in the epilogue of the gate || up product: the activation [M][inter] is all that is written
        OXB_TRY(gemm_device(*wgu, m.pf_hidden, d.h, m.pf_gu, M, d.inter, OXB_GEMM_SWIGLU, nullptr, OXB_PACK_RMSNORM, ffn_norm, d.eps));
        OXB_TRY(gemm_device(*wdn, m.pf_gu, d.inter, m.pf_hidden, M, d.h, OXB_GEMM_RESIDUAL, m.pf_hidden, OXB_PACK_IDENT, nullptr, 0.f));
    }
    if (!d.lm_head) return OXB_HIP_OK;  // the caller asked for the cache rows only
    // last token: final norm, LM head, greedy token (fp32-exact products, as in a decode step)
    const float* final_norm = vec_ptr(d.final_norm, d.h, "final_norm", &rc);
    const Weight* lm = mat_ptr(d.lm_head, d.fmt, d.vocab, d.h, "lm_head", &rc);
    if (rc) return rc;
    float* last = m.hidden + (size_t)seq * d.h;
    OXB_TRY_HIP(hipMemcpyAsync(last, m.pf_hidden + (size_t)(M - 1) * d.h, (size_t)d.h * 4, hipMemcpyDeviceToDevice, st), "last row copy");
    OXB_TRY(gemv_launch(*lm, last, d.h, 1, m.logits + (size_t)seq * d.vocab, d.vocab, OXB_GEMV_PRO_RMSNORM, final_norm, d.eps,
                        OXB_GEMV_STORE, nullptr));
    OXB_TRY_HIP(oxb_launch_argmax(m.logits + (size_t)seq * d.vocab, d.vocab, 1, m.tokens + seq, m.argmax_ws, st), "kernel launch failed: argmax");
    return OXB_HIP_OK;
}

static Model* find_model(uint64_t id) {
    auto it = g_models.find(id);
    return it == g_models.end() ? nullptr : it->second.get();
}

}  // namespace oxb

using namespace oxb;

extern "C" {

int oxb_hip_upload_f32(uint64_t* id, const float* w, size_t n) {
    OXB_API_BEGIN
    std::lock_guard<std::recursive_mutex> lk(g_mu);
    if (!id || !w || n == 0) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: null pointer or empty vector");
    OXB_TRY(ensure_init());
    Vector v;
    v.n = n;
    for (size_t i = 0; i < n; i++) {
        const float a = fabsf(w[i]);
        if (a > v.absmax || a != a) v.absmax = a;  // a NaN sticks
    }
    if (hipMalloc((void**)&v.d, n * sizeof(float)) != hipSuccess)
        return fail(OXB_HIP_OUT_OF_MEMORY, "out of device memory: requested %zu bytes on device %d", n * sizeof(float), g_rt.device);
    hipError_t e = hipMemcpy(v.d, w, n * sizeof(float), hipMemcpyHostToDevice);
    if (e != hipSuccess) {
        (void)hipFree(v.d);
        return hip_fail(e, "vector upload");
    }
    if (*id == 0) *id = g_rt.next_id++;
    auto it = g_rt.vectors.find(*id);
    if (it != g_rt.vectors.end()) {
        (void)hipStreamSynchronize(g_rt.stream);
        (void)hipFree(it->second.d);
        g_rt.weights_gen++;
    }
    g_rt.vectors[*id] = v;
    return OXB_HIP_OK;
    OXB_API_END
}

int oxb_hip_free_f32(uint64_t id) {
    OXB_API_BEGIN
    std::lock_guard<std::recursive_mutex> lk(g_mu);
    auto it = g_rt.vectors.find(id);
    if (it == g_rt.vectors.end()) return fail(OXB_HIP_WEIGHT_NOT_FOUND, "weight handle %llu not found", (unsigned long long)id);
    if (g_rt.ready) (void)hipStreamSynchronize(g_rt.stream);
    (void)hipFree(it->second.d);
    g_rt.vectors.erase(it);
    g_rt.weights_gen++;
    return OXB_HIP_OK;
    OXB_API_END
}

// Slots of the split-KV attention: about one workgroup (slot x kv head x sequence) per CU for the fp16 cache, two for a
// quantised one (widening the codes adds arithmetic that a second resident workgroup hides), no more: every slot pays
// the Q arithmetic and a merge, and walks its chunks with a prefetch.  Measured, 8B shape: four per CU are slower
// everywhere (batch 8 at context 2048 by 12 %, batch 16 by 7 %, one sequence at context 32 000 by 3 %); two per CU
// gain 4 % at batch 32 with the INT8 cache and lose 1-3 % with the fp16 cache.
static uint32_t attn_slots(const Model& m, uint32_t kv_mode) {
    const oxb_model_desc& d = m.d;
    uint32_t n = (d.max_seq + m.chunk - 1) / m.chunk;
    const uint32_t per_cu = kv_mode == OXB_KV_F16 ? 1u : 2u;
    const uint32_t want = (per_cu * g_rt.n_cus + d.nkv * d.batch - 1) / (d.nkv * d.batch);
    if (n > want) n = want;
    if (const char* e = getenv("OXB_HIP_ATTN_SLOTS")) {  // measurement aid: a fixed slot count
        const long v = strtol(e, nullptr, 10);
        if (v > 0) n = (uint32_t)v < n ? (uint32_t)v : n;
    }
    if (n > OXB_ATTN_MAX_SPLITS) n = OXB_ATTN_MAX_SPLITS;
    return n;
}

// (Re)allocates the KV cache in the given storage form, contiguous (n_pages 0) or as a pool of n_pages pages of
// page_size positions.  Row scales start at 0 so that a row never written reads as zeros.  A contiguous head holds a
// whole number of attention chunks of rows, which keeps the kernels' 16-byte scale loads aligned and inside it.
static int alloc_kv_cache(Model& m, uint32_t kv_mode, uint32_t page_size, uint32_t n_pages) {
    const oxb_model_desc& d = m.d;
    free_kv_cache(m);
    m.row_stride = (d.max_seq + OXB_ATTN_CHUNK_POSITIONS - 1) / OXB_ATTN_CHUNK_POSITIONS * OXB_ATTN_CHUNK_POSITIONS;
    const size_t rows = n_pages ? (size_t)n_pages * d.n_layers * d.nkv * page_size : (size_t)d.batch * d.n_layers * d.nkv * m.row_stride;
    const size_t bytes = rows * d.hd * (kv_mode == OXB_KV_F16 ? 2 : 1);
    auto grab = [&](void** p, size_t n) -> int {
        if (hipMalloc(p, n ? n : 16) == hipSuccess) return OXB_HIP_OK;
        *p = nullptr;
        return fail(OXB_HIP_OUT_OF_MEMORY, "out of device memory: requested %zu bytes of KV cache on device %d", n, g_rt.device);
    };
    OXB_TRY(grab(&m.k_cache, bytes));
    OXB_TRY(grab(&m.v_cache, bytes));
    if (kv_mode != OXB_KV_F16) {
        const size_t sb = rows * sizeof(float);
        OXB_TRY(grab((void**)&m.k_scale, sb));
        OXB_TRY(grab((void**)&m.v_scale, sb));
        OXB_TRY_HIP(hipMemset(m.k_scale, 0, sb), "scale clear");
        OXB_TRY_HIP(hipMemset(m.v_scale, 0, sb), "scale clear");
    }
    if (n_pages) {
        uint32_t shift = 0;
        while ((1u << shift) < page_size) shift++;
        m.page_shift = shift;
        m.n_pages = n_pages;
        m.table_stride = m.row_stride / page_size;   // whole attention chunks: the kernels look up every block of a chunk
        m.h_table.assign((size_t)d.batch * m.table_stride, 0u);   // entries of unreserved blocks name page 0: never read
        m.seq_pages.assign(d.batch, {});
        m.free_pages.resize(n_pages);
        for (uint32_t i = 0; i < n_pages; i++) m.free_pages[i] = n_pages - 1 - i;   // page 0 is handed out first
        OXB_TRY(grab((void**)&m.d_table, m.h_table.size() * 4));
        OXB_TRY_HIP(hipMemset(m.d_table, 0, m.h_table.size() * 4), "page table clear");
    }
    m.kv_mode = kv_mode;
    return OXB_HIP_OK;
}

int oxb_hip_model_create(const oxb_model_desc* desc, uint64_t* model) {
    OXB_API_BEGIN
    std::lock_guard<std::recursive_mutex> lk(g_mu);
    if (!desc || !model || !desc->layers) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: null pointer");
    OXB_TRY(ensure_init());
    const oxb_model_desc& d = *desc;
    if (d.fmt != OXB_FMT_Q1 && d.fmt != OXB_FMT_TQ2) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: unknown format %d", d.fmt);
    if (!d.n_layers || !d.h || !d.inter || !d.nq || !d.nkv || !d.max_seq || !d.batch || (d.lm_head && !d.vocab))
        return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: a model dimension is 0");
    if (d.lm_head && !d.final_norm)
        return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: a model with an LM head needs the final norm vector");
    if (d.hd != 32 && d.hd != 64 && d.hd != 128 && d.hd != 256)
        return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: head_dim %u (supported: 32, 64, 128, 256)", d.hd);
    if (d.nq % d.nkv != 0 || d.nq / d.nkv > 16)
        return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: %u query heads per %u kv heads (need a whole ratio <= 16)", d.nq, d.nkv);
    if (d.h % 128 || d.inter % 128 || (d.nq * d.hd) % 128)
        return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: hidden, intermediate and nq*hd must be multiples of 128");
    if (((size_t)d.nq * d.hd + (size_t)d.nq * 65) * sizeof(float) > 60 * 1024)
        return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: nq*hd = %u exceeds what the attention merge holds in LDS", d.nq * d.hd);
    auto mp = std::make_unique<Model>();
    Model& m = *mp;
    m.d = d;
    m.layers.assign(d.layers, d.layers + d.n_layers);
    m.d.layers = nullptr;
    const uint32_t qd = d.nq * d.hd, kd = d.nkv * d.hd, qkv_rows = qd + 2 * kd;
    // check every handle now, so that a decode step cannot fail half way
    int rc = check_model_handles(m);
    if (rc) return rc;

    m.chunk = OXB_ATTN_CHUNK_POSITIONS;
    m.n_splits = attn_slots(m, OXB_KV_F16);
    const uint32_t max_slots = attn_slots(m, OXB_KV_I8);  // what any cache type may ask for: sizes the slot results
    const size_t B = d.batch;
    if ((rc = dev_alloc(m, (void**)&m.hidden, B * d.h * 4)) || (rc = dev_alloc(m, (void**)&m.qkv, B * qkv_rows * 4)) ||
        (rc = dev_alloc(m, (void**)&m.attn_part, B * d.nq * max_slots * (d.hd + OXB_ATTN_PART_PAD) * 4)) ||
        (rc = dev_alloc(m, (void**)&m.attn_out, B * qd * 4)) || (rc = dev_alloc(m, (void**)&m.gu, B * 2 * d.inter * 4)) ||
        (rc = dev_alloc(m, (void**)&m.act, B * d.inter * 4)) ||
        (rc = dev_alloc(m, (void**)&m.logits, B * (d.lm_head ? d.vocab : 1) * 4)) || (rc = dev_alloc(m, (void**)&m.tokens, B * 4)) ||
        (rc = dev_alloc(m, (void**)&m.pos, B * 4)) || (rc = dev_alloc(m, (void**)&m.attn_done, B * d.nkv * 4)) || (rc = dev_alloc(m, &m.argmax_ws, B * OXB_ARGMAX_MAX_PARTS * 8)) || (rc = alloc_kv_cache(m, OXB_KV_F16, 0, 0)) ||
        (rc = dev_alloc(m, (void**)&m.cos_t, (size_t)d.max_seq * (d.hd / 2) * 4)) ||
        (rc = dev_alloc(m, (void**)&m.sin_t, (size_t)d.max_seq * (d.hd / 2) * 4))) {
        free_model(m);
        return rc;
    }
    {
        hipError_t e = hipHostMalloc((void**)&m.h_hidden, B * d.h * 4, hipHostMallocCoherent);
        if (e == hipSuccess) e = hipHostMalloc((void**)&m.h_pos, B * 2 * 4, hipHostMallocCoherent);
        if (e != hipSuccess) {
            free_model(m);
            return fail(OXB_HIP_OUT_OF_MEMORY, "out of host memory: pinned staging of %zu bytes", B * d.h * 4);
        }
        m.h_tokens = m.h_pos + B;
        e = hipMemset(m.attn_done, 0, B * d.nkv * 4);
        if (e != hipSuccess) {
            free_model(m);
            return hip_fail(e, "counter clear");
        }
    }
    // RoPE table, computed as RopeTable::new does (crates/oxibonsai-model/src/layers/rope.rs:27-48): all in f32.
    {
        const size_t half = d.hd / 2;
        std::vector<float> c((size_t)d.max_seq * half), s((size_t)d.max_seq * half);
        for (size_t pos = 0; pos < d.max_seq; pos++)
            for (size_t i = 0; i < half; i++) {
                const float freq = 1.0f / powf(d.rope_theta, 2.0f * (float)i / (float)d.hd);
                const float angle = (float)pos * freq;
                c[pos * half + i] = cosf(angle);
                s[pos * half + i] = sinf(angle);
            }
        hipError_t e = hipMemcpy(m.cos_t, c.data(), c.size() * 4, hipMemcpyHostToDevice);
        if (e == hipSuccess) e = hipMemcpy(m.sin_t, s.data(), s.size() * 4, hipMemcpyHostToDevice);
        if (e != hipSuccess) {
            free_model(m);
            return hip_fail(e, "rope table upload");
        }
    }
    if ((rc = size_gemm_workspaces(m))) {
        free_model(m);
        return rc;
    }
    m.logits_cap = B * (d.lm_head ? d.vocab : 1);
    const char* no_graph = getenv("OXB_HIP_DISABLE_GRAPH");
    m.graph_failed = no_graph && no_graph[0] == '1';
    *model = g_next_model++;
    g_models[*model] = std::move(mp);
    return OXB_HIP_OK;
    OXB_API_END
}

int oxb_hip_model_destroy(uint64_t model) {
    OXB_API_BEGIN
    std::lock_guard<std::recursive_mutex> lk(g_mu);
    Model* m = find_model(model);
    if (!m) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: unknown model %llu", (unsigned long long)model);
    (void)hipStreamSynchronize(g_rt.stream);
    free_model(*m);
    const std::vector<uint64_t> mats = std::move(m->owned_mats), vecs = std::move(m->owned_vecs);
    g_models.erase(model);
    for (uint64_t id : mats) (void)oxb_hip_free_weight(id);
    for (uint64_t id : vecs) (void)oxb_hip_free_f32(id);
    return OXB_HIP_OK;
    OXB_API_END
}

int oxb_hip_model_set_attention(uint64_t model, const oxb_attention_options* opt) {
    OXB_API_BEGIN
    std::lock_guard<std::recursive_mutex> lk(g_mu);
    Model* m = find_model(model);
    if (!m) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: unknown model %llu", (unsigned long long)model);
    if (!opt) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: null pointer");
    if (opt->kv_dtype != OXB_KV_DTYPE_F16 && opt->kv_dtype != OXB_KV_DTYPE_I8 && opt->kv_dtype != OXB_KV_DTYPE_FP8_E4M3)
        return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: unknown KV cache type %d", opt->kv_dtype);
    OXB_TRY_HIP(hipStreamSynchronize(g_rt.stream), "synchronize");
    // the captured decode step holds the cache pointers and the options: it is captured again on the next step
    if (m->graph_exec) (void)hipGraphExecDestroy(m->graph_exec);
    m->graph_exec = nullptr;
    const uint32_t cur_page = m->n_pages ? 1u << m->page_shift : 0u;
    if ((opt->n_pages != 0) != (opt->page_size != 0))
        return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: page_size and n_pages must both be given (paged cache) or both be 0");
    if (opt->n_pages && opt->page_size != 16 && opt->page_size != 32 && opt->page_size != 64 && opt->page_size != 128)
        return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: page_size %u (supported: 16, 32, 64, 128 positions)", opt->page_size);
    if ((uint32_t)opt->kv_dtype != m->kv_mode || opt->n_pages != m->n_pages || opt->page_size != cur_page) {
        const int rc = alloc_kv_cache(*m, (uint32_t)opt->kv_dtype, opt->page_size, opt->n_pages);
        if (rc) {  // leave the model usable: back to the contiguous fp16 cache
            if (alloc_kv_cache(*m, OXB_KV_F16, 0, 0)) free_kv_cache(*m);
            return rc;
        }
    }
    m->n_splits = attn_slots(*m, m->kv_mode);
    m->window = opt->window_size;
    m->sinks = opt->sink_tokens;
    return OXB_HIP_OK;
    OXB_API_END
}

int oxb_hip_model_get_attention(uint64_t model, oxb_attention_options* opt) {
    OXB_API_BEGIN
    std::lock_guard<std::recursive_mutex> lk(g_mu);
    Model* m = find_model(model);
    if (!m) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: unknown model %llu", (unsigned long long)model);
    if (!opt) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: null pointer");
    opt->kv_dtype = (int32_t)m->kv_mode;
    opt->window_size = m->window;
    opt->sink_tokens = m->sinks;
    opt->page_size = m->n_pages ? 1u << m->page_shift : 0u;
    opt->n_pages = m->n_pages;
    return OXB_HIP_OK;
    OXB_API_END
}

int oxb_hip_model_read_kv(uint64_t model, uint32_t seq, uint32_t layer, uint32_t kv_head, uint32_t pos, uint32_t n_pos,
                          void* k_rows, void* v_rows, float* k_scales, float* v_scales) {
    OXB_API_BEGIN
    std::lock_guard<std::recursive_mutex> lk(g_mu);
    Model* m = find_model(model);
    if (!m) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: unknown model %llu", (unsigned long long)model);
    const oxb_model_desc& d = m->d;
    if (seq >= d.batch || layer >= d.n_layers || kv_head >= d.nkv || (uint64_t)pos + n_pos > d.max_seq)
        return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: cache rows (sequence %u, layer %u, head %u, positions %u..%llu) out of range",
                    seq, layer, kv_head, pos, (unsigned long long)pos + n_pos);
    if (!m->k_cache) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: the model has no KV cache");
    if (n_pos == 0) return OXB_HIP_OK;
    OXB_TRY_HIP(hipStreamSynchronize(g_rt.stream), "synchronize");
    const size_t esz = m->kv_mode == OXB_KV_F16 ? 2 : 1, row_bytes = (size_t)d.hd * esz;
    const uint32_t run_max = m->n_pages ? 1u << m->page_shift : n_pos;   // rows of one page are contiguous
    for (uint32_t i = 0; i < n_pos;) {
        const uint32_t p0 = pos + i;
        uint32_t run = m->n_pages ? run_max - (p0 & (run_max - 1)) : n_pos;
        if (run > n_pos - i) run = n_pos - i;
        size_t row;
        if (m->n_pages) {
            const std::vector<uint32_t>& pg = m->seq_pages[seq];
            const size_t blk = p0 >> m->page_shift;
            if (blk >= pg.size())
                return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: position %u of sequence %u lies outside its %zu pages", p0, seq, pg.size());
            row = ((((size_t)layer * d.nkv + kv_head) * m->n_pages + pg[blk]) << m->page_shift) + (p0 & (run_max - 1));
        } else {
            row = (((size_t)seq * d.n_layers + layer) * d.nkv + kv_head) * m->row_stride + p0;
        }
        if (k_rows) OXB_TRY_HIP(hipMemcpy((uint8_t*)k_rows + i * row_bytes, (const uint8_t*)m->k_cache + row * row_bytes, run * row_bytes, hipMemcpyDeviceToHost), "cache read");
        if (v_rows) OXB_TRY_HIP(hipMemcpy((uint8_t*)v_rows + i * row_bytes, (const uint8_t*)m->v_cache + row * row_bytes, run * row_bytes, hipMemcpyDeviceToHost), "cache read");
        if (m->kv_mode != OXB_KV_F16) {
            if (k_scales) OXB_TRY_HIP(hipMemcpy(k_scales + i, m->k_scale + row, (size_t)run * 4, hipMemcpyDeviceToHost), "scale read");
            if (v_scales) OXB_TRY_HIP(hipMemcpy(v_scales + i, m->v_scale + row, (size_t)run * 4, hipMemcpyDeviceToHost), "scale read");
        }
        i += run;
    }
    if (m->kv_mode == OXB_KV_F16)
        for (uint32_t i = 0; i < n_pos; i++) {
            if (k_scales) k_scales[i] = 1.0f;
            if (v_scales) v_scales[i] = 1.0f;
        }
    return OXB_HIP_OK;
    OXB_API_END
}

int oxb_hip_model_kv_reserve(uint64_t model, uint32_t seq, uint32_t n_tokens) {
    OXB_API_BEGIN
    std::lock_guard<std::recursive_mutex> lk(g_mu);
    Model* m = find_model(model);
    if (!m) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: unknown model %llu", (unsigned long long)model);
    if (seq >= m->d.batch) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: sequence %u of a batch of %u", seq, m->d.batch);
    if (n_tokens > m->d.max_seq)
        return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: %u positions exceed the context of %u", n_tokens, m->d.max_seq);
    return kv_reserve(*m, seq, n_tokens);
    OXB_API_END
}

int oxb_hip_model_kv_release(uint64_t model, uint32_t seq) {
    OXB_API_BEGIN
    std::lock_guard<std::recursive_mutex> lk(g_mu);
    Model* m = find_model(model);
    if (!m) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: unknown model %llu", (unsigned long long)model);
    if (seq >= m->d.batch) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: sequence %u of a batch of %u", seq, m->d.batch);
    OXB_TRY_HIP(hipStreamSynchronize(g_rt.stream), "synchronize");
    kv_release(*m, seq);
    return OXB_HIP_OK;
    OXB_API_END
}

int oxb_hip_model_kv_pool(uint64_t model, oxb_kv_pool_info* info) {
    OXB_API_BEGIN
    std::lock_guard<std::recursive_mutex> lk(g_mu);
    Model* m = find_model(model);
    if (!m) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: unknown model %llu", (unsigned long long)model);
    if (!info) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: null pointer");
    info->page_size = m->n_pages ? 1u << m->page_shift : 0u;
    info->total_pages = m->n_pages;
    info->free_pages = (uint32_t)m->free_pages.size();
    return OXB_HIP_OK;
    OXB_API_END
}

int oxb_hip_model_kv_capacity(uint64_t model, uint32_t seq, uint32_t* n_tokens) {
    OXB_API_BEGIN
    std::lock_guard<std::recursive_mutex> lk(g_mu);
    Model* m = find_model(model);
    if (!m) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: unknown model %llu", (unsigned long long)model);
    if (seq >= m->d.batch || !n_tokens) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: sequence %u of a batch of %u", seq, m->d.batch);
    *n_tokens = m->n_pages ? (uint32_t)(m->seq_pages[seq].size() << m->page_shift) : m->d.max_seq;
    return OXB_HIP_OK;
    OXB_API_END
}

int oxb_hip_kv_quantize_rows(int kv_dtype, const float* rows, uint32_t n_rows, uint32_t n, uint8_t* codes, float* scales) {
    OXB_API_BEGIN
    std::lock_guard<std::recursive_mutex> lk(g_mu);
    if (!rows || !codes || !scales) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: null buffer");
    if (kv_dtype != OXB_KV_DTYPE_I8 && kv_dtype != OXB_KV_DTYPE_FP8_E4M3)
        return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: KV cache type %d has no quantised rows", kv_dtype);
    if (n_rows == 0 || n == 0) return OXB_HIP_OK;
    OXB_TRY(ensure_init());
    DevBuf x, c, sc;
    int rc = OXB_HIP_OK;
    const size_t cnt = (size_t)n_rows * n;
    if (!(rc = x.ensure(cnt * 4)) && !(rc = c.ensure(cnt)) && !(rc = sc.ensure((size_t)n_rows * 4))) {
        hipError_t e = hipMemcpyAsync(x.ptr, rows, cnt * 4, hipMemcpyHostToDevice, g_rt.stream);
        if (e == hipSuccess) e = oxb_launch_kv_quantize_rows(kv_dtype, (const float*)x.ptr, n_rows, n, (uint8_t*)c.ptr, (float*)sc.ptr, g_rt.stream);
        if (e == hipSuccess) e = hipMemcpyAsync(codes, c.ptr, cnt, hipMemcpyDeviceToHost, g_rt.stream);
        if (e == hipSuccess) e = hipMemcpyAsync(scales, sc.ptr, (size_t)n_rows * 4, hipMemcpyDeviceToHost, g_rt.stream);
        if (e == hipSuccess) e = hipStreamSynchronize(g_rt.stream);
        if (e != hipSuccess) rc = hip_fail(e, "kv row quantisation");
    }
    x.release();
    c.release();
    sc.release();
    return rc;
    OXB_API_END
}

int oxb_hip_kv_dequantize_rows(int kv_dtype, const uint8_t* codes, const float* scales, uint32_t n_rows, uint32_t n, float* rows) {
    OXB_API_BEGIN
    std::lock_guard<std::recursive_mutex> lk(g_mu);
    if (!rows || !codes || !scales) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: null buffer");
    if (kv_dtype != OXB_KV_DTYPE_I8 && kv_dtype != OXB_KV_DTYPE_FP8_E4M3)
        return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: KV cache type %d has no quantised rows", kv_dtype);
    if (n & 3u) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: rows of %u values (a multiple of 4 is needed)", n);
    if (n_rows == 0 || n == 0) return OXB_HIP_OK;
    OXB_TRY(ensure_init());
    DevBuf x, c, sc;
    int rc = OXB_HIP_OK;
    const size_t cnt = (size_t)n_rows * n;
    if (!(rc = x.ensure(cnt * 4)) && !(rc = c.ensure(cnt)) && !(rc = sc.ensure((size_t)n_rows * 4))) {
        hipError_t e = hipMemcpyAsync(c.ptr, codes, cnt, hipMemcpyHostToDevice, g_rt.stream);
        if (e == hipSuccess) e = hipMemcpyAsync(sc.ptr, scales, (size_t)n_rows * 4, hipMemcpyHostToDevice, g_rt.stream);
        if (e == hipSuccess) e = oxb_launch_kv_dequantize_rows(kv_dtype, (const uint8_t*)c.ptr, (const float*)sc.ptr, n_rows, n, (float*)x.ptr, g_rt.stream);
        if (e == hipSuccess) e = hipMemcpyAsync(rows, x.ptr, cnt * 4, hipMemcpyDeviceToHost, g_rt.stream);
        if (e == hipSuccess) e = hipStreamSynchronize(g_rt.stream);
        if (e != hipSuccess) rc = hip_fail(e, "kv row dequantisation");
    }
    x.release();
    c.release();
    sc.release();
    return rc;
    OXB_API_END
}

int oxb_hip_model_reset(uint64_t model) {
    OXB_API_BEGIN
    std::lock_guard<std::recursive_mutex> lk(g_mu);
    Model* m = find_model(model);
    if (!m) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: unknown model %llu", (unsigned long long)model);
    // positions are supplied per call and attention reads only 0..pos, so nothing has to be cleared; a paged cache
    // takes the sequences' pages back
    (void)hipStreamSynchronize(g_rt.stream);
    for (uint32_t b = 0; b < m->d.batch; b++) kv_release(*m, b);
    return OXB_HIP_OK;
    OXB_API_END
}

static bool stream_is_capturing(hipStream_t st) {
    if (st == g_rt.own_stream) return false;
    hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(st, &cs) != hipSuccess) {
        (void)hipGetLastError();
        return true;  // unknown: launch plainly
    }
    return cs != hipStreamCaptureStatusNone;
}

// One decode step on m.hidden / m.pos (device): replayed from the captured graph, captured on first use, or launched
// kernel by kernel when capture is off or failed.
static int run_decode_step(Model& m) {
    hipStream_t st = g_rt.stream;
    if (!m.d.lm_head) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: the model has no LM head (oxb_hip_decode_hidden returns its normed hidden state)");
    if (m.checked_gen != g_rt.weights_gen) OXB_TRY(check_model_handles(m));
    if (m.graph_exec && m.graph_gen != g_rt.weights_gen) {
        // a weight or norm vector was freed or replaced since the capture: look every handle up again
        (void)hipGraphExecDestroy(m.graph_exec);
        m.graph_exec = nullptr;
    }
    if (m.graph_exec) {
        OXB_TRY_HIP(hipGraphLaunch(m.graph_exec, st), "graph launch");
    } else if (!m.graph_failed && !stream_is_capturing(st)) {
        // Capture the whole token once; on any capture problem fall back to plain launches for good.  The capture
        // records on the library's own stream (nothing runs there); the graph is replayed on the stream in use, so a
        // caller that set its own stream gets the replay too.  A caller's stream that is itself being captured takes
        // the plain launches into the caller's graph.
        hipGraph_t graph = nullptr;
        m.graph_gen = g_rt.weights_gen;
        g_rt.stream = g_rt.own_stream;
        hipError_t e = hipStreamBeginCapture(g_rt.own_stream, hipStreamCaptureModeThreadLocal);
        int rc = OXB_HIP_OK;
        if (e == hipSuccess) {
            rc = encode_decode_step(m, true);
            hipError_t e2 = hipStreamEndCapture(g_rt.own_stream, &graph);
            if (rc == OXB_HIP_OK && e2 == hipSuccess && graph) e = hipGraphInstantiate(&m.graph_exec, graph, nullptr, nullptr, 0);
            else e = e2 == hipSuccess ? hipErrorUnknown : e2;
            if (graph) (void)hipGraphDestroy(graph);
        }
        g_rt.stream = st;
        if (rc) return rc;
        if (e != hipSuccess || !m.graph_exec) {
            (void)hipGetLastError();
            m.graph_exec = nullptr;
            m.graph_failed = true;
            OXB_TRY(encode_decode_step(m, true));
        } else {
            OXB_TRY_HIP(hipGraphLaunch(m.graph_exec, st), "graph launch");
        }
    } else {
        OXB_TRY(encode_decode_step(m, true));
    }
    return OXB_HIP_OK;
}

int oxb_hip_decode(uint64_t model, const float* hidden, const uint32_t* pos, float* logits_or_null, uint32_t* token_out) {
    OXB_API_BEGIN
    std::lock_guard<std::recursive_mutex> lk(g_mu);
    Model* mp = find_model(model);
    if (!mp) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: unknown model %llu", (unsigned long long)model);
    Model& m = *mp;
    const oxb_model_desc& d = m.d;
    if (!hidden || !pos) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: null hidden or pos");
    for (uint32_t b = 0; b < d.batch; b++)
        if (pos[b] >= d.max_seq)
            return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: position %u exceeds the context of %u", pos[b], d.max_seq);
    for (uint32_t b = 0; b < d.batch; b++) OXB_TRY(kv_reserve(m, b, (uint64_t)pos[b] + 1));
    OXB_TRY(kv_sync_table(m));
    hipStream_t st = g_rt.stream;
    // (the previous call ended with a stream synchronisation, so the staging buffers are free)
    memcpy(m.h_hidden, hidden, (size_t)d.batch * d.h * 4);
    memcpy(m.h_pos, pos, (size_t)d.batch * 4);
    // one kernel reads the pinned rows and positions; the step's last kernel leaves the token ids in pinned memory too
    OXB_TRY_HIP(oxb_launch_stage_in(m.h_hidden, d.batch * d.h, m.h_pos, d.batch, m.hidden, m.pos, st), "kernel launch failed: stage_in");
    OXB_TRY(run_decode_step(m));
    if (logits_or_null)
        OXB_TRY_HIP(hipMemcpyAsync(logits_or_null, m.logits, (size_t)d.batch * d.vocab * 4, hipMemcpyDeviceToHost, st), "logits download");
    hipError_t e = hipStreamSynchronize(st);
    if (e != hipSuccess) return fail(OXB_HIP_SYNC_FAILED, "device synchronization failed: decode: %s", hipGetErrorString(e));
    if (token_out) memcpy(token_out, m.h_tokens, (size_t)d.batch * 4);
    return OXB_HIP_OK;
    OXB_API_END
}

int oxb_hip_model_set_lm_head(uint64_t model, uint64_t final_norm, uint64_t lm_head, uint32_t vocab) {
    OXB_API_BEGIN
    std::lock_guard<std::recursive_mutex> lk(g_mu);
    Model* mp = find_model(model);
    if (!mp) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: unknown model %llu", (unsigned long long)model);
    Model& m = *mp;
    if (lm_head && (!final_norm || !vocab))
        return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: an LM head needs the final norm vector and a vocabulary size");
    int rc = OXB_HIP_OK;
    if (final_norm) vec_ptr(final_norm, m.d.h, "final_norm", &rc);
    if (!rc && lm_head) mat_ptr(lm_head, m.d.fmt, vocab, m.d.h, "lm_head", &rc);
    if (rc) return rc;
    OXB_TRY_HIP(hipStreamSynchronize(g_rt.stream), "synchronize");
    if (m.graph_exec) {  // the captured step ends in the old LM head (or in none)
        (void)hipGraphExecDestroy(m.graph_exec);
        m.graph_exec = nullptr;
    }
    const size_t need = (size_t)m.d.batch * (lm_head ? vocab : 1);
    if (need > m.logits_cap) {
        float* p = nullptr;
        OXB_TRY(dev_alloc(m, (void**)&p, need * 4));  // the smaller buffer stays with the model until it is destroyed
        m.logits = p;
        m.logits_cap = need;
    }
    // The new head is committed only if everything that depends on it succeeds: on an error the model keeps the
    // head it had (its graph was dropped above and is captured again by the next step; workspaces only ever grow).
    const oxb_model_desc before = m.d;
    m.d.final_norm = final_norm;
    m.d.lm_head = lm_head;
    m.d.vocab = lm_head ? vocab : 0;
    rc = size_gemm_workspaces(m);
    if (!rc) rc = check_model_handles(m);
    if (rc) m.d = before;
    return rc;
    OXB_API_END
}

int oxb_hip_decode_hidden(uint64_t model, const float* hidden, const uint32_t* pos, float* normed_out) {
    OXB_API_BEGIN
    std::lock_guard<std::recursive_mutex> lk(g_mu);
    Model* mp = find_model(model);
    if (!mp) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: unknown model %llu", (unsigned long long)model);
    Model& m = *mp;
    const oxb_model_desc& d = m.d;
    if (!hidden || !pos || !normed_out) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: null hidden, pos or output");
    for (uint32_t b = 0; b < d.batch; b++)
        if (pos[b] >= d.max_seq)
            return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: position %u exceeds the context of %u", pos[b], d.max_seq);
    // the normed rows go through the gate || up buffer (free once the last layer is done): 2 * inter values per
    // sequence.  Checked, like every argument, before the step touches the cache.
    if ((size_t)2 * d.inter < d.h) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: hidden %u exceeds 2 x intermediate %u", d.h, d.inter);
    if (m.checked_gen != g_rt.weights_gen) OXB_TRY(check_model_handles(m));
    int rc = OXB_HIP_OK;
    const float* final_norm = d.final_norm ? vec_ptr(d.final_norm, d.h, "final_norm", &rc) : nullptr;
    if (rc) return rc;
    for (uint32_t b = 0; b < d.batch; b++) OXB_TRY(kv_reserve(m, b, (uint64_t)pos[b] + 1));
    OXB_TRY(kv_sync_table(m));
    hipStream_t st = g_rt.stream;
    OXB_TRY_HIP(hipMemcpyAsync(m.hidden, hidden, (size_t)d.batch * d.h * 4, hipMemcpyHostToDevice, st), "hidden upload");
    OXB_TRY_HIP(hipMemcpyAsync(m.pos, pos, (size_t)d.batch * 4, hipMemcpyHostToDevice, st), "position upload");
    OXB_TRY(encode_decode_step(m, false));
    float* dst = m.gu;
    OXB_TRY_HIP(oxb_launch_rmsnorm(m.hidden, final_norm, d.h, d.batch, d.eps, dst, st), "kernel launch failed: rmsnorm");
    for (uint32_t b = 0; b < d.batch; b++)
        OXB_TRY_HIP(hipMemcpyAsync(normed_out + (size_t)b * d.h, dst + (size_t)b * d.h, (size_t)d.h * 4, hipMemcpyDeviceToHost, st),
                    "hidden download");
    hipError_t e = hipStreamSynchronize(st);
    if (e != hipSuccess) return fail(OXB_HIP_SYNC_FAILED, "device synchronization failed: decode_hidden: %s", hipGetErrorString(e));
    return OXB_HIP_OK;
    OXB_API_END
}

int oxb_hip_model_set_rope_rows(uint64_t model, uint32_t pos_start, uint32_t n_pos, const float* cos_rows, const float* sin_rows) {
    OXB_API_BEGIN
    std::lock_guard<std::recursive_mutex> lk(g_mu);
    Model* mp = find_model(model);
    if (!mp) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: unknown model %llu", (unsigned long long)model);
    Model& m = *mp;
    if (!cos_rows || !sin_rows || n_pos == 0) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: null table or no positions");
    if ((uint64_t)pos_start + n_pos > m.d.max_seq)
        return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: positions %u..%llu exceed the context of %u", pos_start,
                    (unsigned long long)pos_start + n_pos - 1, m.d.max_seq);
    const size_t half = m.d.hd / 2;
    hipStream_t st = g_rt.stream;
    // ordered on the stream behind every step already issued; pageable host memory is staged before the call returns
    OXB_TRY_HIP(hipMemcpyAsync(m.cos_t + (size_t)pos_start * half, cos_rows, (size_t)n_pos * half * 4, hipMemcpyHostToDevice, st), "rope rows upload");
    OXB_TRY_HIP(hipMemcpyAsync(m.sin_t + (size_t)pos_start * half, sin_rows, (size_t)n_pos * half * 4, hipMemcpyHostToDevice, st), "rope rows upload");
    hipError_t e = hipStreamSynchronize(st);
    if (e != hipSuccess) return fail(OXB_HIP_SYNC_FAILED, "device synchronization failed: rope rows: %s", hipGetErrorString(e));
    return OXB_HIP_OK;
    OXB_API_END
}

int oxb_hip_prefill(uint64_t model, uint32_t seq, const float* hidden, uint32_t n_tokens, uint32_t pos_start,
                    float* logits_or_null, uint32_t* token_out_or_null) {
    OXB_API_BEGIN
    std::lock_guard<std::recursive_mutex> lk(g_mu);
    Model* mp = find_model(model);
    if (!mp) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: unknown model %llu", (unsigned long long)model);
    Model& m = *mp;
    const oxb_model_desc& d = m.d;
    if (!hidden || n_tokens == 0) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: null hidden or no tokens");
    if (!d.lm_head && (logits_or_null || token_out_or_null))
        return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: the model has no LM head: logits and token must be null");
    if (m.checked_gen != g_rt.weights_gen) OXB_TRY(check_model_handles(m));
    if (seq >= d.batch) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: sequence %u of a batch of %u", seq, d.batch);
    if ((uint64_t)pos_start + n_tokens > d.max_seq)
        return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: positions %u..%llu exceed the context of %u", pos_start,
                    (unsigned long long)pos_start + n_tokens - 1, d.max_seq);
    OXB_TRY(kv_reserve(m, seq, (uint64_t)pos_start + n_tokens));
    OXB_TRY(kv_sync_table(m));
    OXB_TRY(ensure_prefill_buffers(m, n_tokens));
    hipStream_t st = g_rt.stream;
    OXB_TRY_HIP(hipMemcpyAsync(m.pf_hidden, hidden, (size_t)n_tokens * d.h * 4, hipMemcpyHostToDevice, st), "hidden upload");
    OXB_TRY(encode_prefill(m, seq, n_tokens, pos_start));
    if (token_out_or_null) OXB_TRY_HIP(hipMemcpyAsync(token_out_or_null, m.tokens + seq, 4, hipMemcpyDeviceToHost, st), "token download");
    if (logits_or_null)
        OXB_TRY_HIP(hipMemcpyAsync(logits_or_null, m.logits + (size_t)seq * d.vocab, (size_t)d.vocab * 4, hipMemcpyDeviceToHost, st), "logits download");
    hipError_t e = hipStreamSynchronize(st);
    if (e != hipSuccess) return fail(OXB_HIP_SYNC_FAILED, "device synchronization failed: prefill: %s", hipGetErrorString(e));
    return OXB_HIP_OK;
    OXB_API_END
}

int oxb_hip_model_uses_graph(uint64_t model) {
    OXB_API_BEGIN
    std::lock_guard<std::recursive_mutex> lk(g_mu);
    Model* m = find_model(model);
    return m && m->graph_exec ? 1 : 0;
    OXB_API_END
}

int oxb_hip_attn_phase(int fmt, const float* hidden, const float* norm_w, float eps, uint64_t qkv_id, uint32_t q_rows,
                       uint32_t k_rows, uint32_t h, float* q, float* k, float* v) {
    OXB_API_BEGIN
    std::lock_guard<std::recursive_mutex> lk(g_mu);
    if (!hidden || !norm_w || !q || !k || !v) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: null buffer");
    if (h % 128 || q_rows == 0 || k_rows == 0) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: h must be a multiple of 128, row counts non-zero");
    const uint32_t rows = q_rows + 2 * k_rows;
    int rc = OXB_HIP_OK;
    const Weight* w = mat_ptr(qkv_id, fmt, rows, h, "qkv", &rc);
    if (rc) return rc;
    OXB_TRY(g_rt.ws_x.ensure((size_t)h * 2 * 4));
    OXB_TRY(g_rt.ws_y.ensure((size_t)rows * 4));
    float* d_hidden = (float*)g_rt.ws_x.ptr;
    float* d_norm = d_hidden + h;
    float* d_qkv = (float*)g_rt.ws_y.ptr;
    hipStream_t st = g_rt.stream;
    OXB_TRY_HIP(hipMemcpyAsync(d_hidden, hidden, (size_t)h * 4, hipMemcpyHostToDevice, st), "hidden upload");
    OXB_TRY_HIP(hipMemcpyAsync(d_norm, norm_w, (size_t)h * 4, hipMemcpyHostToDevice, st), "norm upload");
    OXB_TRY(gemv_launch(*w, d_hidden, h, 1, d_qkv, rows, OXB_GEMV_PRO_RMSNORM, d_norm, eps, OXB_GEMV_STORE, nullptr));
    OXB_TRY_HIP(hipMemcpyAsync(q, d_qkv, (size_t)q_rows * 4, hipMemcpyDeviceToHost, st), "q download");
    OXB_TRY_HIP(hipMemcpyAsync(k, d_qkv + q_rows, (size_t)k_rows * 4, hipMemcpyDeviceToHost, st), "k download");
    OXB_TRY_HIP(hipMemcpyAsync(v, d_qkv + q_rows + k_rows, (size_t)k_rows * 4, hipMemcpyDeviceToHost, st), "v download");
    hipError_t e = hipStreamSynchronize(st);
    if (e != hipSuccess) return fail(OXB_HIP_SYNC_FAILED, "device synchronization failed: attn_phase: %s", hipGetErrorString(e));
    return OXB_HIP_OK;
    OXB_API_END
}

int oxb_hip_ffn_phase(int fmt, float* hidden, const float* attn_out, const float* norm_w, float eps, uint64_t o_id,
                      uint64_t gate_up_id, uint64_t down_id, uint32_t h, uint32_t inter, uint32_t attn_k) {
    OXB_API_BEGIN
    std::lock_guard<std::recursive_mutex> lk(g_mu);
    if (!hidden || !attn_out || !norm_w) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: null buffer");
    if (h % 128 || inter % 128 || attn_k % 128) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: dimensions must be multiples of 128");
    int rc = OXB_HIP_OK;
    const Weight* wo = mat_ptr(o_id, fmt, h, attn_k, "attn_proj", &rc);
    const Weight* wgu = mat_ptr(gate_up_id, fmt, 2 * inter, h, "gate_up", &rc);
    const Weight* wdn = mat_ptr(down_id, fmt, h, inter, "down", &rc);
    if (rc) return rc;
    OXB_TRY(g_rt.ws_x.ensure(((size_t)h * 2 + attn_k) * 4));
    OXB_TRY(g_rt.ws_y.ensure((size_t)3 * inter * 4));
    float* d_hidden = (float*)g_rt.ws_x.ptr;
    float* d_norm = d_hidden + h;
    float* d_attn = d_norm + h;
    float* d_gu = (float*)g_rt.ws_y.ptr;
    float* d_act = d_gu + 2 * (size_t)inter;
    hipStream_t st = g_rt.stream;
    OXB_TRY_HIP(hipMemcpyAsync(d_hidden, hidden, (size_t)h * 4, hipMemcpyHostToDevice, st), "hidden upload");
    OXB_TRY_HIP(hipMemcpyAsync(d_norm, norm_w, (size_t)h * 4, hipMemcpyHostToDevice, st), "norm upload");
    OXB_TRY_HIP(hipMemcpyAsync(d_attn, attn_out, (size_t)attn_k * 4, hipMemcpyHostToDevice, st), "attn_out upload");
    OXB_TRY(encode_ffn(d_hidden, d_attn, d_norm, eps, *wo, *wgu, *wdn, d_gu, d_act, h, inter, attn_k, 1, nullptr));
    OXB_TRY_HIP(hipMemcpyAsync(hidden, d_hidden, (size_t)h * 4, hipMemcpyDeviceToHost, st), "hidden download");
    hipError_t e = hipStreamSynchronize(st);
    if (e != hipSuccess) return fail(OXB_HIP_SYNC_FAILED, "device synchronization failed: ffn_phase: %s", hipGetErrorString(e));
    return OXB_HIP_OK;
    OXB_API_END
}

// ---------------------------------------------------------------------------
// Token embedding tables, the on-device greedy loop, and the GGUF loader.
// ---------------------------------------------------------------------------
static Embedding* find_embedding(uint64_t id) {
    auto it = g_embeddings.find(id);
    return it == g_embeddings.end() ? nullptr : &it->second;
}

int oxb_hip_upload_embedding(uint64_t* id, const void* table, size_t n_bytes, int gguf_type, uint32_t vocab, uint32_t h) {
    OXB_API_BEGIN
    std::lock_guard<std::recursive_mutex> lk(g_mu);
    if (!id || !table) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: null id or table");
    if (gguf_type != GGUF_F32 && gguf_type != GGUF_F16 && gguf_type != GGUF_Q1_0_G128 && gguf_type != GGUF_TQ2_0_G128)
        return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: embedding tensor type %d (supported: 0 F32, 1 F16, 41, 42)", gguf_type);
    if (vocab == 0 || h == 0 || (gguf_type >= 41 && h % 128))
        return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: embedding of %u rows x %u values", vocab, h);
    const size_t need = (size_t)gguf_tensor_bytes((uint32_t)gguf_type, (uint64_t)vocab * h);
    if (n_bytes < need)
        return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: embedding buffer holds %zu bytes, %zu needed", n_bytes, need);
    OXB_TRY(ensure_init());
    Embedding e;
    e.type = gguf_type, e.vocab = vocab, e.h = h, e.bytes = need;
    if (hipMalloc(&e.d, need) != hipSuccess)
        return fail(OXB_HIP_OUT_OF_MEMORY, "out of device memory: requested %zu bytes on device %d", need, g_rt.device);
    hipError_t he = hipMemcpy(e.d, table, need, hipMemcpyHostToDevice);
    if (he != hipSuccess) {
        (void)hipFree(e.d);
        return hip_fail(he, "embedding upload");
    }
    if (*id == 0) *id = g_rt.next_id++;
    if (Embedding* old = find_embedding(*id)) (void)hipFree(old->d);
    g_embeddings[*id] = e;
    return OXB_HIP_OK;
    OXB_API_END
}

int oxb_hip_free_embedding(uint64_t id) {
    OXB_API_BEGIN
    std::lock_guard<std::recursive_mutex> lk(g_mu);
    Embedding* e = find_embedding(id);
    if (!e) return fail(OXB_HIP_WEIGHT_NOT_FOUND, "weight handle %llu (embedding) not found", (unsigned long long)id);
    (void)hipStreamSynchronize(g_rt.stream);
    (void)hipFree(e->d);
    g_embeddings.erase(id);
    return OXB_HIP_OK;
    OXB_API_END
}

static int check_ids(const Embedding& e, const uint32_t* ids, size_t n) {
    for (size_t i = 0; i < n; i++)
        if (ids[i] >= e.vocab)  // model/types/mod.rs:649-657
            return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: token_id %u out of range (vocab=%u)", ids[i], e.vocab);
    return OXB_HIP_OK;
}

int oxb_hip_embedding_rows(uint64_t embedding, const uint32_t* ids, uint32_t n, float* out) {
    OXB_API_BEGIN
    std::lock_guard<std::recursive_mutex> lk(g_mu);
    Embedding* e = find_embedding(embedding);
    if (!e) return fail(OXB_HIP_WEIGHT_NOT_FOUND, "weight handle %llu (embedding) not found", (unsigned long long)embedding);
    if (n == 0) return OXB_HIP_OK;
    if (!ids || !out) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: null ids or out");
    OXB_TRY(check_ids(*e, ids, n));
    OXB_TRY(g_rt.ws_x.ensure((size_t)n * 4));
    OXB_TRY(g_rt.ws_y.ensure((size_t)n * e->h * 4));
    hipStream_t st = g_rt.stream;
    OXB_TRY_HIP(hipMemcpyAsync(g_rt.ws_x.ptr, ids, (size_t)n * 4, hipMemcpyHostToDevice, st), "token id upload");
    OXB_TRY_HIP(oxb_launch_embedding_gather(e->d, e->type, e->vocab, e->h, (const uint32_t*)g_rt.ws_x.ptr, n, (float*)g_rt.ws_y.ptr, st),
                "kernel launch failed: embedding_gather");
    OXB_TRY_HIP(hipMemcpyAsync(out, g_rt.ws_y.ptr, (size_t)n * e->h * 4, hipMemcpyDeviceToHost, st), "embedding download");
    hipError_t he = hipStreamSynchronize(st);
    if (he != hipSuccess) return fail(OXB_HIP_SYNC_FAILED, "device synchronization failed: embedding_rows: %s", hipGetErrorString(he));
    return OXB_HIP_OK;
    OXB_API_END
}

static int model_and_embedding(uint64_t model, uint64_t embedding, Model** m, Embedding** e) {
    *m = find_model(model);
    if (!*m) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: unknown model %llu", (unsigned long long)model);
    *e = find_embedding(embedding);
    if (!*e) return fail(OXB_HIP_WEIGHT_NOT_FOUND, "weight handle %llu (embedding) not found", (unsigned long long)embedding);
    if ((*e)->h != (*m)->d.h)
        return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: embedding rows hold %u values, the model's hidden size is %u", (*e)->h, (*m)->d.h);
    return OXB_HIP_OK;
}

static int check_sampling(const oxb_sampling& sp, uint32_t /*vocab*/) {
    if (!(sp.temperature >= 0.0f)) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: temperature %g", (double)sp.temperature);
    if (!(sp.top_p > 0.0f)) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: top_p %g", (double)sp.top_p);
    return OXB_HIP_OK;
}

static int decode_tokens_impl(uint64_t model, uint64_t embedding, const uint32_t* tokens, const uint32_t* pos, uint32_t n_steps,
                              const oxb_sampling* sp, uint64_t* rng_state, uint32_t* tokens_out) {
    std::lock_guard<std::recursive_mutex> lk(g_mu);
    Model* mp;
    Embedding* e;
    OXB_TRY(model_and_embedding(model, embedding, &mp, &e));
    Model& m = *mp;
    const oxb_model_desc& d = m.d;
    if (n_steps == 0) return OXB_HIP_OK;
    if (!tokens || !pos || !tokens_out) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: null tokens, pos or tokens_out");
    if (e->vocab < d.vocab)  // every argmax result must name a row of the table
        return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: embedding has %u rows, the LM head %u", e->vocab, d.vocab);
    OXB_TRY(check_ids(*e, tokens, d.batch));
    for (uint32_t b = 0; b < d.batch; b++)
        if ((uint64_t)pos[b] + n_steps > d.max_seq)
            return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: positions %u..%llu exceed the context of %u", pos[b],
                        (unsigned long long)pos[b] + n_steps - 1, d.max_seq);
    for (uint32_t b = 0; b < d.batch; b++) OXB_TRY(kv_reserve(m, b, (uint64_t)pos[b] + n_steps));
    OXB_TRY(kv_sync_table(m));
    const bool sampled = sp && sp->temperature >= 1e-6f;  // below: greedy (sampling.rs:89-92)
    if (sp) OXB_TRY(check_sampling(*sp, d.vocab));
    if (sampled && !rng_state) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: null rng_state");
    OXB_TRY(m.tok_hist.ensure((size_t)n_steps * d.batch * 4));
    hipStream_t st = g_rt.stream;
    if (sampled) {
        OXB_TRY(m.sample_ws.ensure(oxb_sample_ws_bytes(d.vocab, d.batch)));
        OXB_TRY(m.rng.ensure((size_t)d.batch * 8));
        OXB_TRY_HIP(hipMemcpyAsync(m.rng.ptr, rng_state, (size_t)d.batch * 8, hipMemcpyHostToDevice, st), "rng state upload");
    }
    uint32_t* hist = (uint32_t*)m.tok_hist.ptr;
    OXB_TRY_HIP(hipMemcpyAsync(m.tokens, tokens, (size_t)d.batch * 4, hipMemcpyHostToDevice, st), "token upload");
    OXB_TRY_HIP(hipMemcpyAsync(m.pos, pos, (size_t)d.batch * 4, hipMemcpyHostToDevice, st), "position upload");
    for (uint32_t i = 0; i < n_steps; i++) {
        OXB_TRY_HIP(oxb_launch_embedding_gather(e->d, e->type, e->vocab, d.h, m.tokens, d.batch, m.hidden, st),
                    "kernel launch failed: embedding_gather");
        OXB_TRY(run_decode_step(m));  // m.logits, m.tokens <- argmax
        if (sampled)
            OXB_TRY_HIP(oxb_launch_sample(m.logits, d.vocab, d.batch, sp->temperature, sp->top_k, sp->top_p, (uint64_t*)m.rng.ptr,
                                          m.tokens, m.sample_ws.ptr, st),
                        "kernel launch failed: sample");
        OXB_TRY_HIP(oxb_launch_token_step(m.tokens, hist + (size_t)i * d.batch, m.pos, d.batch, st), "kernel launch failed: token_step");
    }
    OXB_TRY_HIP(hipMemcpyAsync(tokens_out, hist, (size_t)n_steps * d.batch * 4, hipMemcpyDeviceToHost, st), "token download");
    if (sampled) OXB_TRY_HIP(hipMemcpyAsync(rng_state, m.rng.ptr, (size_t)d.batch * 8, hipMemcpyDeviceToHost, st), "rng state download");
    hipError_t he = hipStreamSynchronize(st);
    if (he != hipSuccess) return fail(OXB_HIP_SYNC_FAILED, "device synchronization failed: decode_tokens: %s", hipGetErrorString(he));
    return OXB_HIP_OK;
}

int oxb_hip_decode_tokens(uint64_t model, uint64_t embedding, const uint32_t* tokens, const uint32_t* pos, uint32_t n_steps,
                          uint32_t* tokens_out) {
    OXB_API_BEGIN
    return decode_tokens_impl(model, embedding, tokens, pos, n_steps, nullptr, nullptr, tokens_out);
    OXB_API_END
}

int oxb_hip_decode_tokens_sampled(uint64_t model, uint64_t embedding, const uint32_t* tokens, const uint32_t* pos, uint32_t n_steps,
                                  const oxb_sampling* params, uint64_t* rng_state, uint32_t* tokens_out) {
    OXB_API_BEGIN
    if (!params) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: null sampling parameters");
    return decode_tokens_impl(model, embedding, tokens, pos, n_steps, params, rng_state, tokens_out);
    OXB_API_END
}

int oxb_hip_sum_in_order(const float* x, uint32_t n, float* sum_out) {
    OXB_API_BEGIN
    std::lock_guard<std::recursive_mutex> lk(g_mu);
    if (!x || !sum_out || n == 0) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: null pointer or no elements");
    OXB_TRY(ensure_init());
    OXB_TRY(g_rt.ws_y.ensure((size_t)n * 4 + 256));
    float* d_x = (float*)g_rt.ws_y.ptr;
    float* d_sum = (float*)((uint8_t*)g_rt.ws_y.ptr + (((size_t)n * 4 + 255) & ~(size_t)255));
    hipStream_t st = g_rt.stream;
    OXB_TRY_HIP(hipMemcpyAsync(d_x, x, (size_t)n * 4, hipMemcpyHostToDevice, st), "upload");
    OXB_TRY_HIP(oxb_launch_sum_in_order(d_x, n, d_sum, st), "kernel launch failed: sum_in_order");
    OXB_TRY_HIP(hipMemcpyAsync(sum_out, d_sum, 4, hipMemcpyDeviceToHost, st), "download");
    hipError_t he = hipStreamSynchronize(st);
    if (he != hipSuccess) return fail(OXB_HIP_SYNC_FAILED, "device synchronization failed: sum_in_order: %s", hipGetErrorString(he));
    return OXB_HIP_OK;
    OXB_API_END
}

int oxb_hip_sample_logits(const float* logits, uint32_t vocab, uint32_t batch, const oxb_sampling* params, uint64_t* rng_state,
                          uint32_t* tokens_out) {
    OXB_API_BEGIN
    std::lock_guard<std::recursive_mutex> lk(g_mu);
    if (!logits || !params || !rng_state || !tokens_out || vocab == 0 || batch == 0)
        return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: null pointer or empty logits");
    OXB_TRY(check_sampling(*params, vocab));
    if ((vocab + 2047u) / 2048u > 256u) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: %u logits per row (at most 524288)", vocab);
    OXB_TRY(ensure_init());
    const size_t lb = (size_t)batch * vocab * 4, wb = oxb_sample_ws_bytes(vocab, batch);
    OXB_TRY(g_rt.ws_y.ensure(lb + wb + 256));
    OXB_TRY(g_rt.ws_x.ensure((size_t)batch * 16));
    float* d_logits = (float*)g_rt.ws_y.ptr;
    void* d_ws = (uint8_t*)g_rt.ws_y.ptr + ((lb + 255) & ~(size_t)255);
    uint64_t* d_rng = (uint64_t*)g_rt.ws_x.ptr;
    uint32_t* d_tok = (uint32_t*)(d_rng + batch);
    hipStream_t st = g_rt.stream;
    OXB_TRY_HIP(hipMemcpyAsync(d_logits, logits, lb, hipMemcpyHostToDevice, st), "logits upload");
    OXB_TRY_HIP(hipMemcpyAsync(d_rng, rng_state, (size_t)batch * 8, hipMemcpyHostToDevice, st), "rng state upload");
    if (params->temperature < 1e-6f) {
        OXB_TRY(g_rt.ws_aux.ensure((size_t)batch * OXB_ARGMAX_MAX_PARTS * 8));
        OXB_TRY_HIP(oxb_launch_argmax(d_logits, vocab, batch, d_tok, g_rt.ws_aux.ptr, st), "kernel launch failed: argmax");
    } else {
        OXB_TRY_HIP(oxb_launch_sample(d_logits, vocab, batch, params->temperature, params->top_k, params->top_p, d_rng, d_tok, d_ws, st),
                    "kernel launch failed: sample");
    }
    OXB_TRY_HIP(hipMemcpyAsync(tokens_out, d_tok, (size_t)batch * 4, hipMemcpyDeviceToHost, st), "token download");
    OXB_TRY_HIP(hipMemcpyAsync(rng_state, d_rng, (size_t)batch * 8, hipMemcpyDeviceToHost, st), "rng state download");
    hipError_t he = hipStreamSynchronize(st);
    if (he != hipSuccess) return fail(OXB_HIP_SYNC_FAILED, "device synchronization failed: sample_logits: %s", hipGetErrorString(he));
    return OXB_HIP_OK;
    OXB_API_END
}

int oxb_hip_prefill_tokens(uint64_t model, uint64_t embedding, uint32_t seq, const uint32_t* ids, uint32_t n_tokens,
                           uint32_t pos_start, float* logits_or_null, uint32_t* token_out_or_null) {
    OXB_API_BEGIN
    std::lock_guard<std::recursive_mutex> lk(g_mu);
    Model* mp;
    Embedding* e;
    OXB_TRY(model_and_embedding(model, embedding, &mp, &e));
    Model& m = *mp;
    const oxb_model_desc& d = m.d;
    if (!ids || n_tokens == 0) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: null ids or no tokens");
    if (!d.lm_head && (logits_or_null || token_out_or_null))
        return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: the model has no LM head: logits and token must be null");
    if (m.checked_gen != g_rt.weights_gen) OXB_TRY(check_model_handles(m));
    if (seq >= d.batch) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: sequence %u of a batch of %u", seq, d.batch);
    if ((uint64_t)pos_start + n_tokens > d.max_seq)
        return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: positions %u..%llu exceed the context of %u", pos_start,
                    (unsigned long long)pos_start + n_tokens - 1, d.max_seq);
    OXB_TRY(check_ids(*e, ids, n_tokens));
    OXB_TRY(kv_reserve(m, seq, (uint64_t)pos_start + n_tokens));
    OXB_TRY(kv_sync_table(m));
    OXB_TRY(ensure_prefill_buffers(m, n_tokens));
    OXB_TRY(m.tok_ids.ensure((size_t)n_tokens * 4));
    hipStream_t st = g_rt.stream;
    OXB_TRY_HIP(hipMemcpyAsync(m.tok_ids.ptr, ids, (size_t)n_tokens * 4, hipMemcpyHostToDevice, st), "token id upload");
    OXB_TRY_HIP(oxb_launch_embedding_gather(e->d, e->type, e->vocab, d.h, (const uint32_t*)m.tok_ids.ptr, n_tokens, m.pf_hidden, st),
                "kernel launch failed: embedding_gather");
    OXB_TRY(encode_prefill(m, seq, n_tokens, pos_start));
    if (token_out_or_null) OXB_TRY_HIP(hipMemcpyAsync(token_out_or_null, m.tokens + seq, 4, hipMemcpyDeviceToHost, st), "token download");
    if (logits_or_null)
        OXB_TRY_HIP(hipMemcpyAsync(logits_or_null, m.logits + (size_t)seq * d.vocab, (size_t)d.vocab * 4, hipMemcpyDeviceToHost, st), "logits download");
    hipError_t he = hipStreamSynchronize(st);
    if (he != hipSuccess) return fail(OXB_HIP_SYNC_FAILED, "device synchronization failed: prefill_tokens: %s", hipGetErrorString(he));
    return OXB_HIP_OK;
    OXB_API_END
}

// --- GGUF ---------------------------------------------------------------------------------------------------
static int gguf_fail(const std::string& why) { return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: GGUF: %s", why.c_str()); }

// Configuration the way Qwen3Config::from_metadata reads it (crates/oxibonsai-core/src/config.rs:41-118):
// "<architecture>.<key>" first, then "llm.<key>", then the Bonsai-8B default.
static int gguf_describe(const GgufFile& g, oxb_gguf_info* info) {
    memset(info, 0, sizeof *info);
    info->version = g.version;
    info->alignment = g.alignment;
    info->n_tensors = g.n_tensors;
    info->n_metadata = g.n_kv;
    std::string arch = "qwen3", name = "Bonsai-8B";
    (void)g.get_str("general.architecture", &arch);
    (void)g.get_str("general.name", &name);
    snprintf(info->architecture, sizeof info->architecture, "%s", arch.c_str());
    snprintf(info->name, sizeof info->name, "%s", name.c_str());
    auto u32 = [&](const char* key, uint32_t dflt) {
        uint32_t v = dflt;
        if (!g.get_u32(arch + "." + key, &v)) (void)g.get_u32(std::string("llm.") + key, &v);
        return v;
    };
    auto f32 = [&](const char* key, float dflt) {
        float v = dflt;
        if (!g.get_f32(arch + "." + key, &v)) (void)g.get_f32(std::string("llm.") + key, &v);
        return v;
    };
    info->h = u32("embedding_length", 4096);
    info->n_layers = u32("block_count", 36);
    info->nq = u32("attention.head_count", 32);
    info->nkv = u32("attention.head_count_kv", 8);
    info->inter = u32("feed_forward_length", 14336);
    info->vocab = u32("vocab_size", 151936);
    info->context_length = u32("context_length", 65536);
    info->eps = f32("attention.layer_norm_rms_epsilon", 1e-6f);
    info->rope_theta = f32("rope.freq_base", 1000000.0f);
    if (info->nq == 0) return gguf_fail("attention.head_count is 0");
    info->hd = info->h / info->nq;
    // the embedding tensor's row count overrides the metadata (model/types/mod.rs:73-86)
    const GgufTensor* emb = g.find("token_embd.weight");
    if (!emb) return gguf_fail("tensor not found: token_embd.weight");
    if (emb->shape.size() >= 2 && emb->shape[1] <= UINT32_MAX) info->vocab = (uint32_t)emb->shape[1];
    info->embedding_type = (int)emb->type;
    info->lm_head_rows = info->vocab;
    if (const GgufTensor* out = g.find("output.weight"))
        if (out->shape.size() >= 2 && out->shape[1] <= UINT32_MAX) info->lm_head_rows = (uint32_t)out->shape[1];
    const GgufTensor* q = g.find("blk.0.attn_q.weight");
    if (!q) return gguf_fail("tensor not found: blk.0.attn_q.weight");
    if (q->type == GGUF_Q1_0_G128) info->fmt = OXB_FMT_Q1;
    else if (q->type == GGUF_TQ2_0_G128) info->fmt = OXB_FMT_TQ2;
    else return gguf_fail("blk.0.attn_q.weight has tensor type " + std::to_string(q->type) + "; this tier runs Q1_0_g128 (41) and TQ2_0_g128 (42)");
    return OXB_HIP_OK;
}

int oxb_hip_gguf_info(const char* path, oxb_gguf_info* info) {
    OXB_API_BEGIN
    if (!info) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: null info");
    GgufFile g;
    std::string err;
    if (!g.open(path, &err)) return gguf_fail(err);
    return gguf_describe(g, info);
    OXB_API_END
}

int oxb_hip_gguf_metadata(const char* path, const char* key, char* out, size_t out_cap) {
    OXB_API_BEGIN
    if (!key || !out || out_cap == 0) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: null key or output");
    GgufFile g;
    std::string err;
    if (!g.open(path, &err)) return gguf_fail(err);
    auto it = g.meta.find(key);
    if (it == g.meta.end()) return fail(OXB_HIP_WEIGHT_NOT_FOUND, "metadata key %s not found", key);
    const GgufValue& v = it->second;
    switch (v.type) {
        case 0: case 2: case 4: case 10: snprintf(out, out_cap, "%llu", (unsigned long long)v.u); break;
        case 1: case 3: case 5: case 11: snprintf(out, out_cap, "%lld", (long long)v.i); break;
        case 6: case 12: snprintf(out, out_cap, "%.9g", v.f); break;
        case 7: snprintf(out, out_cap, "%s", v.u ? "true" : "false"); break;
        case 8: snprintf(out, out_cap, "%s", v.s.c_str()); break;
        default: snprintf(out, out_cap, "[%llu x type %u]", (unsigned long long)v.count, v.elem_type); break;
    }
    return OXB_HIP_OK;
    OXB_API_END
}

int oxb_hip_gguf_tensor(const char* path, const char* name, int* type, uint32_t* n_dims, uint64_t shape4[4],
                        uint64_t* file_offset, uint64_t* n_bytes) {
    OXB_API_BEGIN
    if (!name) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: null name");
    GgufFile g;
    std::string err;
    if (!g.open(path, &err)) return gguf_fail(err);
    const GgufTensor* t = g.find(name);
    if (!t) return fail(OXB_HIP_WEIGHT_NOT_FOUND, "tensor not found: %s", name);
    if (type) *type = (int)t->type;
    if (n_dims) *n_dims = (uint32_t)t->shape.size();
    if (shape4)
        for (size_t i = 0; i < 4; i++) shape4[i] = i < t->shape.size() ? t->shape[i] : 0;
    if (file_offset) *file_offset = g.data_offset + t->offset;
    if (n_bytes) *n_bytes = t->bytes;
    return OXB_HIP_OK;
    OXB_API_END
}

// A tensor that must exist with the given type(s) and GGUF shape [in (, out)].
static int gguf_require(const GgufFile& g, const std::string& name, uint32_t type_a, uint32_t type_b, uint64_t in, uint64_t out,
                        const GgufTensor** t) {
    *t = g.find(name);
    if (!*t) return gguf_fail("tensor not found: " + name);
    const GgufTensor& x = **t;
    if (x.type != type_a && x.type != type_b)
        return gguf_fail(name + " has tensor type " + std::to_string(x.type) + ", expected " + std::to_string(type_a) +
                         (type_b != type_a ? " or " + std::to_string(type_b) : ""));
    const bool shape_ok = out ? (x.shape.size() == 2 && x.shape[0] == in && x.shape[1] == out) : (x.shape.size() == 1 && x.shape[0] == in);
    if (!shape_ok) {
        std::string sh;
        for (uint64_t v : x.shape) sh += (sh.empty() ? "" : ", ") + std::to_string(v);
        return gguf_fail(name + " has shape [" + sh + "], expected [" + std::to_string(in) + (out ? ", " + std::to_string(out) : "") + "]");
    }
    if (!x.data) return gguf_fail("unexpected end of file at offset " + std::to_string(g.data_offset + x.offset + x.bytes) + " (tensor " + name + ")");
    return OXB_HIP_OK;
}

// Norm vector, F32 or F16 widened (model/weight_loaders.rs:24-46) -> resident fp32 vector owned by the model.
static int gguf_vector(const GgufFile& g, Model& m, const std::string& name, uint32_t n, uint64_t* id) {
    const GgufTensor* t;
    OXB_TRY(gguf_require(g, name, GGUF_F32, GGUF_F16, n, 0, &t));
    std::vector<float> v(n);
    if (t->type == GGUF_F32) memcpy(v.data(), t->data, (size_t)n * 4);
    else
        for (uint32_t i = 0; i < n; i++) {
            uint16_t b;
            memcpy(&b, t->data + 2 * (size_t)i, 2);
            v[i] = __half2float(__ushort_as_half(b));
        }
    *id = 0;
    OXB_TRY(oxb_hip_upload_f32(id, v.data(), n));
    m.owned_vecs.push_back(*id);
    return OXB_HIP_OK;
}

// Row concatenation of projection matrices that share k (Q|K|V, gate|up): their AoS block arrays back to back
// (crates/oxibonsai-model/src/block/types/upload.rs:21-39) -> one resident matrix owned by the model.
static int gguf_matrix(const GgufFile& g, Model& m, int fmt, const std::vector<std::pair<std::string, uint32_t>>& parts, uint32_t k,
                       uint64_t* id) {
    const uint32_t type = fmt == OXB_FMT_Q1 ? GGUF_Q1_0_G128 : GGUF_TQ2_0_G128;
    std::vector<const GgufTensor*> ts(parts.size());
    uint32_t rows = 0;
    size_t bytes = 0;
    for (size_t i = 0; i < parts.size(); i++) {
        OXB_TRY(gguf_require(g, parts[i].first, type, type, k, parts[i].second, &ts[i]));
        rows += parts[i].second;
        bytes += ts[i]->bytes;
    }
    *id = 0;
    int rc;
    if (parts.size() == 1) {
        rc = upload_weight(id, fmt, ts[0]->data, ts[0]->bytes, rows, k);
    } else {
        std::vector<uint8_t> cat(bytes);
        size_t off = 0;
        for (const GgufTensor* t : ts) {
            memcpy(cat.data() + off, t->data, t->bytes);
            off += t->bytes;
        }
        rc = upload_weight(id, fmt, cat.data(), bytes, rows, k);
    }
    if (rc) return rc;
    m.owned_mats.push_back(*id);
    return OXB_HIP_OK;
}

int oxb_hip_load_gguf(const char* path, uint32_t max_seq, uint32_t batch, uint64_t* model, uint64_t* embedding,
                      oxb_gguf_info* info_or_null) {
    OXB_API_BEGIN
    std::lock_guard<std::recursive_mutex> lk(g_mu);
    if (!model || !embedding) return fail(OXB_HIP_INVALID_ARGUMENT, "invalid argument: null model or embedding pointer");
    GgufFile g;
    std::string err;
    if (!g.open(path, &err)) return gguf_fail(err);
    oxb_gguf_info info;
    OXB_TRY(gguf_describe(g, &info));
    if (info_or_null) *info_or_null = info;
    // every layer brings nine tensors of its own: a block count beyond that (or beyond any model this tier could hold)
    // is a damaged or hostile header, not a model; nothing is allocated for it
    if (info.n_layers == 0 || info.n_layers > 4096 || (uint64_t)info.n_layers * 9 > g.n_tensors)
        return gguf_fail("block_count " + std::to_string(info.n_layers) + " does not fit a file of " + std::to_string(g.n_tensors) + " tensors");
    if (info.h % 128 || info.inter % 128 || info.hd == 0 || info.h != info.nq * info.hd)
        return gguf_fail("hidden " + std::to_string(info.h) + " / heads " + std::to_string(info.nq) + " / intermediate " +
                         std::to_string(info.inter) + " do not fit this tier (multiples of 128, hidden = heads x head_dim)");
    OXB_TRY(ensure_init());

    // uploads are collected in a scratch model so that any failure frees what was uploaded so far
    Model owner;
    std::vector<oxb_layer_ids> layers(info.n_layers);
    uint64_t final_norm = 0, lm_head = 0;
    const uint32_t qd = info.nq * info.hd, kd = info.nkv * info.hd;
    int rc = OXB_HIP_OK;
    for (uint32_t L = 0; L < info.n_layers && !rc; L++) {
        const std::string b = "blk." + std::to_string(L) + ".";
        oxb_layer_ids& ly = layers[L];
        (rc = gguf_vector(g, owner, b + "attn_norm.weight", info.h, &ly.attn_norm)) ||
            (rc = gguf_vector(g, owner, b + "ffn_norm.weight", info.h, &ly.ffn_norm)) ||
            (rc = gguf_vector(g, owner, b + "attn_q_norm.weight", info.hd, &ly.q_norm)) ||
            (rc = gguf_vector(g, owner, b + "attn_k_norm.weight", info.hd, &ly.k_norm)) ||
            (rc = gguf_matrix(g, owner, info.fmt, {{b + "attn_q.weight", qd}, {b + "attn_k.weight", kd}, {b + "attn_v.weight", kd}}, info.h, &ly.qkv)) ||
            (rc = gguf_matrix(g, owner, info.fmt, {{b + "attn_output.weight", info.h}}, qd, &ly.o)) ||
            (rc = gguf_matrix(g, owner, info.fmt, {{b + "ffn_gate.weight", info.inter}, {b + "ffn_up.weight", info.inter}}, info.h, &ly.gate_up)) ||
            (rc = gguf_matrix(g, owner, info.fmt, {{b + "ffn_down.weight", info.h}}, info.inter, &ly.down));
    }
    if (!rc) rc = gguf_vector(g, owner, "output_norm.weight", info.h, &final_norm);
    // the LM head's row count comes from its own shape (model/weight_loaders.rs:654-666)
    const uint32_t lm_rows = info.lm_head_rows;
    if (!rc && !g.find("output.weight")) rc = gguf_fail("tensor not found: output.weight");
    if (!rc) rc = gguf_matrix(g, owner, info.fmt, {{"output.weight", lm_rows}}, info.h, &lm_head);
    uint64_t emb_id = 0;
    if (!rc) {
        const GgufTensor* emb;
        rc = gguf_require(g, "token_embd.weight", (uint32_t)info.embedding_type, (uint32_t)info.embedding_type, info.h, info.vocab, &emb);
        if (!rc) rc = oxb_hip_upload_embedding(&emb_id, emb->data, emb->bytes, info.embedding_type, info.vocab, info.h);
    }
    uint64_t mid = 0;
    if (!rc) {
        oxb_model_desc d;
        memset(&d, 0, sizeof d);
        d.fmt = info.fmt;
        d.n_layers = info.n_layers, d.h = info.h, d.inter = info.inter, d.nq = info.nq, d.nkv = info.nkv, d.hd = info.hd;
        d.vocab = lm_rows;
        d.max_seq = max_seq ? max_seq : info.context_length;
        d.batch = batch;
        d.eps = info.eps, d.rope_theta = info.rope_theta;
        d.layers = layers.data();
        d.final_norm = final_norm, d.lm_head = lm_head;
        rc = oxb_hip_model_create(&d, &mid);
    }
    if (rc) {
        for (uint64_t id : owner.owned_mats) (void)oxb_hip_free_weight(id);
        for (uint64_t id : owner.owned_vecs) (void)oxb_hip_free_f32(id);
        if (emb_id) (void)oxb_hip_free_embedding(emb_id);
        return rc;
    }
    Model* m = find_model(mid);
    m->owned_mats = std::move(owner.owned_mats);
    m->owned_vecs = std::move(owner.owned_vecs);
    *model = mid;
    *embedding = emb_id;
    return OXB_HIP_OK;
    OXB_API_END
}

}  // extern "C"
