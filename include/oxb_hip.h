/*
 * oxb_hip.h — C ABI of the `native-hip` kernel tier (liboxb_hip.so / liboxb_hip.a).
 *
 * This is what a Rust `NativeHipBackend: GpuBackendTrait` binds through
 * `extern "C"`; each entry point names the reference interface it stands in
 * for.  Paths are relative to the reference checkout; KG = crates/oxibonsai-kernels/src/gpu_backend.
 *
 * Conventions
 *   - every function returns an oxb_status; 0 is success.  The text of the last
 *     failure on the calling thread is available from oxb_hip_last_error().
 *     Codes follow GpuError (KG/mod.rs:317-342) and CudaGraphError::WeightNotFound
 *     (KG/cuda_graph/types.rs:25-39).  No C++ exception crosses the boundary.
 *   - pointers without a `d_` prefix are HOST pointers borrowed for the call;
 *     `d_` pointers are DEVICE pointers.  The library owns all weight memory.
 *   - calls are serialised by an internal mutex and run on one stream
 *     (the library's own, or the one given to oxb_hip_set_stream), like the
 *     reference's Mutex-guarded CudaGraph singleton (KG/cuda_graph/cudagraph_type.rs:18-32).
 *   - there is no CPU fallback: without a usable GPU every compute entry point
 *     returns OXB_HIP_NOT_AVAILABLE and the caller decides (the reference's
 *     dispatcher falls back to its CPU tiers on Err, crates/oxibonsai-kernels/src/dispatch.rs:471-483).
 */
#ifndef OXB_HIP_H
#define OXB_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
    OXB_HIP_OK = 0,
    OXB_HIP_NOT_AVAILABLE = 1,     /* GpuError::NotAvailable      */
    OXB_HIP_OUT_OF_MEMORY = 2,     /* GpuError::OutOfMemory       */
    OXB_HIP_KERNEL_LAUNCH = 3,     /* GpuError::KernelLaunch      */
    OXB_HIP_SYNC_FAILED = 4,       /* GpuError::SyncFailed        */
    OXB_HIP_INVALID_ARGUMENT = 5,  /* GpuError::InvalidArgument   */
    OXB_HIP_WEIGHT_NOT_FOUND = 6   /* CudaGraphError::WeightNotFound */
} oxb_status;

enum { OXB_HIP_FMT_Q1 = 0, OXB_HIP_FMT_TQ2 = 1 };

/* ---- lifecycle: CudaGraph::global() / NativeCudaBackend::new  (KG/cuda_graph/cudagraph_type.rs, KG/mod.rs:1092-1106) */
int  oxb_hip_init(int device_ordinal);            /* idempotent */
void oxb_hip_shutdown(void);                      /* frees every weight and workspace */
/* GpuBackendTrait::name / device_count / memory_info  (KG/mod.rs:360-406) */
int  oxb_hip_device_count(void);
int  oxb_hip_device_info(char* name, size_t name_cap, size_t* free_bytes, size_t* total_bytes);
/* GpuBackendTrait::synchronize (KG/mod.rs:403) */
int  oxb_hip_synchronize(void);
/* Run on the caller's HIP stream (hipStream_t passed as void*); NULL restores the library's own stream.
 * The decode step's graph is recorded on the library's own stream and replayed on the stream in use. */
int  oxb_hip_set_stream(void* hip_stream);
const char* oxb_hip_last_error(void);

/* ---- weights: GpuBackendTrait::upload_weights_raw (KG/mod.rs:445) and upload_weights_ternary (:472).
 * aos = n_rows * (k/128) blocks in the reference's byte order: Q1 18 B [d f16][qs 16], TQ2 34 B [qs 32][d f16].
 * *id == 0 on entry asks the library to allocate a handle; a non-zero *id is used as given
 * (the fused paths key weights by caller-chosen ids, crates/oxibonsai-model/src/model/types/forward_cuda/q1.rs:71-72)
 * and replaces a weight already stored under it. */
int  oxb_hip_upload_q1(uint64_t* id, const uint8_t* aos, size_t n_bytes, uint32_t n_rows, uint32_t k);
int  oxb_hip_upload_tq2(uint64_t* id, const uint8_t* aos, size_t n_bytes, uint32_t n_rows, uint32_t k);
/* The same uploads as the trait has them, bytes (or blocks) only: upload_weights_raw(&self, blocks: &[u8]) (KG/mod.rs:445)
 * and upload_weights_ternary(&self, blocks: &[BlockTQ2_0_g128]) (KG/mod.rs:472; n_bytes = 34 * blocks.len()).  The weight
 * takes its shape from the first call that names one - gemv_q1_g128_cached(handle, input, n_rows, k) (KG/mod.rs:457), a GEMM,
 * or oxb_hip_model_create through the model's dimensions - which must satisfy n_rows * k / 128 == number of blocks; the
 * device then repacks the bytes into the resident layout (the result is what the shaped upload stores, bit for bit) and
 * the shape stays.  That first call must not run inside a stream capture.  Until then oxb_hip_weight_info reports
 * 0 x 0 and oxb_hip_dequant fails. */
int  oxb_hip_upload_q1_raw(uint64_t* id, const uint8_t* aos, size_t n_bytes);
int  oxb_hip_upload_tq2_raw(uint64_t* id, const uint8_t* aos, size_t n_bytes);
int  oxb_hip_free_weight(uint64_t id);
int  oxb_hip_weight_info(uint64_t id, int* fmt, uint32_t* n_rows, uint32_t* k, size_t* resident_bytes);
/* Decode the resident copy back to fp32 [n_rows][k]: dequant_1bit_g128 / dequant_tq2_0_g128
 * (crates/oxibonsai-kernels/src/dequant.rs:15-37, dequant_ternary.rs:42-64) run on the device layout. */
int  oxb_hip_dequant(uint64_t id, float* out, size_t out_len);

/* ---- GEMV / GEMM on resident weights: gemv_q1_g128_cached (KG/mod.rs:457), gemv_tq2_g128_cached (:484).
 * x: [batch][k], y: [batch][n_rows], both row-major fp32; batch >= 1 (one pass over the weights serves up to eight
 * vectors).
 * Non-finite activations, a deliberate difference: the kernels turn each activation vector into fixed point, which
 * has no infinity, so a vector that holds an infinity or a NaN anywhere gives a quiet NaN in EVERY output row of that
 * vector.  The reference's fp32 sums (crates/oxibonsai-kernels/src/gemv.rs:60-84) give +-infinity in the rows a lone
 * infinity reaches with one sign and NaN where +inf meets -inf or a NaN; none of its tests fixes the case.  The same
 * holds for the fused model entry points, whose projections are these kernels. */
int  oxb_hip_gemv(uint64_t id, const float* x, float* y, uint32_t n_rows, uint32_t k, uint32_t batch);
/* Same with device-resident x / y, asynchronous on the current stream. */
int  oxb_hip_gemv_dev(uint64_t id, const float* d_x, float* d_y, uint32_t n_rows, uint32_t k, uint32_t batch);

/* ---- uncached one-shot calls: gemv_q1_g128 (KG/mod.rs:412), gemm_q1_g128 (:425) and their ternary twins.
 * Validation follows the scalar kernels (crates/oxibonsai-kernels/src/gemv.rs:32-58): k % 128, buffer lengths. */
int  oxb_hip_gemv_q1_g128(const uint8_t* aos, size_t n_bytes, const float* x, size_t x_len,
                          float* y, size_t y_len, uint32_t n_rows, uint32_t k);
int  oxb_hip_gemv_tq2_g128(const uint8_t* aos, size_t n_bytes, const float* x, size_t x_len,
                           float* y, size_t y_len, uint32_t n_rows, uint32_t k);

/* ---- prefill GEMM: GpuBackendTrait::gemm_q1_g128 (KG/mod.rs:425-441; scalar semantics K/gemm.rs:19-87,
 * K/gemm_ternary.rs:35-69; CUDA tier: gemm_q1_g128_v7 / gemm_tq2_g128_v7, KG/cuda_prefill_kernels.rs:74-140, 457-551).
 * y[m][n_rows] = x[m][k] * W^T on the fp16 matrix cores with fp32 accumulation: weights and products are exact,
 * activations are rounded to fp16 after a per-row power-of-two scaling (relative 2^-11 per element).  Use
 * oxb_hip_gemv with batch = m where fp32-exact products are required.  _dev takes device pointers and does not
 * synchronize. */
int  oxb_hip_gemm(uint64_t id, const float* x, float* y, uint32_t m, uint32_t n_rows, uint32_t k);
int  oxb_hip_gemm_dev(uint64_t id, const float* d_x, float* d_y, uint32_t m, uint32_t n_rows, uint32_t k);
/* oxb_hip_gemm_dev for callers that cannot allocate (no counterpart in the reference): code under HIP graph capture,
 * serving loops and harnesses that forbid hipMalloc.  Same kernels and results, but the call's scratch - packed fp16
 * activations, per-row exponents, the partial sums of a K split - lies in a 32 MiB array inside the library's code
 * object instead of a workspace that grows on demand; no allocation or free of device memory happens in the call.  A shape
 * whose scratch exceeds the array is OXB_HIP_INVALID_ARGUMENT (the message gives both sizes).  Every call on a GPU
 * uses that GPU's one array: calls that overlap in time (different streams) race. */
int  oxb_hip_gemm_dev_static(uint64_t id, const float* d_x, float* d_y, uint32_t m, uint32_t n_rows, uint32_t k);

/* ---- batch_ffn_phase (KG/mod.rs:519; CUDA: KG/cuda_graph/nativecudabackend_traits.rs:122-188 -> encode_ffn_phase,
 * KG/cuda_graph/cudagraph_encoding.rs:72-160): hidden += O * attn_out; normed = RMSNorm(hidden); hidden += down * SwiGLU(gate||up * normed),
 * in place on the host vector `hidden[h]`.  fmt selects Q1 / TQ2 weights; gate_up holds the gate rows, then the up rows. */
int  oxb_hip_ffn_phase(int fmt, float* hidden, const float* attn_out, const float* norm_w, float eps,
                       uint64_t o_id, uint64_t gate_up_id, uint64_t down_id, uint32_t h, uint32_t inter, uint32_t attn_k);

/* ---- batch_attn_phase (KG/mod.rs:501-512; the Metal tier's implementation: KG/scirs2_backend.rs:1187-1232):
 * normed = RMSNorm(hidden, norm_w, eps); [q | k | v] = qkv * normed in one launch; q receives q_rows values, k and v
 * k_rows each.  The reference's dispatcher keeps this phase switched off (crates/oxibonsai-kernels/src/dispatch.rs:605-621)
 * and its CUDA tier leaves the trait default (Ok(None)); offered so that the trait binds completely. */
int  oxb_hip_attn_phase(int fmt, const float* hidden, const float* norm_w, float eps, uint64_t qkv_id, uint32_t q_rows,
                        uint32_t k_rows, uint32_t h, float* q, float* k, float* v);

/* ---- fused whole-model decode: try_cuda_full_forward[_ternary]_with_gpu_lm_head
 * (KG/cuda_full_layer/encode_q1.rs:881-900, encode_ternary.rs:755-774) with per-layer parameters as in
 * CudaFullForwardLayerParams (KG/cuda_full_layer/mod.rs:250-268): norm vectors and weight matrices are named by
 * handle.  Norm vectors are uploaded with oxb_hip_upload_f32; `qkv` is the Q|K|V row concatenation
 * ((nq + 2 nkv) * hd rows), `gate_up` the gate|up concatenation (2 * inter rows), as the reference builds them
 * (crates/oxibonsai-model/src/block/types/upload.rs:21-39). */
int  oxb_hip_upload_f32(uint64_t* id, const float* w, size_t n);
int  oxb_hip_free_f32(uint64_t id);
typedef struct { uint64_t attn_norm, qkv, q_norm, k_norm, o, ffn_norm, gate_up, down; } oxb_layer_ids;
typedef struct {
    int fmt;                       /* OXB_HIP_FMT_Q1 / OXB_HIP_FMT_TQ2 for every matrix */
    uint32_t n_layers, h, inter, nq, nkv, hd, vocab, max_seq, batch;
    float eps, rope_theta;
    const oxb_layer_ids* layers;   /* [n_layers], read during the call only */
    uint64_t final_norm, lm_head;  /* lm_head == 0: no LM head on the device (vocab is ignored; final_norm may be 0 too) */
} oxb_model_desc;
/* Allocates the FP16 KV cache [batch][layer][kv_head][max_seq rounded up to 128][hd] (CudaKvCache, KG/cuda_full_layer/mod.rs:112-139),
 * the activation buffers (mod.rs:149-181) and the RoPE table (crates/oxibonsai-model/src/layers/rope.rs:27-48). */
int  oxb_hip_model_create(const oxb_model_desc* desc, uint64_t* model);
int  oxb_hip_model_reset(uint64_t model);
int  oxb_hip_model_destroy(uint64_t model);
/* One token for each of the `batch` sequences: hidden[batch][h] are the embedding rows, pos[batch] the positions.
 * Runs all layers, the final norm, the LM head and a first-maximum argmax on the device (a HIP graph after the first
 * call).  logits_or_null: [batch][vocab]; token_out: [batch] greedy ids (either may be NULL).
 * Batches of up to 4 use the fp32-exact GEMV (one pass over the weights); from 5 sequences on the projections run as
 * fp16 matrix-core GEMMs (the arithmetic of oxb_hip_gemm / oxb_hip_prefill). */
int  oxb_hip_decode(uint64_t model, const float* hidden, const uint32_t* pos, float* logits_or_null, uint32_t* token_out);
/* The same step without the LM head: try_cuda_full_forward / try_cuda_full_forward_ternary
 * (KG/cuda_full_layer/encode_q1.rs:813-830, encode_ternary.rs:694-711) return the hidden state after the last layer and
 * the final RMSNorm (final_norm_bytes: Option - a model created with final_norm == 0 returns the un-normed state);
 * the caller runs its own LM head.  normed_out: [batch][h].  Plain launches, no graph. */
int  oxb_hip_decode_hidden(uint64_t model, const float* hidden, const uint32_t* pos, float* normed_out);
/* Gives a model its final norm vector and LM head after the fact, or other ones (lm_head == 0 takes the LM head away).
 * The reference's entry points name them per call (final_norm_handle, lm_head_handle, lm_head_bytes, vocab_size,
 * encode_q1.rs:881-900), and try_cuda_full_forward_with_gpu_lm_head continues on the cache try_cuda_full_forward
 * filled: the KV cache and the positions decoded so far stay as they are. */
int  oxb_hip_model_set_lm_head(uint64_t model, uint64_t final_norm, uint64_t lm_head, uint32_t vocab);
/* The reference's entry points receive the RoPE rows of their positions from the caller (rope_cos / rope_sin of `pos`,
 * hd/2 values each, encode_q1.rs:816-817; cos_table / sin_table [batch_size][hd/2] for a prefill, KG/cuda_prefill/try_apis.rs:48-49).
 * This call stores such rows for positions pos_start .. pos_start + n_pos - 1 in the model's table, in place of the
 * values oxb_hip_model_create worked out from rope_theta, so that a caller with its own table (scaled or extended
 * RoPE) gets its own angles. */
int  oxb_hip_model_set_rope_rows(uint64_t model, uint32_t pos_start, uint32_t n_pos, const float* cos_rows, const float* sin_rows);
/* Batched prefill: try_cuda_prefill / try_cuda_prefill_ternary (KG/cuda_prefill/try_apis.rs:42, 318; per layer
 * encode_prefill_layer[_ternary], KG/cuda_prefill/encode_q1.rs:123, encode_ternary.rs:114).  hidden = [n_tokens][h]
 * embedding rows of sequence `seq` (0 .. batch-1) for positions pos_start .. pos_start + n_tokens - 1; keys and
 * values of those positions are written to the sequence's cache, so decode (or another prefill chunk) continues
 * at pos_start + n_tokens.  Projections run as prefill GEMMs (oxb_hip_gemm), attention as one causal launch per
 * layer; logits [vocab] and the greedy token are those of the last token (either pointer may be null). */
int  oxb_hip_prefill(uint64_t model, uint32_t seq, const float* hidden, uint32_t n_tokens, uint32_t pos_start,
                     float* logits_or_null, uint32_t* token_out_or_null);
int  oxb_hip_model_uses_graph(uint64_t model);   /* 1 once the decode step is replayed from a captured graph */

/* ---- long-context options of the attention kernels (decode and prefill), modelled on what the reference's CPU
 * library offers beside its plain cache:
 *  - sliding window with attention sinks: SlidingWindowConfig { window_size, sink_tokens } and is_in_window
 *    (crates/oxibonsai-model/src/layers/sliding_window.rs:11-43, 173-189): the query at position p sees key k iff
 *    k < sink_tokens or p - k < window_size - sink_tokens.  window_size 0 switches the window off (every key up to
 *    p is visible).  The cache keeps every row (no eviction); chunks outside the window are not read.
 *  - quantised KV rows: one byte per value and one f32 scale per (position, kv head).  OXB_KV_DTYPE_I8 follows
 *    QuantizedKvLayer / quantize_row_i8 (crates/oxibonsai-model/src/kv_cache_quant.rs:46-62, 98-195),
 *    OXB_KV_DTYPE_FP8_E4M3 follows Fp8KvLayer / quantize_row_fp8 with Fp8KvFormat::E4M3 (:502-540) and
 *    fp8_e4m3_encode (crates/oxibonsai-core/src/quant_fp8.rs:47-160); attention reads code * scale (:69-71, :545-556).
 *    Device layout: codes [batch][layer][kv_head][max_seq rounded up to 128][hd] (head-major, where the reference's layer keeps
 *    [token][head][dim]), scales [batch][layer][kv_head][max_seq rounded up to 128].  Fp8KvFormat::E5M2 is not
 *    offered: its row quantiser turns the row maximum into infinity whenever max / scale rounds above 57344
 *    (quant_fp8.rs:229-231), about one row in five.
 *  - paged cache: PagedKvCache / BlockPool / BlockTable (crates/oxibonsai-model/src/paged_kv_cache.rs:70-160, 187-236,
 *    294-345).  The cache is a pool of n_pages pages of page_size positions (DEFAULT_BLOCK_SIZE = 16, :33); a page number
 *    stands for those positions in every layer and kv head (device rows [layer][kv_head][page][position][hd], where the
 *    reference allocates one page per layer in lockstep), so one table of page numbers per sequence serves all layers.  The model's `batch`
 *    sequence slots take the place of the reference's sequence ids.  Pages are handed out lazily: decode and prefill
 *    calls reserve what the positions they write need, as write_kv does (:447-470); when the pool is empty they fail
 *    with OXB_HIP_OUT_OF_MEMORY ("out of memory: no free KV blocks", PagedKvError::OutOfMemory) and the pages taken
 *    so far stay with the sequence, as in ensure_capacity (:394-433).  The kernels look the page of a position up in
 *    the table; everything else (window, quantised rows) combines freely.
 * oxb_hip_model_set_attention may be called at any time between steps; changing kv_dtype, page_size or n_pages
 * replaces the cache, so the sequences start again at position 0. */
enum { OXB_KV_DTYPE_F16 = 0, OXB_KV_DTYPE_I8 = 1, OXB_KV_DTYPE_FP8_E4M3 = 2 };
typedef struct {
    int32_t kv_dtype;       /* OXB_KV_DTYPE_* */
    uint32_t window_size;   /* 0 = no window */
    uint32_t sink_tokens;
    uint32_t page_size;     /* paged cache: positions per page (16, 32, 64 or 128); 0 = contiguous cache */
    uint32_t n_pages;       /* paged cache: pages in the pool, shared by the model's sequences; 0 = contiguous cache */
} oxb_attention_options;
int  oxb_hip_model_set_attention(uint64_t model, const oxb_attention_options* opt);
int  oxb_hip_model_get_attention(uint64_t model, oxb_attention_options* opt);
/* Cache rows of positions pos .. pos + n_pos - 1 of one kv head as stored (QuantizedKvLayer::get_key / get_value
 * without the dequantisation, kv_cache_quant.rs:204-228): k_rows / v_rows receive n_pos * hd elements (2-byte fp16
 * or 1-byte codes), k_scales / v_scales n_pos row scales (1.0 for an fp16 cache).  Any pointer may be NULL. */
int  oxb_hip_model_read_kv(uint64_t model, uint32_t seq, uint32_t layer, uint32_t kv_head, uint32_t pos, uint32_t n_pos,
                           void* k_rows, void* v_rows, float* k_scales, float* v_scales);
/* Paged cache bookkeeping (each is a no-op / trivial answer for a contiguous cache):
 * reserve  = PagedKvCache::ensure_capacity (:394-433): pages for positions 0 .. n_tokens - 1 of sequence slot `seq`;
 * release  = drop_sequence (:362-375): the slot's pages return to the pool (oxb_hip_model_reset releases every slot);
 * pool     = BlockPool::free_count / total_count (:138-146); capacity = BlockTable::token_capacity (:233-236). */
typedef struct { uint32_t page_size, total_pages, free_pages; } oxb_kv_pool_info;
int  oxb_hip_model_kv_reserve(uint64_t model, uint32_t seq, uint32_t n_tokens);
int  oxb_hip_model_kv_release(uint64_t model, uint32_t seq);
int  oxb_hip_model_kv_pool(uint64_t model, oxb_kv_pool_info* info);
int  oxb_hip_model_kv_capacity(uint64_t model, uint32_t seq, uint32_t* n_tokens);
/* quantize_row_i8 / quantize_row_fp8 on the device for n_rows rows of n values each (host buffers): the same
 * routine the attention kernels store new rows with. */
int  oxb_hip_kv_quantize_rows(int kv_dtype, const float* rows, uint32_t n_rows, uint32_t n, uint8_t* codes, float* scales);
/* The way back, code * scale (dequantize_row, crates/oxibonsai-model/src/kv_cache_quant.rs:69-71, 545-556; fp8_e4m3_decode,
 * crates/oxibonsai-core/src/quant_fp8.rs), with the widening of the codes that the attention kernels use; n % 4 == 0. */
int  oxb_hip_kv_dequantize_rows(int kv_dtype, const uint8_t* codes, const float* scales, uint32_t n_rows, uint32_t n, float* rows);

/* ---- the steps either side of the fused forward: checkpoint file -> device, token ids in, token ids out.
 * oxb_hip_gguf_info (no GPU needed) and oxb_hip_load_gguf read a GGUF file the way GgufFile::parse does
 * (crates/oxibonsai-core/src/gguf/reader.rs:11-80, header.rs, metadata.rs, tensor_info.rs) and assemble the model
 * the way BonsaiModel::from_gguf does (crates/oxibonsai-model/src/model/types/mod.rs:71-160; tensor names
 * gguf/tensor_info.rs:211-230; configuration keys crates/oxibonsai-core/src/config.rs:41-118 with head_dim =
 * hidden / heads and the vocabulary taken from token_embd's shape; norm vectors F32 or F16 widened,
 * model/weight_loaders.rs:24-46; shapes in GGUF order [in, out]).  Every projection matrix and output.weight must be
 * Q1_0_g128 (type 41) or TQ2_0_g128 (type 42), one format for the whole file; anything else is InvalidArgument. */
typedef struct {
    uint32_t version, alignment;
    uint64_t n_tensors, n_metadata;
    int fmt;                        /* OXB_HIP_FMT_* of the projection matrices (type of blk.0.attn_q.weight) */
    int embedding_type;             /* GGUF type id of token_embd.weight: 0 F32, 1 F16, 41 Q1_0_g128, 42 TQ2_0_g128 */
    uint32_t n_layers, h, inter, nq, nkv, hd, vocab, context_length;
    float eps, rope_theta;
    char architecture[32], name[64];
    uint32_t lm_head_rows;          /* rows of output.weight = logits per position (model/weight_loaders.rs:654-666); `vocab` counts the rows of token_embd.weight */
} oxb_gguf_info;
int  oxb_hip_gguf_info(const char* path, oxb_gguf_info* info);
/* Directory access without a GPU: one metadata value rendered as text (integers, floats with %.9g, strings as they
 * are, bools as true/false, arrays as "[<count> x type <id>]"), and one tensor's entry (GGUF type id, shape in file
 * order, absolute file offset of its data = data section start + tensor offset, byte size; size 0 for a type this
 * tier does not read).  A missing key / tensor is OXB_HIP_WEIGHT_NOT_FOUND (BonsaiError::TensorNotFound,
 * gguf/tensor_info.rs:86-91). */
int  oxb_hip_gguf_metadata(const char* path, const char* key, char* out, size_t out_cap);
int  oxb_hip_gguf_tensor(const char* path, const char* name, int* type, uint32_t* n_dims, uint64_t shape4[4],
                         uint64_t* file_offset, uint64_t* n_bytes);
/* Uploads every tensor, creates the model (max_seq == 0: the file's context length) and the embedding table.  The
 * model owns its weights: oxb_hip_model_destroy frees them; the embedding is freed with oxb_hip_free_embedding. */
int  oxb_hip_load_gguf(const char* path, uint32_t max_seq, uint32_t batch, uint64_t* model, uint64_t* embedding,
                       oxb_gguf_info* info_or_null);
/* Token embedding table kept on the device in its stored form: vocab rows of h values, gguf_type 0 (F32), 1 (F16),
 * 41 or 42 (rows of h/128 blocks); a row is widened / dequantised when it is looked up, with the values
 * load_f32_tensor produces (model/weight_loaders.rs:24-86). */
int  oxb_hip_upload_embedding(uint64_t* id, const void* table, size_t n_bytes, int gguf_type, uint32_t vocab, uint32_t h);
int  oxb_hip_free_embedding(uint64_t id);
int  oxb_hip_embedding_rows(uint64_t embedding, const uint32_t* ids, uint32_t n, float* out);   /* out: [n][h] */
/* Greedy decode without a host round trip per token: the embedding row copy that precedes the forward
 * (model/types/mod.rs:647-658) and the argmax that follows it (temperature 0, crates/oxibonsai-runtime/src/sampling.rs:182)
 * stay on the device.  tokens[batch] are the ids to feed at pos[batch]; n_steps forwards run back to back, each
 * feeding the previous step's argmax; tokens_out[n_steps][batch] receives every step's ids. */
int  oxb_hip_decode_tokens(uint64_t model, uint64_t embedding, const uint32_t* tokens, const uint32_t* pos,
                           uint32_t n_steps, uint32_t* tokens_out);
/* The same loop with Sampler::sample (crates/oxibonsai-runtime/src/sampling.rs:84-177) on the device instead of the
 * argmax: v / temperature, the top_k largest, softmax, top-p cut with renormalisation, one xorshift64 draw
 * (sampling.rs:73-80) per step and sequence, cumulative pick.  rng_state[batch] holds one generator state per
 * sequence (the reference's Sampler seed) and is advanced in place.  temperature < 1e-6 is the greedy loop (the
 * device argmax keeps the FIRST maximum, the reference's host argmax the last; they differ only on exact ties).
 * With 1 <= top_k <= 128 the device sampler works on the candidates in descending order, where the reference
 * keeps whatever order its partial selection leaves when top_p == 1 (its pick is then an equally valid draw from
 * the same distribution, not the same token).  top_k = 0 or >= vocab switches the filter off as in the reference
 * (sampling.rs:111; the Creative preset): the whole vocabulary in index order, every f32 sum taken element by
 * element in the reference's order, a stable descending sort for top-p.  A top_k between 129 and vocab - 1 sorts
 * the whole row (descending, stable) and continues with its first top_k entries in that order.  Repetition penalty
 * is not part of Sampler::sample. */
typedef struct { float temperature; uint32_t top_k; float top_p; } oxb_sampling;
int  oxb_hip_decode_tokens_sampled(uint64_t model, uint64_t embedding, const uint32_t* tokens, const uint32_t* pos,
                                   uint32_t n_steps, const oxb_sampling* params, uint64_t* rng_state, uint32_t* tokens_out);
/* The sampler alone on host logits [batch][vocab] (vocab <= 524288). */
int  oxb_hip_sample_logits(const float* logits, uint32_t vocab, uint32_t batch, const oxb_sampling* params,
                           uint64_t* rng_state, uint32_t* tokens_out);
/* oxb_hip_prefill with the embedding rows gathered on the device from token ids. */
int  oxb_hip_prefill_tokens(uint64_t model, uint64_t embedding, uint32_t seq, const uint32_t* ids, uint32_t n_tokens,
                            uint32_t pos_start, float* logits_or_null, uint32_t* token_out_or_null);

/* ---- host-only helpers (no GPU needed): the upload-time repack, exposed so it can be checked on any machine.
 * reformat_q1_aos_to_soa / reformat_tq2_blocks_to_soa (KG/cuda_graph/cudagraph_reformat_*_group.rs). */
int  oxb_hip_repack_sizes(int fmt, uint32_t n_rows, uint32_t k, size_t* codes_bytes, size_t* scales_bytes);
int  oxb_hip_repack(int fmt, const uint8_t* aos, size_t n_bytes, uint32_t n_rows, uint32_t k,
                    uint8_t* codes, size_t codes_cap, uint8_t* scales, size_t scales_cap);
int  oxb_hip_unpack(int fmt, const uint8_t* codes, size_t codes_len, const uint8_t* scales, size_t scales_len,
                    uint32_t n_rows, uint32_t k, uint8_t* aos, size_t aos_cap);

#ifdef __cplusplus
}
#endif
#endif /* OXB_HIP_H */
