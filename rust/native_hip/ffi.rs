//! `extern "C"` declarations of `include/oxb_hip.h`, one for one, and the mapping of its status codes.
//!
//! Linking (crates/oxibonsai-kernels/build.rs, under `CARGO_FEATURE_NATIVE_HIP`):
//!
//! ```ignore
//! let dir = std::env::var("OXB_HIP_LIB_DIR").expect("OXB_HIP_LIB_DIR = directory holding liboxb_hip.a");
//! println!("cargo:rustc-link-search=native={dir}");
//! println!("cargo:rustc-link-lib=static=oxb_hip");
//! println!("cargo:rustc-link-search=native=/opt/rocm/lib");
//! println!("cargo:rustc-link-lib=dylib=amdhip64");
//! println!("cargo:rustc-link-lib=dylib=stdc++");
//! ```
//!
//! and in Cargo.toml: `native-hip = ["gpu"]` (no new Rust dependency).

use core::ffi::{c_char, c_int, c_void};

use super::super::GpuError;
use super::HipGraphError;

pub const OXB_HIP_OK: c_int = 0;
pub const OXB_HIP_NOT_AVAILABLE: c_int = 1;
pub const OXB_HIP_OUT_OF_MEMORY: c_int = 2;
pub const OXB_HIP_KERNEL_LAUNCH: c_int = 3;
pub const OXB_HIP_SYNC_FAILED: c_int = 4;
pub const OXB_HIP_INVALID_ARGUMENT: c_int = 5;
pub const OXB_HIP_WEIGHT_NOT_FOUND: c_int = 6;

pub const OXB_HIP_FMT_Q1: c_int = 0;
pub const OXB_HIP_FMT_TQ2: c_int = 1;

#[repr(C)]
#[derive(Clone, Copy, Default)]
pub struct OxbLayerIds {
    pub attn_norm: u64,
    pub qkv: u64,
    pub q_norm: u64,
    pub k_norm: u64,
    pub o: u64,
    pub ffn_norm: u64,
    pub gate_up: u64,
    pub down: u64,
}

#[repr(C)]
pub struct OxbModelDesc {
    pub fmt: c_int,
    pub n_layers: u32,
    pub h: u32,
    pub inter: u32,
    pub nq: u32,
    pub nkv: u32,
    pub hd: u32,
    pub vocab: u32,
    pub max_seq: u32,
    pub batch: u32,
    pub eps: f32,
    pub rope_theta: f32,
    pub layers: *const OxbLayerIds,
    pub final_norm: u64,
    pub lm_head: u64,
}

#[repr(C)]
pub struct OxbAttentionOptions {
    pub kv_dtype: i32,
    pub window_size: u32,
    pub sink_tokens: u32,
    pub page_size: u32,
    pub n_pages: u32,
}

#[repr(C)]
pub struct OxbKvPoolInfo {
    pub page_size: u32,
    pub total_pages: u32,
    pub free_pages: u32,
}

#[repr(C)]
pub struct OxbSampling {
    pub temperature: f32,
    pub top_k: u32,
    pub top_p: f32,
}

#[repr(C)]
pub struct OxbGgufInfo {
    pub version: u32,
    pub alignment: u32,
    pub n_tensors: u64,
    pub n_metadata: u64,
    pub fmt: c_int,
    pub embedding_type: c_int,
    pub n_layers: u32,
    pub h: u32,
    pub inter: u32,
    pub nq: u32,
    pub nkv: u32,
    pub hd: u32,
    pub vocab: u32,
    pub context_length: u32,
    pub eps: f32,
    pub rope_theta: f32,
    pub architecture: [c_char; 32],
    pub name: [c_char; 64],
    pub lm_head_rows: u32,
}

extern "C" {
    // lifecycle
    pub fn oxb_hip_init(device_ordinal: c_int) -> c_int;
    pub fn oxb_hip_shutdown();
    pub fn oxb_hip_device_count() -> c_int;
    pub fn oxb_hip_device_info(name: *mut c_char, name_cap: usize, free_bytes: *mut usize, total_bytes: *mut usize) -> c_int;
    pub fn oxb_hip_synchronize() -> c_int;
    pub fn oxb_hip_set_stream(hip_stream: *mut c_void) -> c_int;
    pub fn oxb_hip_last_error() -> *const c_char;
    // weights
    pub fn oxb_hip_upload_q1(id: *mut u64, aos: *const u8, n_bytes: usize, n_rows: u32, k: u32) -> c_int;
    pub fn oxb_hip_upload_tq2(id: *mut u64, aos: *const u8, n_bytes: usize, n_rows: u32, k: u32) -> c_int;
    pub fn oxb_hip_upload_q1_raw(id: *mut u64, aos: *const u8, n_bytes: usize) -> c_int;
    pub fn oxb_hip_upload_tq2_raw(id: *mut u64, aos: *const u8, n_bytes: usize) -> c_int;
    pub fn oxb_hip_free_weight(id: u64) -> c_int;
    pub fn oxb_hip_weight_info(id: u64, fmt: *mut c_int, n_rows: *mut u32, k: *mut u32, resident_bytes: *mut usize) -> c_int;
    pub fn oxb_hip_dequant(id: u64, out: *mut f32, out_len: usize) -> c_int;
    // GEMV / GEMM
    pub fn oxb_hip_gemv(id: u64, x: *const f32, y: *mut f32, n_rows: u32, k: u32, batch: u32) -> c_int;
    pub fn oxb_hip_gemv_dev(id: u64, d_x: *const f32, d_y: *mut f32, n_rows: u32, k: u32, batch: u32) -> c_int;
    pub fn oxb_hip_gemv_q1_g128(aos: *const u8, n_bytes: usize, x: *const f32, x_len: usize, y: *mut f32, y_len: usize,
                                n_rows: u32, k: u32) -> c_int;
    pub fn oxb_hip_gemv_tq2_g128(aos: *const u8, n_bytes: usize, x: *const f32, x_len: usize, y: *mut f32, y_len: usize,
                                 n_rows: u32, k: u32) -> c_int;
    pub fn oxb_hip_gemm(id: u64, x: *const f32, y: *mut f32, m: u32, n_rows: u32, k: u32) -> c_int;
    pub fn oxb_hip_gemm_dev(id: u64, d_x: *const f32, d_y: *mut f32, m: u32, n_rows: u32, k: u32) -> c_int;
    /// No allocation inside the call (for callers under graph capture or in loops that must not call hipMalloc):
    /// scratch is a 32 MiB array inside the library, larger shapes are `InvalidArgument`, overlapping calls race.
    pub fn oxb_hip_gemm_dev_static(id: u64, d_x: *const f32, d_y: *mut f32, m: u32, n_rows: u32, k: u32) -> c_int;
    // batched phases
    pub fn oxb_hip_attn_phase(fmt: c_int, hidden: *const f32, norm_w: *const f32, eps: f32, qkv_id: u64, q_rows: u32,
                              k_rows: u32, h: u32, q: *mut f32, k: *mut f32, v: *mut f32) -> c_int;
    pub fn oxb_hip_ffn_phase(fmt: c_int, hidden: *mut f32, attn_out: *const f32, norm_w: *const f32, eps: f32, o_id: u64,
                             gate_up_id: u64, down_id: u64, h: u32, inter: u32, attn_k: u32) -> c_int;
    // fused model
    pub fn oxb_hip_upload_f32(id: *mut u64, w: *const f32, n: usize) -> c_int;
    pub fn oxb_hip_free_f32(id: u64) -> c_int;
    pub fn oxb_hip_model_create(desc: *const OxbModelDesc, model: *mut u64) -> c_int;
    pub fn oxb_hip_model_reset(model: u64) -> c_int;
    pub fn oxb_hip_model_destroy(model: u64) -> c_int;
    pub fn oxb_hip_decode(model: u64, hidden: *const f32, pos: *const u32, logits_or_null: *mut f32, token_out: *mut u32) -> c_int;
    pub fn oxb_hip_decode_hidden(model: u64, hidden: *const f32, pos: *const u32, normed_out: *mut f32) -> c_int;
    pub fn oxb_hip_model_set_lm_head(model: u64, final_norm: u64, lm_head: u64, vocab: u32) -> c_int;
    pub fn oxb_hip_model_set_rope_rows(model: u64, pos_start: u32, n_pos: u32, cos_rows: *const f32, sin_rows: *const f32) -> c_int;
    pub fn oxb_hip_prefill(model: u64, seq: u32, hidden: *const f32, n_tokens: u32, pos_start: u32,
                           logits_or_null: *mut f32, token_out_or_null: *mut u32) -> c_int;
    pub fn oxb_hip_model_uses_graph(model: u64) -> c_int;
    // long-context options
    pub fn oxb_hip_model_set_attention(model: u64, opt: *const OxbAttentionOptions) -> c_int;
    pub fn oxb_hip_model_get_attention(model: u64, opt: *mut OxbAttentionOptions) -> c_int;
    pub fn oxb_hip_model_read_kv(model: u64, seq: u32, layer: u32, kv_head: u32, pos: u32, n_pos: u32, k_rows: *mut c_void,
                                 v_rows: *mut c_void, k_scales: *mut f32, v_scales: *mut f32) -> c_int;
    pub fn oxb_hip_model_kv_reserve(model: u64, seq: u32, n_tokens: u32) -> c_int;
    pub fn oxb_hip_model_kv_release(model: u64, seq: u32) -> c_int;
    pub fn oxb_hip_model_kv_pool(model: u64, info: *mut OxbKvPoolInfo) -> c_int;
    pub fn oxb_hip_model_kv_capacity(model: u64, seq: u32, n_tokens: *mut u32) -> c_int;
    pub fn oxb_hip_kv_quantize_rows(kv_dtype: c_int, rows: *const f32, n_rows: u32, n: u32, codes: *mut u8, scales: *mut f32) -> c_int;
    pub fn oxb_hip_kv_dequantize_rows(kv_dtype: c_int, codes: *const u8, scales: *const f32, n_rows: u32, n: u32, rows: *mut f32) -> c_int;
    // checkpoint file, token ids
    pub fn oxb_hip_gguf_info(path: *const c_char, info: *mut OxbGgufInfo) -> c_int;
    pub fn oxb_hip_gguf_metadata(path: *const c_char, key: *const c_char, out: *mut c_char, out_cap: usize) -> c_int;
    pub fn oxb_hip_gguf_tensor(path: *const c_char, name: *const c_char, ty: *mut c_int, n_dims: *mut u32, shape4: *mut u64,
                               file_offset: *mut u64, n_bytes: *mut u64) -> c_int;
    pub fn oxb_hip_load_gguf(path: *const c_char, max_seq: u32, batch: u32, model: *mut u64, embedding: *mut u64,
                             info_or_null: *mut OxbGgufInfo) -> c_int;
    pub fn oxb_hip_upload_embedding(id: *mut u64, table: *const c_void, n_bytes: usize, gguf_type: c_int, vocab: u32, h: u32) -> c_int;
    pub fn oxb_hip_free_embedding(id: u64) -> c_int;
    pub fn oxb_hip_embedding_rows(embedding: u64, ids: *const u32, n: u32, out: *mut f32) -> c_int;
    pub fn oxb_hip_decode_tokens(model: u64, embedding: u64, tokens: *const u32, pos: *const u32, n_steps: u32, tokens_out: *mut u32) -> c_int;
    pub fn oxb_hip_decode_tokens_sampled(model: u64, embedding: u64, tokens: *const u32, pos: *const u32, n_steps: u32,
                                         params: *const OxbSampling, rng_state: *mut u64, tokens_out: *mut u32) -> c_int;
    pub fn oxb_hip_sample_logits(logits: *const f32, vocab: u32, batch: u32, params: *const OxbSampling, rng_state: *mut u64,
                                 tokens_out: *mut u32) -> c_int;
    pub fn oxb_hip_prefill_tokens(model: u64, embedding: u64, seq: u32, ids: *const u32, n_tokens: u32, pos_start: u32,
                                  logits_or_null: *mut f32, token_out_or_null: *mut u32) -> c_int;
    // host-only repack helpers
    pub fn oxb_hip_repack_sizes(fmt: c_int, n_rows: u32, k: u32, codes_bytes: *mut usize, scales_bytes: *mut usize) -> c_int;
    pub fn oxb_hip_repack(fmt: c_int, aos: *const u8, n_bytes: usize, n_rows: u32, k: u32, codes: *mut u8, codes_cap: usize,
                          scales: *mut u8, scales_cap: usize) -> c_int;
    pub fn oxb_hip_unpack(fmt: c_int, codes: *const u8, codes_len: usize, scales: *const u8, scales_len: usize, n_rows: u32,
                          k: u32, aos: *mut u8, aos_cap: usize) -> c_int;
}

/// Text of the last failure on this thread.
pub(crate) fn last_error() -> String {
    // SAFETY: the library returns a pointer to a thread-local, NUL-terminated string that stays valid until the
    // next failing call on this thread.
    unsafe { std::ffi::CStr::from_ptr(oxb_hip_last_error()) }.to_string_lossy().into_owned()
}

/// Status code -> `GpuError`, for the trait methods.  `GpuError` has no variant for a missing weight handle; the
/// CUDA tier reports it as `KernelLaunch(e.to_string())` (`cuda_graph/nativecudabackend_traits.rs:90-101`) and so
/// does this one.  The library's messages already start with the variant's prefix ("invalid argument: ..."), which
/// is stripped so that `Display` does not print it twice.
pub(crate) fn check(code: c_int) -> Result<(), GpuError> {
    if code == OXB_HIP_OK {
        return Ok(());
    }
    let msg = last_error();
    let tail = |prefix: &str| msg.strip_prefix(prefix).unwrap_or(&msg).to_string();
    Err(match code {
        OXB_HIP_NOT_AVAILABLE => GpuError::NotAvailable(tail("GPU not available: ")),
        OXB_HIP_OUT_OF_MEMORY => {
            // "out of device memory: requested N bytes on device D"
            let mut nums = msg.split(|c: char| !c.is_ascii_digit()).filter(|s| !s.is_empty()).map(|s| s.parse::<usize>().unwrap_or(0));
            GpuError::OutOfMemory { requested: nums.next().unwrap_or(0), device: nums.next().unwrap_or(0) }
        }
        OXB_HIP_KERNEL_LAUNCH | OXB_HIP_WEIGHT_NOT_FOUND => GpuError::KernelLaunch(tail("kernel launch failed: ")),
        OXB_HIP_SYNC_FAILED => GpuError::SyncFailed(tail("device synchronization failed: ")),
        _ => GpuError::InvalidArgument(tail("invalid argument: ")),
    })
}

/// Status code -> `HipGraphError`, for the fused entry points.  `id` names the handle the call was about.
pub(crate) fn check_graph(code: c_int, id: u64) -> Result<(), HipGraphError> {
    match code {
        OXB_HIP_OK => Ok(()),
        OXB_HIP_NOT_AVAILABLE => Err(HipGraphError::DeviceNotFound(last_error())),
        OXB_HIP_WEIGHT_NOT_FOUND => Err(HipGraphError::WeightNotFound(id)),
        OXB_HIP_INVALID_ARGUMENT => Err(HipGraphError::WeightLayoutError(last_error())),
        _ => Err(HipGraphError::DriverError(last_error())),
    }
}
