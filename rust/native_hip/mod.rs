//! `native-hip` kernel tier: Q1_0_g128 / TQ2_0_g128 GEMV, GEMM and the fused decode / prefill paths on AMD
//! Instinct MI355X (gfx950) through `liboxb_hip.a` (C ABI: `include/oxb_hip.h`).
//!
//! Drop this directory into `crates/oxibonsai-kernels/src/gpu_backend/native_hip/` and add to
//! `gpu_backend/mod.rs`, beside the `cuda_*` modules (mod.rs:49-99, re-exports :153-170):
//!
//! ```ignore
//! #[cfg(all(feature = "native-hip", target_os = "linux"))]
//! pub mod native_hip;
//! #[cfg(all(feature = "native-hip", target_os = "linux"))]
//! pub use native_hip::{
//!     try_hip_ffn, try_hip_full_forward, try_hip_full_forward_ternary,
//!     try_hip_full_forward_ternary_with_gpu_lm_head, try_hip_full_forward_with_gpu_lm_head, try_hip_prefill,
//!     try_hip_prefill_ternary, try_hip_qkv, HipFullForwardLayerParams, HipFullForwardLayerParamsTernary,
//!     HipGraphError, NativeHipBackend,
//! };
//! ```
//!
//! and in `select_backend()` (mod.rs:1051-1136), between the scirs2 arm (:1068-1090) and the native CUDA arm
//! (:1092-1106):
//!
//! ```ignore
//! #[cfg(all(feature = "native-hip", target_os = "linux"))]
//! {
//!     match NativeHipBackend::new() {
//!         Ok(b) => {
//!             tracing::info!("select_backend: NativeHipBackend initialised");
//!             return Box::new(b);
//!         }
//!         Err(e) => {
//!             warn!("select_backend: NativeHipBackend init failed ({e}), trying next");
//!         }
//!     }
//! }
//! ```
//!
//! Every function here has the name, argument list and return type of its `cuda` counterpart, so the model crate's
//! call sites (`crates/oxibonsai-model/src/model/types/forward_cuda/q1.rs`, `ternary.rs`) switch tiers by a `cfg`
//! on the function name alone.  The one type that differs is the error of the prefill entry points
//! (`try_cuda_prefill` returns `Result<(), CudaGraphError>`, `cuda_prefill/try_apis.rs:318-342`): the model crate only
//! formats it (`forward_cuda/q1.rs` logs `{e}` and falls back), and for code that does name the type this module
//! converts (`From<HipGraphError> for CudaGraphError`, when both tiers are compiled in) or, in a build without the
//! CUDA tier, offers the HIP error under the CUDA name (`pub use native_hip::CudaGraphError`).

pub mod backend;
pub mod ffi;
pub mod full_forward;
pub mod prefill;

pub use backend::NativeHipBackend;
pub use full_forward::{
    try_hip_ffn, try_hip_full_forward, try_hip_full_forward_ternary,
    try_hip_full_forward_ternary_with_gpu_lm_head, try_hip_full_forward_with_gpu_lm_head, try_hip_qkv,
    HipFullForwardLayerParams, HipFullForwardLayerParamsTernary,
};
pub use prefill::{try_hip_prefill, try_hip_prefill_ternary};

/// Errors of the fused entry points; the variants of `CudaGraphError`
/// (`gpu_backend/cuda_graph/types.rs:25-39`) that can occur without a run-time compiler.
#[derive(Debug)]
pub enum HipGraphError {
    /// No gfx950 device, or the HIP runtime is not present (`OXB_HIP_NOT_AVAILABLE`).
    DeviceNotFound(String),
    /// HIP runtime error: allocation, launch or synchronisation (`OXB_HIP_OUT_OF_MEMORY`, `_KERNEL_LAUNCH`, `_SYNC_FAILED`).
    DriverError(String),
    /// A requested weight handle was not found in the library's cache (`OXB_HIP_WEIGHT_NOT_FOUND`).
    WeightNotFound(u64),
    /// Lengths or dimensions do not fit together (`OXB_HIP_INVALID_ARGUMENT`).
    WeightLayoutError(String),
    /// A mutex was poisoned.
    LockPoisoned,
}

/// Both tiers compiled in: a `?` in code written against the CUDA tier's error type takes a HIP error as it is.
/// Every variant has its namesake in `CudaGraphError` (`gpu_backend/cuda_graph/types.rs:25-39`).
#[cfg(all(feature = "native-cuda", any(target_os = "linux", target_os = "windows")))]
impl From<HipGraphError> for super::cuda_graph::CudaGraphError {
    fn from(e: HipGraphError) -> Self {
        use super::cuda_graph::CudaGraphError as C;
        match e {
            HipGraphError::DeviceNotFound(s) => C::DeviceNotFound(s),
            HipGraphError::DriverError(s) => C::DriverError(s),
            HipGraphError::WeightNotFound(id) => C::WeightNotFound(id),
            HipGraphError::WeightLayoutError(s) => C::WeightLayoutError(s),
            HipGraphError::LockPoisoned => C::LockPoisoned,
        }
    }
}

/// Without the CUDA tier the name `CudaGraphError` is free: call sites that spell it keep compiling.
#[cfg(not(all(feature = "native-cuda", any(target_os = "linux", target_os = "windows"))))]
pub type CudaGraphError = HipGraphError;

impl std::fmt::Display for HipGraphError {
    fn fmt(&self, f: &mut std::fmt::Formatter<'_>) -> std::fmt::Result {
        match self {
            Self::DeviceNotFound(s) => write!(f, "HIP device not found: {s}"),
            Self::DriverError(s) => write!(f, "HIP driver error: {s}"),
            Self::WeightNotFound(id) => write!(f, "weight handle {id} not found in cache"),
            Self::WeightLayoutError(s) => write!(f, "weight layout error: {s}"),
            Self::LockPoisoned => write!(f, "mutex lock poisoned"),
        }
    }
}

impl std::error::Error for HipGraphError {}
