//! `NativeHipBackend`: `GpuBackendTrait` (gpu_backend/mod.rs:358-534) over the C ABI.  The twin of
//! `NativeCudaBackend` (gpu_backend/cuda_graph/types.rs:84-97, trait impl nativecudabackend_traits.rs:18-189).

use super::super::{CpuBackend, DeviceBuffer, GpuBackendTrait, GpuError};
use super::ffi::{self, check};
use crate::weight_cache::GpuWeightHandle;

/// Q1_0_g128 / TQ2_0_g128 kernels on one MI355X through `liboxb_hip`.
///
/// Returned by `select_backend` when a gfx950 device is present and the `native-hip` feature is enabled.
pub struct NativeHipBackend {
    /// The dense-f32 helper operations of the trait (`alloc`, `matvec`, `relu`, `softmax`) are not on the
    /// sub-2-bit path; like the CUDA tier this one hands them to the CPU backend.
    cpu_fallback: CpuBackend,
}

impl NativeHipBackend {
    /// Initialise the backend (fails with `NotAvailable` if there is no usable GPU).
    pub fn new() -> Result<Self, GpuError> {
        // SAFETY: plain C call, no pointers.
        check(unsafe { ffi::oxb_hip_init(0) })?;
        Ok(Self { cpu_fallback: CpuBackend::new() })
    }
}

fn dim(v: usize, what: &str) -> Result<u32, GpuError> {
    u32::try_from(v).map_err(|_| GpuError::InvalidArgument(format!("{what} = {v} does not fit 32 bits")))
}

/// The format of a cached weight, for the two batched phases whose trait signatures do not say it.
fn weight_fmt(handle: GpuWeightHandle) -> Result<core::ffi::c_int, GpuError> {
    let mut fmt: core::ffi::c_int = 0;
    // SAFETY: out-pointers are valid or null as the header allows.
    check(unsafe {
        ffi::oxb_hip_weight_info(handle.id(), &mut fmt, core::ptr::null_mut(), core::ptr::null_mut(), core::ptr::null_mut())
    })?;
    Ok(fmt)
}

impl GpuBackendTrait for NativeHipBackend {
    fn name(&self) -> &'static str {
        "native-hip"
    }
    fn is_accelerated(&self) -> bool {
        true
    }
    fn device_count(&self) -> usize {
        1 // the library drives the one device it was initialised on, as the CUDA tier does
    }
    fn alloc(&self, size: usize, device_id: usize) -> Result<DeviceBuffer, GpuError> {
        self.cpu_fallback.alloc(size, device_id)
    }
    fn host_to_device(&self, src: &[f32], device_id: usize) -> Result<DeviceBuffer, GpuError> {
        self.cpu_fallback.host_to_device(src, device_id)
    }
    fn device_to_host(&self, buf: &DeviceBuffer) -> Result<Vec<f32>, GpuError> {
        self.cpu_fallback.device_to_host(buf)
    }
    fn matvec(&self, a: &DeviceBuffer, x: &DeviceBuffer, m: usize, k: usize, device_id: usize) -> Result<DeviceBuffer, GpuError> {
        self.cpu_fallback.matvec(a, x, m, k, device_id)
    }
    fn relu(&self, x: &DeviceBuffer, device_id: usize) -> Result<DeviceBuffer, GpuError> {
        self.cpu_fallback.relu(x, device_id)
    }
    fn softmax(&self, x: &DeviceBuffer, size: usize, device_id: usize) -> Result<DeviceBuffer, GpuError> {
        self.cpu_fallback.softmax(x, size, device_id)
    }
    fn synchronize(&self, _device_id: usize) -> Result<(), GpuError> {
        // SAFETY: plain C call.
        check(unsafe { ffi::oxb_hip_synchronize() })
    }
    fn memory_info(&self, _device_id: usize) -> Result<(usize, usize), GpuError> {
        let (mut free, mut total) = (0usize, 0usize);
        // SAFETY: a null name with capacity 0 is allowed; the two out-pointers are valid.
        check(unsafe { ffi::oxb_hip_device_info(core::ptr::null_mut(), 0, &mut free, &mut total) })?;
        Ok((free, total))
    }

    fn gemv_q1_g128(&self, block_bytes: &[u8], input: &[f32], n_rows: usize, k: usize) -> Result<Vec<f32>, GpuError> {
        let mut y = vec![0.0_f32; n_rows];
        // SAFETY: every pointer comes with the length of its slice; the library checks them against n_rows and k.
        check(unsafe {
            ffi::oxb_hip_gemv_q1_g128(block_bytes.as_ptr(), block_bytes.len(), input.as_ptr(), input.len(), y.as_mut_ptr(),
                                      y.len(), dim(n_rows, "n_rows")?, dim(k, "k")?)
        })?;
        Ok(y)
    }

    fn gemm_q1_g128(&self, block_bytes: &[u8], input: &[f32], m: usize, n_rows: usize, k: usize) -> Result<Vec<f32>, GpuError> {
        if input.len() < m * k {
            return Err(GpuError::InvalidArgument(format!("input holds {} values, {} needed", input.len(), m * k)));
        }
        let handle = self.upload_weights_raw(block_bytes)?;
        let mut y = vec![0.0_f32; m * n_rows];
        // One pass over the weights for all m rows; products stay fp32-exact (the trait's default loops over
        // gemv_q1_g128, whose arithmetic this keeps).  oxb_hip_gemm is the fp16 matrix-core route for prefill.
        // SAFETY: lengths checked above; y holds m * n_rows values.
        let r = check(unsafe {
            ffi::oxb_hip_gemv(handle.id(), input.as_ptr(), y.as_mut_ptr(), dim(n_rows, "n_rows")?, dim(k, "k")?, dim(m, "m")?)
        });
        // SAFETY: plain C call.
        let _ = unsafe { ffi::oxb_hip_free_weight(handle.id()) };
        r.map(|()| y)
    }

    fn upload_weights_raw(&self, block_bytes: &[u8]) -> Result<GpuWeightHandle, GpuError> {
        let mut id = 0u64; // 0: the library allocates the handle (ids from 2^40 up, clear of the model's own)
        // SAFETY: pointer and length of one slice.  The shape is bound by the first call that names it.
        check(unsafe { ffi::oxb_hip_upload_q1_raw(&mut id, block_bytes.as_ptr(), block_bytes.len()) })?;
        Ok(GpuWeightHandle(id))
    }

    fn gemv_q1_g128_cached(&self, handle: GpuWeightHandle, input: &[f32], n_rows: usize, k: usize) -> Result<Vec<f32>, GpuError> {
        if input.len() < k {
            return Err(GpuError::InvalidArgument(format!("input holds {} values, {k} needed", input.len())));
        }
        let mut y = vec![0.0_f32; n_rows];
        // SAFETY: input holds k values, y n_rows.
        check(unsafe { ffi::oxb_hip_gemv(handle.id(), input.as_ptr(), y.as_mut_ptr(), dim(n_rows, "n_rows")?, dim(k, "k")?, 1) })?;
        Ok(y)
    }

    fn upload_weights_ternary(&self, blocks: &[oxibonsai_core::BlockTQ2_0_g128]) -> Result<GpuWeightHandle, GpuError> {
        let mut id = 0u64;
        // BlockTQ2_0_g128 is #[repr(C)] { qs: [u8; 32], d: f16 } = 34 bytes: the byte order the library reads.
        let n_bytes = std::mem::size_of_val(blocks);
        // SAFETY: the slice's own memory, viewed as bytes.
        check(unsafe { ffi::oxb_hip_upload_tq2_raw(&mut id, blocks.as_ptr() as *const u8, n_bytes) })?;
        Ok(GpuWeightHandle(id))
    }

    fn gemv_tq2_g128_cached(&self, handle: GpuWeightHandle, input: &[f32], n_rows: usize, k: usize) -> Result<Vec<f32>, GpuError> {
        self.gemv_q1_g128_cached(handle, input, n_rows, k) // the handle knows its format
    }

    #[allow(clippy::type_complexity)]
    fn batch_attn_phase(&self, hidden: &[f32], norm_weight: &[f32], norm_eps: f32, qkv_handle: GpuWeightHandle, q_rows: usize,
                        k_rows: usize, h: usize) -> Result<Option<(Vec<f32>, Vec<f32>, Vec<f32>)>, GpuError> {
        if hidden.len() < h || norm_weight.len() < h {
            return Err(GpuError::InvalidArgument(format!("hidden / norm_weight shorter than h = {h}")));
        }
        let (mut q, mut k, mut v) = (vec![0.0_f32; q_rows], vec![0.0_f32; k_rows], vec![0.0_f32; k_rows]);
        // SAFETY: lengths checked above; q, k, v hold what the call writes.
        check(unsafe {
            ffi::oxb_hip_attn_phase(weight_fmt(qkv_handle)?, hidden.as_ptr(), norm_weight.as_ptr(), norm_eps, qkv_handle.id(),
                                    dim(q_rows, "q_rows")?, dim(k_rows, "k_rows")?, dim(h, "h")?, q.as_mut_ptr(),
                                    k.as_mut_ptr(), v.as_mut_ptr())
        })?;
        Ok(Some((q, k, v)))
    }

    fn batch_ffn_phase(&self, hidden: &mut [f32], attn_out: &[f32], norm_weight: &[f32], norm_eps: f32,
                       attn_proj_handle: GpuWeightHandle, gate_up_handle: GpuWeightHandle, down_handle: GpuWeightHandle,
                       h: usize, intermediate: usize, attn_proj_k: usize) -> Result<bool, GpuError> {
        if hidden.len() < h || norm_weight.len() < h || attn_out.len() < attn_proj_k {
            return Err(GpuError::InvalidArgument("hidden / norm_weight / attn_out shorter than their dimension".into()));
        }
        // A handle that is not cached means "not batched": the caller takes its per-operation path
        // (nativecudabackend_traits.rs:134-165 returns Ok(false) there as well).
        let fmt = match weight_fmt(attn_proj_handle) {
            Ok(f) => f,
            Err(_) => return Ok(false),
        };
        // SAFETY: lengths checked above.
        let rc = unsafe {
            ffi::oxb_hip_ffn_phase(fmt, hidden.as_mut_ptr(), attn_out.as_ptr(), norm_weight.as_ptr(), norm_eps,
                                   attn_proj_handle.id(), gate_up_handle.id(), down_handle.id(), dim(h, "h")?,
                                   dim(intermediate, "intermediate")?, dim(attn_proj_k, "attn_proj_k")?)
        };
        if rc == ffi::OXB_HIP_WEIGHT_NOT_FOUND {
            return Ok(false);
        }
        check(rc).map(|()| true)
    }
}
