//! Batched prefill with the argument lists of `try_cuda_prefill` / `try_cuda_prefill_ternary`
//! (gpu_backend/cuda_prefill/try_apis.rs:42-66, 318-342).  The prefill fills the KV cache of the same process-wide
//! model the decode entry points of `full_forward.rs` read, so `forward_prefill` followed by `forward` continues as
//! with the CUDA tier.

use core::ffi::c_int;

use super::ffi::{self, check_graph};
use super::full_forward::{views_q1, views_ternary, with_model, HipFullForwardLayerParams, HipFullForwardLayerParamsTernary, LayerView};
use super::HipGraphError;

#[allow(clippy::too_many_arguments)]
fn prefill(
    fmt: c_int,
    hidden_batch: &[f32],
    batch_size: usize,
    pos_start: usize,
    n_layers: usize,
    layers: &[LayerView<'_>],
    cos_table: &[f32],
    sin_table: &[f32],
    hidden_size: usize,
    intermediate_size: usize,
    nq: usize,
    nkv: usize,
    head_dim: usize,
    heads_per_group: usize,
    eps: f32,
    max_seq_len: usize,
    final_norm_handle: Option<u64>,
    final_norm_bytes: Option<&[f32]>,
    final_norm_eps: f32,
    lm_head_handle: Option<u64>,
    lm_head_bytes: Option<&[u8]>,
    lm_head_out_features: usize,
    logits_out: Option<&mut Vec<f32>>,
    greedy_token_id_out: Option<&mut u32>,
) -> Result<(), HipGraphError> {
    // the checks of try_cuda_prefill, in its order (try_apis.rs:67-98)
    if layers.len() != n_layers {
        return Err(HipGraphError::WeightLayoutError(format!("layer_params length mismatch: need {n_layers}, got {}", layers.len())));
    }
    let half_dim = head_dim / 2;
    if hidden_batch.len() < batch_size * hidden_size {
        return Err(HipGraphError::WeightLayoutError(format!(
            "hidden_batch too short: need {}, got {}",
            batch_size * hidden_size,
            hidden_batch.len()
        )));
    }
    if cos_table.len() < batch_size * half_dim {
        return Err(HipGraphError::WeightLayoutError(format!("cos_table too short: need {}, got {}", batch_size * half_dim, cos_table.len())));
    }
    if sin_table.len() < batch_size * half_dim {
        return Err(HipGraphError::WeightLayoutError(format!("sin_table too short: need {}, got {}", batch_size * half_dim, sin_table.len())));
    }
    if nkv == 0 || heads_per_group != nq / nkv {
        return Err(HipGraphError::WeightLayoutError(format!("heads_per_group {heads_per_group} is not nq / nkv = {nq} / {nkv}")));
    }
    if batch_size == 0 {
        return Ok(());
    }
    // the library applies one epsilon to every norm; the reference's callers pass the same value twice
    if final_norm_bytes.is_some() && final_norm_eps != eps {
        return Err(HipGraphError::WeightLayoutError(format!("final_norm_eps {final_norm_eps} differs from the layers' eps {eps}")));
    }
    let final_norm = match (final_norm_handle, final_norm_bytes) {
        (Some(id), Some(w)) => Some((id, w)),
        _ => None,
    };
    let lm_head = match (lm_head_handle, lm_head_bytes, final_norm) {
        (Some(id), Some(bytes), Some(_)) => Some((id, bytes, lm_head_out_features)),
        _ => None,
    };
    let wants_output = logits_out.is_some() || greedy_token_id_out.is_some();
    if wants_output && lm_head.is_none() {
        return Err(HipGraphError::WeightLayoutError("logits or a token were asked for without final norm and LM head".into()));
    }
    let to_u32 = |v: usize| u32::try_from(v).map_err(|_| HipGraphError::WeightLayoutError(format!("{v} does not fit 32 bits")));
    let (n_tokens, p0) = (to_u32(batch_size)?, to_u32(pos_start)?);
    with_model(fmt, layers, nq, nkv, head_dim, hidden_size, intermediate_size, max_seq_len, eps, final_norm, lm_head, |model| {
        // SAFETY: both tables hold batch_size rows of head_dim / 2 values (checked above).
        check_graph(unsafe { ffi::oxb_hip_model_set_rope_rows(model, p0, n_tokens, cos_table.as_ptr(), sin_table.as_ptr()) }, 0)?;
        let logits_ptr = match logits_out {
            Some(v) => {
                v.clear();
                v.resize(lm_head_out_features, 0.0);
                v.as_mut_ptr()
            }
            None => core::ptr::null_mut(),
        };
        let token_ptr = greedy_token_id_out.map_or(core::ptr::null_mut(), |t| t as *mut u32);
        // SAFETY: hidden_batch holds batch_size * hidden_size values; the output pointers are null or sized above.
        check_graph(unsafe { ffi::oxb_hip_prefill(model, 0, hidden_batch.as_ptr(), n_tokens, p0, logits_ptr, token_ptr) }, 0)
    })
}

/// Batch prefill (all layers, then final norm + LM head of the last token) for Q1 models.  Only the last token's
/// logits are returned in `logits_out` / `greedy_token_id_out`.
#[allow(clippy::too_many_arguments)]
pub fn try_hip_prefill(
    hidden_batch: &[f32],
    batch_size: usize,
    pos_start: usize,
    n_layers: usize,
    layer_params: &[HipFullForwardLayerParams<'_>],
    cos_table: &[f32],
    sin_table: &[f32],
    hidden_size: usize,
    intermediate_size: usize,
    nq: usize,
    nkv: usize,
    head_dim: usize,
    heads_per_group: usize,
    eps: f32,
    max_seq_len: usize,
    final_norm_handle: Option<u64>,
    final_norm_bytes: Option<&[f32]>,
    final_norm_eps: f32,
    lm_head_handle: Option<u64>,
    lm_head_bytes: Option<&[u8]>,
    lm_head_out_features: usize,
    logits_out: Option<&mut Vec<f32>>,
    greedy_token_id_out: Option<&mut u32>,
) -> Result<(), HipGraphError> {
    let views = views_q1(layer_params);
    prefill(ffi::OXB_HIP_FMT_Q1, hidden_batch, batch_size, pos_start, n_layers, &views, cos_table, sin_table, hidden_size,
            intermediate_size, nq, nkv, head_dim, heads_per_group, eps, max_seq_len, final_norm_handle, final_norm_bytes,
            final_norm_eps, lm_head_handle, lm_head_bytes, lm_head_out_features, logits_out, greedy_token_id_out)
}

/// `try_hip_prefill` for TQ2 ternary models.
#[allow(clippy::too_many_arguments)]
pub fn try_hip_prefill_ternary(
    hidden_batch: &[f32],
    batch_size: usize,
    pos_start: usize,
    n_layers: usize,
    layer_params: &[HipFullForwardLayerParamsTernary<'_>],
    cos_table: &[f32],
    sin_table: &[f32],
    hidden_size: usize,
    intermediate_size: usize,
    nq: usize,
    nkv: usize,
    head_dim: usize,
    heads_per_group: usize,
    eps: f32,
    max_seq_len: usize,
    final_norm_handle: Option<u64>,
    final_norm_bytes: Option<&[f32]>,
    final_norm_eps: f32,
    lm_head_handle: Option<u64>,
    lm_head_bytes: Option<&[u8]>,
    lm_head_out_features: usize,
    logits_out: Option<&mut Vec<f32>>,
    greedy_token_id_out: Option<&mut u32>,
) -> Result<(), HipGraphError> {
    let views = views_ternary(layer_params);
    prefill(ffi::OXB_HIP_FMT_TQ2, hidden_batch, batch_size, pos_start, n_layers, &views, cos_table, sin_table, hidden_size,
            intermediate_size, nq, nkv, head_dim, heads_per_group, eps, max_seq_len, final_norm_handle, final_norm_bytes,
            final_norm_eps, lm_head_handle, lm_head_bytes, lm_head_out_features, logits_out, greedy_token_id_out)
}
