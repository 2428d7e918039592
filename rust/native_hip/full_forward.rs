//! The fused entry points the model crate calls, with the argument lists of their CUDA counterparts:
//!
//! | here                                            | reference                                                                  |
//! |-------------------------------------------------|----------------------------------------------------------------------------|
//! | `HipFullForwardLayerParams`                     | `CudaFullForwardLayerParams`, cuda_full_layer/mod.rs:250-268               |
//! | `HipFullForwardLayerParamsTernary`              | `CudaFullForwardLayerParamsTernary`, cuda_full_layer/encode_ternary.rs:62-97 |
//! | `try_hip_full_forward`                          | `try_cuda_full_forward`, cuda_full_layer/encode_q1.rs:813-830              |
//! | `try_hip_full_forward_with_gpu_lm_head`         | `try_cuda_full_forward_with_gpu_lm_head`, encode_q1.rs:881-900             |
//! | `try_hip_full_forward_ternary`                  | `try_cuda_full_forward_ternary`, encode_ternary.rs:694-711                 |
//! | `try_hip_full_forward_ternary_with_gpu_lm_head` | `try_cuda_full_forward_ternary_with_gpu_lm_head`, encode_ternary.rs:755-774 |
//! | `try_hip_ffn`                                   | `try_cuda_ffn`, cuda_graph/functions.rs:76-115                             |
//! | `try_hip_qkv`                                   | `try_cuda_qkv`, cuda_graph/functions.rs:124-145                            |
//!
//! Call sites: crates/oxibonsai-model/src/model/types/forward_cuda/q1.rs:148-165 (layers only), :284-303 (Q1 with
//! LM head), :204-223 (ternary with LM head).
//!
//! One process-wide model lives behind a mutex, as the CUDA tier keeps one `CudaGraph` with its KV cache and
//! cached layer weights (cuda_full_layer/mod.rs:112-139, get_or_build_model_weights).  Weights are uploaded on
//! the first call under the caller's handle ids and found by id afterwards.

use std::sync::Mutex;

use core::ffi::c_int;
use tracing::warn;

use super::ffi::{self, check_graph, OxbLayerIds, OxbModelDesc};
use super::HipGraphError;

/// Per-layer parameters of the Q1 full-forward path (field for field `CudaFullForwardLayerParams`).
pub struct HipFullForwardLayerParams<'a> {
    pub attn_norm_handle: u64,
    pub attn_norm_bytes: &'a [f32],
    /// Handle of the fused Q‖K‖V weight; `fused_qkv_bytes` are its Q1_0_g128 blocks, 18 bytes each.
    pub fused_qkv_handle: u64,
    pub fused_qkv_bytes: &'a [u8],
    pub q_norm_handle: u64,
    pub q_norm_bytes: &'a [f32],
    pub k_norm_handle: u64,
    pub k_norm_bytes: &'a [f32],
    pub attn_proj_handle: u64,
    pub attn_proj_bytes: &'a [u8],
    pub ffn_norm_handle: u64,
    pub ffn_norm_bytes: &'a [f32],
    /// Handle of the fused gate‖up weight: `gate_bytes` followed by `up_bytes`.
    pub gate_up_handle: u64,
    pub gate_bytes: &'a [u8],
    pub up_bytes: &'a [u8],
    pub down_handle: u64,
    pub down_bytes: &'a [u8],
}

/// The same for TQ2_0_g128 weights, 34 bytes per block (field for field `CudaFullForwardLayerParamsTernary`).
pub struct HipFullForwardLayerParamsTernary<'a> {
    pub attn_norm_handle: u64,
    pub attn_norm_bytes: &'a [f32],
    pub fused_qkv_handle: u64,
    pub fused_qkv_bytes: &'a [u8],
    pub q_norm_handle: u64,
    pub q_norm_bytes: &'a [f32],
    pub k_norm_handle: u64,
    pub k_norm_bytes: &'a [f32],
    pub attn_proj_handle: u64,
    pub attn_proj_bytes: &'a [u8],
    pub ffn_norm_handle: u64,
    pub ffn_norm_bytes: &'a [f32],
    pub gate_up_handle: u64,
    pub gate_bytes: &'a [u8],
    pub up_bytes: &'a [u8],
    pub down_handle: u64,
    pub down_bytes: &'a [u8],
}

/// What both parameter structs say, format aside.
pub(super) struct LayerView<'a> {
    pub vecs: [(u64, &'a [f32]); 4], // attn_norm, q_norm, k_norm, ffn_norm
    pub qkv: (u64, &'a [u8]),
    pub o: (u64, &'a [u8]),
    pub gate_up: (u64, &'a [u8], &'a [u8]),
    pub down: (u64, &'a [u8]),
}

macro_rules! layer_view {
    ($lp:expr) => {
        LayerView {
            vecs: [
                ($lp.attn_norm_handle, $lp.attn_norm_bytes),
                ($lp.q_norm_handle, $lp.q_norm_bytes),
                ($lp.k_norm_handle, $lp.k_norm_bytes),
                ($lp.ffn_norm_handle, $lp.ffn_norm_bytes),
            ],
            qkv: ($lp.fused_qkv_handle, $lp.fused_qkv_bytes),
            o: ($lp.attn_proj_handle, $lp.attn_proj_bytes),
            gate_up: ($lp.gate_up_handle, $lp.gate_bytes, $lp.up_bytes),
            down: ($lp.down_handle, $lp.down_bytes),
        }
    };
}
pub(super) fn views_q1<'a>(lps: &'a [HipFullForwardLayerParams<'a>]) -> Vec<LayerView<'a>> {
    lps.iter().map(|lp| layer_view!(lp)).collect()
}
pub(super) fn views_ternary<'a>(lps: &'a [HipFullForwardLayerParamsTernary<'a>]) -> Vec<LayerView<'a>> {
    lps.iter().map(|lp| layer_view!(lp)).collect()
}

#[derive(Clone, Copy, PartialEq, Eq)]
struct ModelKey {
    fmt: c_int,
    n_layers: usize,
    first_qkv: u64,
    last_down: u64,
    dims: [usize; 6], // nq, nkv, head_dim, hidden, intermediate, max_seq_len
}

struct ModelState {
    key: ModelKey,
    model: u64,
    final_norm: u64, // 0: none attached
    lm_head: u64,    // 0: none attached
    vocab: usize,
}

static MODEL: Mutex<Option<ModelState>> = Mutex::new(None);

/// Is a matrix cached under `id`?  (`get_or_upload_weight_soa`: upload on the first call only.)
fn weight_cached(id: u64) -> bool {
    // SAFETY: null out-pointers are allowed.
    let rc = unsafe {
        ffi::oxb_hip_weight_info(id, core::ptr::null_mut(), core::ptr::null_mut(), core::ptr::null_mut(), core::ptr::null_mut())
    };
    rc == ffi::OXB_HIP_OK
}

pub(super) fn get_or_upload_weight(fmt: c_int, id: u64, bytes: &[u8]) -> Result<(), HipGraphError> {
    if weight_cached(id) {
        return Ok(());
    }
    let mut id_io = id;
    // SAFETY: pointer and length of one slice; bytes alone, the first user names the shape.
    let rc = unsafe {
        if fmt == ffi::OXB_HIP_FMT_Q1 {
            ffi::oxb_hip_upload_q1_raw(&mut id_io, bytes.as_ptr(), bytes.len())
        } else {
            ffi::oxb_hip_upload_tq2_raw(&mut id_io, bytes.as_ptr(), bytes.len())
        }
    };
    check_graph(rc, id)
}

pub(super) fn get_or_upload_fused(fmt: c_int, id: u64, parts: &[&[u8]]) -> Result<(), HipGraphError> {
    if weight_cached(id) {
        return Ok(());
    }
    let mut fused = Vec::with_capacity(parts.iter().map(|p| p.len()).sum());
    for p in parts {
        fused.extend_from_slice(p);
    }
    get_or_upload_weight(fmt, id, &fused)
}

fn upload_vector(id: u64, w: &[f32]) -> Result<(), HipGraphError> {
    let mut id_io = id;
    // SAFETY: pointer and length of one slice.
    check_graph(unsafe { ffi::oxb_hip_upload_f32(&mut id_io, w.as_ptr(), w.len()) }, id)
}

fn dim(v: usize) -> Result<u32, HipGraphError> {
    u32::try_from(v).map_err(|_| HipGraphError::WeightLayoutError(format!("dimension {v} does not fit 32 bits")))
}

/// Finds or builds the process-wide model for these layers, makes sure it carries the wanted final norm / LM head,
/// and runs `f` on its id under the lock.
#[allow(clippy::too_many_arguments)]
pub(super) fn with_model<R>(
    fmt: c_int,
    layers: &[LayerView<'_>],
    nq: usize,
    nkv: usize,
    head_dim: usize,
    hidden_size: usize,
    intermediate_size: usize,
    max_seq_len: usize,
    norm_eps: f32,
    final_norm: Option<(u64, &[f32])>,
    lm_head: Option<(u64, &[u8], usize)>,
    f: impl FnOnce(u64) -> Result<R, HipGraphError>,
) -> Result<R, HipGraphError> {
    let (first, last) = match (layers.first(), layers.last()) {
        (Some(a), Some(b)) => (a, b),
        _ => return Err(HipGraphError::WeightLayoutError("no layers".into())),
    };
    let key = ModelKey {
        fmt,
        n_layers: layers.len(),
        first_qkv: first.qkv.0,
        last_down: last.down.0,
        dims: [nq, nkv, head_dim, hidden_size, intermediate_size, max_seq_len],
    };
    let mut guard = MODEL.lock().map_err(|_| HipGraphError::LockPoisoned)?;
    if guard.as_ref().map(|s| s.key != key).unwrap_or(false) {
        if let Some(old) = guard.take() {
            // SAFETY: plain C call.  The weights stay cached under their ids, as in the reference's weight cache.
            let _ = unsafe { ffi::oxb_hip_model_destroy(old.model) };
        }
    }
    if guard.is_none() {
        // SAFETY: plain C call.
        check_graph(unsafe { ffi::oxb_hip_init(0) }, 0)?;
        let mut ids = Vec::with_capacity(layers.len());
        for lv in layers {
            for (id, w) in lv.vecs {
                upload_vector(id, w)?;
            }
            get_or_upload_weight(fmt, lv.qkv.0, lv.qkv.1)?;
            get_or_upload_weight(fmt, lv.o.0, lv.o.1)?;
            get_or_upload_fused(fmt, lv.gate_up.0, &[lv.gate_up.1, lv.gate_up.2])?;
            get_or_upload_weight(fmt, lv.down.0, lv.down.1)?;
            ids.push(OxbLayerIds {
                attn_norm: lv.vecs[0].0,
                qkv: lv.qkv.0,
                q_norm: lv.vecs[1].0,
                k_norm: lv.vecs[2].0,
                o: lv.o.0,
                ffn_norm: lv.vecs[3].0,
                gate_up: lv.gate_up.0,
                down: lv.down.0,
            });
        }
        let desc = OxbModelDesc {
            fmt,
            n_layers: dim(layers.len())?,
            h: dim(hidden_size)?,
            inter: dim(intermediate_size)?,
            nq: dim(nq)?,
            nkv: dim(nkv)?,
            hd: dim(head_dim)?,
            vocab: 0,
            max_seq: dim(max_seq_len)?,
            batch: 1,
            eps: norm_eps,
            // every position gets its RoPE rows from the caller before it is used (set_rope_rows below)
            rope_theta: 10000.0,
            layers: ids.as_ptr(),
            final_norm: 0,
            lm_head: 0,
        };
        let mut model = 0u64;
        // SAFETY: desc and the ids it points to live across the call; the library copies what it keeps.
        check_graph(unsafe { ffi::oxb_hip_model_create(&desc, &mut model) }, first.qkv.0)?;
        *guard = Some(ModelState { key, model, final_norm: 0, lm_head: 0, vocab: 0 });
    }
    let state = guard.as_mut().ok_or(HipGraphError::LockPoisoned)?;
    let want_norm = final_norm.map(|(id, _)| id).unwrap_or(0);
    let (want_lm, want_vocab) = lm_head.map(|(id, _, v)| (id, v)).unwrap_or((state.lm_head, state.vocab));
    let keep_lm = lm_head.is_none() && want_norm == state.final_norm; // a layers-only call leaves an attached LM head alone
    if !keep_lm && (want_norm != state.final_norm || want_lm != state.lm_head || want_vocab != state.vocab) {
        if let Some((id, w)) = final_norm {
            upload_vector(id, w)?;
        }
        let (lm_id, vocab) = match lm_head {
            Some((id, bytes, vocab)) => {
                get_or_upload_weight(fmt, id, bytes)?;
                (id, vocab)
            }
            None => (0, 0),
        };
        // SAFETY: plain C call; the KV cache and the positions decoded so far stay.
        check_graph(unsafe { ffi::oxb_hip_model_set_lm_head(state.model, want_norm, lm_id, dim(vocab)?) }, lm_id)?;
        state.final_norm = want_norm;
        state.lm_head = lm_id;
        state.vocab = vocab;
    }
    f(state.model)
}

#[allow(clippy::too_many_arguments)]
fn full_forward(
    fmt: c_int,
    hidden: &[f32],
    layers: &[LayerView<'_>],
    rope_cos: &[f32],
    rope_sin: &[f32],
    pos: usize,
    nq: usize,
    nkv: usize,
    head_dim: usize,
    norm_eps: f32,
    hidden_size: usize,
    intermediate_size: usize,
    max_seq_len: usize,
    final_norm: Option<(u64, &[f32])>,
    lm_head: Option<(u64, &[u8], usize)>,
) -> Result<Vec<f32>, HipGraphError> {
    let half = head_dim / 2;
    if hidden.len() < hidden_size || rope_cos.len() < half || rope_sin.len() < half {
        return Err(HipGraphError::WeightLayoutError(format!(
            "hidden holds {} values ({hidden_size} needed), rope rows {} / {} ({half} needed)",
            hidden.len(),
            rope_cos.len(),
            rope_sin.len()
        )));
    }
    let p = dim(pos)?;
    with_model(fmt, layers, nq, nkv, head_dim, hidden_size, intermediate_size, max_seq_len, norm_eps, final_norm, lm_head, |model| {
        // SAFETY: the two rows hold head_dim / 2 values each (checked above).
        check_graph(unsafe { ffi::oxb_hip_model_set_rope_rows(model, p, 1, rope_cos.as_ptr(), rope_sin.as_ptr()) }, 0)?;
        match lm_head {
            Some((id, _, vocab)) => {
                let mut logits = vec![0.0_f32; vocab];
                // SAFETY: hidden holds hidden_size values, logits vocab; the token pointer may be null.
                check_graph(unsafe { ffi::oxb_hip_decode(model, hidden.as_ptr(), &p, logits.as_mut_ptr(), core::ptr::null_mut()) }, id)?;
                Ok(logits)
            }
            None => {
                let mut out = vec![0.0_f32; hidden_size];
                // SAFETY: hidden and out hold hidden_size values.
                check_graph(unsafe { ffi::oxb_hip_decode_hidden(model, hidden.as_ptr(), &p, out.as_mut_ptr()) }, 0)?;
                Ok(out)
            }
        }
    })
}

fn ok_or_warn(what: &str, pos: usize, r: Result<Vec<f32>, HipGraphError>) -> Option<Vec<f32>> {
    if let Err(ref e) = r {
        warn!("HIP {what} error at pos={pos}: {e}");
    }
    r.ok()
}

/// All transformer layers (and the final RMSNorm when `final_norm_bytes` is given) on the GPU; the hidden state
/// comes back.  `None` on any error: callers fall back to their CPU path.  `heads_per_group` is implied by
/// `nq / nkv` and only checked.
#[allow(clippy::too_many_arguments)]
pub fn try_hip_full_forward(
    hidden: &[f32],
    layer_params: &[HipFullForwardLayerParams<'_>],
    rope_cos: &[f32],
    rope_sin: &[f32],
    pos: usize,
    nq: usize,
    nkv: usize,
    head_dim: usize,
    heads_per_group: usize,
    norm_eps: f32,
    hidden_size: usize,
    intermediate_size: usize,
    max_seq_len: usize,
    final_norm_bytes: Option<&[f32]>,
    final_norm_handle: u64,
) -> Option<Vec<f32>> {
    if nkv == 0 || heads_per_group != nq / nkv {
        warn!("HIP full-forward: heads_per_group {heads_per_group} is not nq / nkv = {nq} / {nkv}");
        return None;
    }
    let views = views_q1(layer_params);
    let r = full_forward(ffi::OXB_HIP_FMT_Q1, hidden, &views, rope_cos, rope_sin, pos, nq, nkv, head_dim, norm_eps, hidden_size,
                         intermediate_size, max_seq_len, final_norm_bytes.map(|w| (final_norm_handle, w)), None);
    ok_or_warn("full-forward", pos, r)
}

/// All layers, the final RMSNorm and the Q1 LM-head GEMV on the GPU (one captured graph per token); the logits
/// come back.
#[allow(clippy::too_many_arguments)]
pub fn try_hip_full_forward_with_gpu_lm_head(
    hidden: &[f32],
    layer_params: &[HipFullForwardLayerParams<'_>],
    rope_cos: &[f32],
    rope_sin: &[f32],
    pos: usize,
    nq: usize,
    nkv: usize,
    head_dim: usize,
    heads_per_group: usize,
    norm_eps: f32,
    hidden_size: usize,
    intermediate_size: usize,
    max_seq_len: usize,
    final_norm_bytes: Option<&[f32]>,
    final_norm_handle: u64,
    lm_head_handle: u64,
    lm_head_bytes: &[u8],
    vocab_size: usize,
) -> Option<Vec<f32>> {
    if nkv == 0 || heads_per_group != nq / nkv {
        warn!("HIP full-forward: heads_per_group {heads_per_group} is not nq / nkv = {nq} / {nkv}");
        return None;
    }
    // the device LM head reads the normed state: without a final norm vector there is nothing to attach it to
    let final_norm = final_norm_bytes.map(|w| (final_norm_handle, w))?;
    let views = views_q1(layer_params);
    let r = full_forward(ffi::OXB_HIP_FMT_Q1, hidden, &views, rope_cos, rope_sin, pos, nq, nkv, head_dim, norm_eps, hidden_size,
                         intermediate_size, max_seq_len, Some(final_norm), Some((lm_head_handle, lm_head_bytes, vocab_size)));
    ok_or_warn("full-forward+lm_head", pos, r)
}

/// `try_hip_full_forward` for ternary (TQ2_0_g128) models.
#[allow(clippy::too_many_arguments)]
pub fn try_hip_full_forward_ternary(
    hidden: &[f32],
    layer_params: &[HipFullForwardLayerParamsTernary<'_>],
    rope_cos: &[f32],
    rope_sin: &[f32],
    pos: usize,
    nq: usize,
    nkv: usize,
    head_dim: usize,
    heads_per_group: usize,
    norm_eps: f32,
    hidden_size: usize,
    intermediate_size: usize,
    max_seq_len: usize,
    final_norm_bytes: Option<&[f32]>,
    final_norm_handle: u64,
) -> Option<Vec<f32>> {
    if nkv == 0 || heads_per_group != nq / nkv {
        warn!("HIP ternary full-forward: heads_per_group {heads_per_group} is not nq / nkv = {nq} / {nkv}");
        return None;
    }
    let views = views_ternary(layer_params);
    let r = full_forward(ffi::OXB_HIP_FMT_TQ2, hidden, &views, rope_cos, rope_sin, pos, nq, nkv, head_dim, norm_eps, hidden_size,
                         intermediate_size, max_seq_len, final_norm_bytes.map(|w| (final_norm_handle, w)), None);
    ok_or_warn("ternary full-forward", pos, r)
}

/// `try_hip_full_forward_with_gpu_lm_head` for ternary models (TQ2 LM head).
#[allow(clippy::too_many_arguments)]
pub fn try_hip_full_forward_ternary_with_gpu_lm_head(
    hidden: &[f32],
    layer_params: &[HipFullForwardLayerParamsTernary<'_>],
    rope_cos: &[f32],
    rope_sin: &[f32],
    pos: usize,
    nq: usize,
    nkv: usize,
    head_dim: usize,
    heads_per_group: usize,
    norm_eps: f32,
    hidden_size: usize,
    intermediate_size: usize,
    max_seq_len: usize,
    final_norm_bytes: Option<&[f32]>,
    final_norm_handle: u64,
    lm_head_handle: u64,
    lm_head_bytes: &[u8],
    vocab_size: usize,
) -> Option<Vec<f32>> {
    if nkv == 0 || heads_per_group != nq / nkv {
        warn!("HIP ternary full-forward: heads_per_group {heads_per_group} is not nq / nkv = {nq} / {nkv}");
        return None;
    }
    let final_norm = final_norm_bytes.map(|w| (final_norm_handle, w))?;
    let views = views_ternary(layer_params);
    let r = full_forward(ffi::OXB_HIP_FMT_TQ2, hidden, &views, rope_cos, rope_sin, pos, nq, nkv, head_dim, norm_eps, hidden_size,
                         intermediate_size, max_seq_len, Some(final_norm), Some((lm_head_handle, lm_head_bytes, vocab_size)));
    ok_or_warn("ternary full-forward+lm_head", pos, r)
}

/// The FFN phase of one Q1 layer: hidden += O · attn_out; hidden += down · SwiGLU(gate‖up · RMSNorm(hidden)).
/// Weights are uploaded on the first call and found by id afterwards.
#[allow(clippy::too_many_arguments)]
pub fn try_hip_ffn(
    hidden: &mut [f32],
    attn_out: &[f32],
    norm_weight: &[f32],
    eps: f32,
    attn_proj_handle_id: u64,
    attn_proj_bytes: &[u8],
    gate_up_handle_id: u64,
    gate_bytes: &[u8],
    up_bytes: &[u8],
    down_handle_id: u64,
    down_bytes: &[u8],
    hidden_size: usize,
    intermediate_size: usize,
) -> Result<(), HipGraphError> {
    if hidden.len() < hidden_size || norm_weight.len() < hidden_size {
        return Err(HipGraphError::WeightLayoutError(format!("hidden / norm_weight shorter than {hidden_size}")));
    }
    // the attention output has as many values as the projection has columns: blocks / rows * 128
    if hidden_size == 0 || attn_proj_bytes.len() % (18 * hidden_size) != 0 {
        return Err(HipGraphError::WeightLayoutError(format!("attn_proj holds {} bytes for {hidden_size} rows", attn_proj_bytes.len())));
    }
    let attn_k = attn_proj_bytes.len() / 18 / hidden_size * 128;
    if attn_out.len() < attn_k {
        return Err(HipGraphError::WeightLayoutError(format!("attn_out holds {} values, {attn_k} needed", attn_out.len())));
    }
    // SAFETY: plain C call.
    check_graph(unsafe { ffi::oxb_hip_init(0) }, 0)?;
    let fmt = ffi::OXB_HIP_FMT_Q1;
    get_or_upload_weight(fmt, attn_proj_handle_id, attn_proj_bytes)?;
    get_or_upload_fused(fmt, gate_up_handle_id, &[gate_bytes, up_bytes])?;
    get_or_upload_weight(fmt, down_handle_id, down_bytes)?;
    // SAFETY: lengths checked above.
    let rc = unsafe {
        ffi::oxb_hip_ffn_phase(fmt, hidden.as_mut_ptr(), attn_out.as_ptr(), norm_weight.as_ptr(), eps, attn_proj_handle_id,
                               gate_up_handle_id, down_handle_id, dim(hidden_size)?, dim(intermediate_size)?, dim(attn_k)?)
    };
    check_graph(rc, attn_proj_handle_id)
}

/// The fused Q‖K‖V projection of one Q1 layer: output[0..n_rows] = [Q; K; V] · input.
#[allow(clippy::too_many_arguments)]
pub fn try_hip_qkv(
    input: &[f32],
    output: &mut [f32],
    weight_handle_id: u64,
    q_bytes: &[u8],
    k_bytes: &[u8],
    v_bytes: &[u8],
    n_rows: usize,
    k: usize,
) -> Result<(), HipGraphError> {
    if input.len() < k || output.len() < n_rows {
        return Err(HipGraphError::WeightLayoutError(format!(
            "input holds {} values ({k} needed), output {} ({n_rows} needed)",
            input.len(),
            output.len()
        )));
    }
    // SAFETY: plain C call.
    check_graph(unsafe { ffi::oxb_hip_init(0) }, 0)?;
    get_or_upload_fused(ffi::OXB_HIP_FMT_Q1, weight_handle_id, &[q_bytes, k_bytes, v_bytes])?;
    // SAFETY: lengths checked above.
    let rc = unsafe { ffi::oxb_hip_gemv(weight_handle_id, input.as_ptr(), output.as_mut_ptr(), dim(n_rows)?, dim(k)?, 1) };
    check_graph(rc, weight_handle_id)
}
