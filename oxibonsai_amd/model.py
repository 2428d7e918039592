"""Host-side mirror of the reference's fused whole-model GPU forward.

``HipModel`` plays the part of ``BonsaiModel``'s GPU branch
(crates/oxibonsai-model/src/model/types/forward_cuda/{q1,ternary}.rs): it uploads every
layer's blocks once (fused Q|K|V and gate|up concatenations are made on the AoS bytes, as
crates/oxibonsai-model/src/block/types/upload.rs:21-39 does), then each ``forward`` is one
call of ``oxb_hip_decode`` = ``try_cuda_full_forward_with_gpu_lm_head``."""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import _lib
from .backend import GpuError, NativeHipBackend, _check
from .synth import Q1


class _LayerIds(C.Structure):
    _fields_ = [(n, C.c_uint64) for n in ("attn_norm", "qkv", "q_norm", "k_norm", "o", "ffn_norm", "gate_up", "down")]


class _ModelDesc(C.Structure):
    _fields_ = [("fmt", C.c_int)] + [(n, C.c_uint32) for n in
                                      ("n_layers", "h", "inter", "nq", "nkv", "hd", "vocab", "max_seq", "batch")] + \
               [("eps", C.c_float), ("rope_theta", C.c_float), ("layers", C.POINTER(_LayerIds)),
                ("final_norm", C.c_uint64), ("lm_head", C.c_uint64)]


class GgufInfo(C.Structure):
    """oxb_gguf_info: what GgufFile::parse + Qwen3Config::from_metadata tell about a checkpoint."""
    _fields_ = [("version", C.c_uint32), ("alignment", C.c_uint32), ("n_tensors", C.c_uint64), ("n_metadata", C.c_uint64),
                ("fmt", C.c_int), ("embedding_type", C.c_int)] + \
               [(n, C.c_uint32) for n in ("n_layers", "h", "inter", "nq", "nkv", "hd", "vocab", "context_length")] + \
               [("eps", C.c_float), ("rope_theta", C.c_float), ("architecture", C.c_char * 32), ("name", C.c_char * 64),
                ("lm_head_rows", C.c_uint32)]

    def as_dict(self) -> dict:
        d = {n: getattr(self, n) for n, _ in self._fields_}
        d["architecture"], d["name"] = self.architecture.decode(), self.name.decode()
        return d


def gguf_info(path: str) -> dict:
    """Header, configuration and formats of a GGUF checkpoint; needs no GPU
    (GgufFile::parse, crates/oxibonsai-core/src/gguf/reader.rs:25-66; Qwen3Config::from_metadata, config.rs:41-118)."""
    info = GgufInfo()
    _check(_lib.lib().oxb_hip_gguf_info(str(path).encode(), C.byref(info)))
    return info.as_dict()


def gguf_metadata(path: str, key: str) -> str:
    """One metadata value of a GGUF file as text (MetadataStore::get, crates/oxibonsai-core/src/gguf/metadata.rs:94)."""
    buf = C.create_string_buffer(4096)
    _check(_lib.lib().oxb_hip_gguf_metadata(str(path).encode(), key.encode(), buf, len(buf)))
    return buf.value.decode()


def gguf_tensor(path: str, name: str) -> dict:
    """Directory entry of one tensor (TensorStore::require, gguf/tensor_info.rs:86): type id, shape in file order,
    absolute file offset of the data and its size in bytes."""
    t, nd, sh, off, nb = C.c_int(0), C.c_uint32(0), (C.c_uint64 * 4)(), C.c_uint64(0), C.c_uint64(0)
    _check(_lib.lib().oxb_hip_gguf_tensor(str(path).encode(), name.encode(), C.byref(t), C.byref(nd), sh, C.byref(off), C.byref(nb)))
    return {"type": t.value, "shape": [int(sh[i]) for i in range(min(nd.value, 4))], "n_dims": nd.value,
            "file_offset": off.value, "bytes": nb.value}


class Sampling(C.Structure):
    """oxb_sampling: the SamplingParams fields Sampler::sample reads (crates/oxibonsai-runtime/src/sampling.rs:14-27)."""
    _fields_ = [("temperature", C.c_float), ("top_k", C.c_uint32), ("top_p", C.c_float)]


def sample_logits(logits, temperature: float, top_k: int, top_p: float, rng_state):
    """Sampler::sample on the device for rows of host logits -> (tokens [batch], advanced rng states [batch])."""
    a = np.ascontiguousarray(logits, dtype=np.float32)
    a = a.reshape(1, -1) if a.ndim == 1 else a
    st = np.ascontiguousarray(np.broadcast_to(np.asarray(rng_state, dtype=np.uint64), (a.shape[0],))).copy()
    out = np.empty(a.shape[0], dtype=np.uint32)
    sp = Sampling(temperature, top_k, top_p)
    _check(_lib.lib().oxb_hip_sample_logits(a.ctypes.data_as(_lib.f32p), a.shape[1], a.shape[0], C.byref(sp),
                                            st.ctypes.data_as(_lib.u64p), out.ctypes.data_as(_lib.u32p)))
    return out, st


def sum_in_order(x) -> np.float32:
    """((0 + x[0]) + x[1]) + ... in f32 on the device, the order of the reference's softmax loop (sampling.rs:126-130)."""
    a = np.ascontiguousarray(x, dtype=np.float32).ravel()
    out = np.zeros(1, dtype=np.float32)
    _check(_lib.lib().oxb_hip_sum_in_order(a.ctypes.data_as(_lib.f32p), a.size, out.ctypes.data_as(_lib.f32p)))
    return out[0]


KV_F16, KV_I8, KV_FP8_E4M3 = 0, 1, 2   # OXB_KV_DTYPE_*


class AttentionOptions(C.Structure):
    """oxb_attention_options: KV cache storage type, SlidingWindowConfig { window_size, sink_tokens }
    (crates/oxibonsai-model/src/layers/sliding_window.rs:11-43; window_size 0 = no window) and the page pool of a paged
    cache (crates/oxibonsai-model/src/paged_kv_cache.rs; page_size = n_pages = 0: contiguous cache)."""
    _fields_ = [("kv_dtype", C.c_int32), ("window_size", C.c_uint32), ("sink_tokens", C.c_uint32),
                ("page_size", C.c_uint32), ("n_pages", C.c_uint32)]


class KvPoolInfo(C.Structure):
    _fields_ = [("page_size", C.c_uint32), ("total_pages", C.c_uint32), ("free_pages", C.c_uint32)]


def kv_quantize_rows(kv_dtype: int, rows):
    """quantize_row_i8 / quantize_row_fp8 (crates/oxibonsai-model/src/kv_cache_quant.rs:46-62, 519-540) on the device
    -> (codes uint8 [n_rows][n], scales f32 [n_rows])."""
    lib = _lib.lib()
    a = np.ascontiguousarray(rows, dtype=np.float32)
    if a.ndim != 2:
        raise ValueError("rows must be a 2-D array")
    codes = np.empty(a.shape, dtype=np.uint8)
    scales = np.empty(a.shape[0], dtype=np.float32)
    _check(lib.oxb_hip_kv_quantize_rows(kv_dtype, a.ctypes.data_as(_lib.f32p), a.shape[0], a.shape[1],
                                        codes.ctypes.data_as(_lib.u8p), scales.ctypes.data_as(_lib.f32p)))
    return codes, scales


def kv_dequantize_rows(kv_dtype: int, codes, scales) -> np.ndarray:
    """dequantize_row (crates/oxibonsai-model/src/kv_cache_quant.rs:69-71, 545-556) on the device, through the
    widening the attention kernels use: codes uint8 [n_rows][n], scales f32 [n_rows] -> f32 [n_rows][n]."""
    lib = _lib.lib()
    c = np.ascontiguousarray(codes, dtype=np.uint8)
    s = np.ascontiguousarray(scales, dtype=np.float32).reshape(-1)
    if c.ndim != 2 or s.size != c.shape[0]:
        raise ValueError("codes must be 2-D with one scale per row")
    out = np.empty(c.shape, dtype=np.float32)
    _check(lib.oxb_hip_kv_dequantize_rows(kv_dtype, c.ctypes.data_as(_lib.u8p), s.ctypes.data_as(_lib.f32p), c.shape[0], c.shape[1],
                                          out.ctypes.data_as(_lib.f32p)))
    return out


class Embedding:
    """Token embedding table resident on the device in its stored form (F32, F16, Q1_0_g128 or TQ2_0_g128)."""

    def __init__(self, table, gguf_type: int, vocab: int, h: int, _id: int = 0):
        self._lib = _lib.lib()
        if _id:
            self.id = _id
        else:
            a = np.ascontiguousarray(table)
            eid = C.c_uint64(0)
            _check(self._lib.oxb_hip_upload_embedding(C.byref(eid), a.ctypes.data_as(C.c_void_p), a.nbytes, gguf_type, vocab, h))
            self.id = eid.value
        self.vocab, self.h, self.gguf_type = vocab, h, gguf_type

    def rows(self, ids) -> np.ndarray:
        iv = np.ascontiguousarray(ids, dtype=np.uint32).reshape(-1)
        out = np.empty((iv.size, self.h), dtype=np.float32)
        _check(self._lib.oxb_hip_embedding_rows(self.id, iv.ctypes.data_as(_lib.u32p), iv.size, out.ctypes.data_as(_lib.f32p)))
        return out

    def close(self):
        if self.id:
            _check(self._lib.oxb_hip_free_embedding(self.id))
            self.id = 0


class HipModel:
    """cfg: fmt, n_layers, h, inter, nq, nkv, hd, vocab, max_seq, eps, rope_theta.
    weights: dict of oxibonsai_amd.synth.make_model (reference AoS blocks + f32 norm vectors)."""

    def __init__(self, backend: NativeHipBackend, cfg: dict, weights: dict, batch: int = 1, lm_head: bool = True,
                 shaped_uploads: bool = True):
        """lm_head=False builds the model of try_cuda_full_forward (no LM head on the device: forward_hidden only);
        shaped_uploads=False uploads every matrix as bytes alone, as the reference's callers do, and lets the model's
        dimensions give them their shapes."""
        self.be, self.cfg, self.batch = backend, cfg, batch
        self._lib = _lib.lib()
        self._mats, self._vecs = [], []
        self._shaped, self._has_lm = shaped_uploads, lm_head
        fmt, h, inter, hd = cfg["fmt"], cfg["h"], cfg["inter"], cfg["hd"]
        qd, kd = cfg["nq"] * hd, cfg["nkv"] * hd
        ids = (_LayerIds * cfg["n_layers"])()
        for i, lw in enumerate(weights["layers"]):
            qkv = np.concatenate([lw["q"], lw["k"], lw["v"]])
            gate_up = np.concatenate([lw["gate"], lw["up"]])
            ids[i] = _LayerIds(self._vec(lw["attn_norm"]), self._mat(qkv, qd + 2 * kd, h), self._vec(lw["q_norm"]),
                               self._vec(lw["k_norm"]), self._mat(lw["o"], h, qd), self._vec(lw["ffn_norm"]),
                               self._mat(gate_up, 2 * inter, h), self._mat(lw["down"], h, inter))
        self._ids = ids
        desc = _ModelDesc(fmt, cfg["n_layers"], h, inter, cfg["nq"], cfg["nkv"], hd, cfg["vocab"], cfg["max_seq"], batch,
                          cfg["eps"], cfg["rope_theta"], ids, self._vec(weights["final_norm"]),
                          self._mat(weights["lm_head"], cfg["vocab"], h) if lm_head else 0)
        mid = C.c_uint64(0)
        _check(self._lib.oxb_hip_model_create(C.byref(desc), C.byref(mid)))
        self.id = mid.value

    @classmethod
    def from_gguf(cls, backend: NativeHipBackend, path: str, max_seq: int = 0, batch: int = 1):
        """BonsaiModel::from_gguf (crates/oxibonsai-model/src/model/types/mod.rs:71-160) on the device:
        -> (model, embedding, info dict).  The model owns the weights it uploaded."""
        self = cls.__new__(cls)
        self.be, self.batch = backend, batch
        self._lib = _lib.lib()
        self._mats, self._vecs = [], []
        self._shaped, self._has_lm = True, True
        info, mid, eid = GgufInfo(), C.c_uint64(0), C.c_uint64(0)
        _check(self._lib.oxb_hip_load_gguf(str(path).encode(), max_seq, batch, C.byref(mid), C.byref(eid), C.byref(info)))
        d = info.as_dict()
        self.cfg = dict(fmt=d["fmt"], n_layers=d["n_layers"], h=d["h"], inter=d["inter"], nq=d["nq"], nkv=d["nkv"], hd=d["hd"],
                        vocab=d["lm_head_rows"], max_seq=max_seq or d["context_length"], eps=d["eps"], rope_theta=d["rope_theta"])
        self.id = mid.value
        return self, Embedding(None, d["embedding_type"], d["vocab"], d["h"], _id=eid.value), d

    def _mat(self, blocks, n_rows, k):
        fmt = self.cfg["fmt"]
        shape = (n_rows, k) if self._shaped else (None, None)
        h = self.be.upload_weights_raw(blocks, *shape) if fmt == Q1 else self.be.upload_weights_ternary(blocks, *shape)
        self._mats.append(h)
        return int(h)

    def _vec(self, v):
        a = np.ascontiguousarray(v, dtype=np.float32)
        hid = C.c_uint64(0)
        _check(self._lib.oxb_hip_upload_f32(C.byref(hid), a.ctypes.data_as(_lib.f32p), a.size))
        self._vecs.append(hid.value)
        return hid.value

    def forward(self, hidden, pos, want_logits: bool = True):
        """hidden: [batch, h] embedding rows; pos: [batch] positions -> (logits [batch, vocab] or None, tokens [batch])."""
        n = self.batch * self.cfg["h"]
        if type(hidden) is np.ndarray and hidden.dtype == np.float32 and hidden.size == n and hidden.flags.c_contiguous:
            hv = hidden             # (the per-token call of a decode loop: nothing to convert)
        else:
            hv = np.ascontiguousarray(hidden, dtype=np.float32).reshape(self.batch, self.cfg["h"])
        io = self.__dict__.get("_io")
        if io is None:      # position and token arrays of the calls, with their pointers
            pb, tb = np.zeros(self.batch, dtype=np.uint32), np.zeros(self.batch, dtype=np.uint32)
            io = self._io = (pb, tb, pb.ctypes.data_as(_lib.u32p), tb.ctypes.data_as(_lib.u32p))
        io[0][:] = pos      # a scalar, or one position per sequence
        logits = np.empty((self.batch, self.cfg["vocab"]), dtype=np.float32) if want_logits else None
        _check(self._lib.oxb_hip_decode(self.id, hv.ctypes.data_as(_lib.f32p), io[2],
                                        logits.ctypes.data_as(_lib.f32p) if want_logits else None, io[3]))
        return logits, io[1].copy()

    def forward_hidden(self, hidden, pos) -> np.ndarray:
        """All layers and the final norm, no LM head (try_cuda_full_forward, gpu_backend/cuda_full_layer/encode_q1.rs:813):
        hidden [batch, h], pos [batch] -> normed hidden state [batch, h]."""
        hv = np.ascontiguousarray(hidden, dtype=np.float32).reshape(self.batch, self.cfg["h"])
        pv = np.ascontiguousarray(np.broadcast_to(np.asarray(pos, dtype=np.uint32), (self.batch,)))
        out = np.empty((self.batch, self.cfg["h"]), dtype=np.float32)
        _check(self._lib.oxb_hip_decode_hidden(self.id, hv.ctypes.data_as(_lib.f32p), pv.ctypes.data_as(_lib.u32p),
                                               out.ctypes.data_as(_lib.f32p)))
        return out

    def set_lm_head(self, final_norm, lm_head_blocks, vocab: int):
        """Attach (or replace) the final norm vector and the LM head of a live model; the KV cache stays.
        lm_head_blocks None takes the LM head away."""
        fn = self._vec(final_norm) if final_norm is not None else 0
        lm = self._mat(lm_head_blocks, vocab, self.cfg["h"]) if lm_head_blocks is not None else 0
        _check(self._lib.oxb_hip_model_set_lm_head(self.id, fn, lm, vocab if lm else 0))
        self._has_lm = bool(lm)
        self.cfg = dict(self.cfg, vocab=vocab)

    def set_rope_rows(self, pos_start: int, cos_rows, sin_rows):
        """The caller's own RoPE rows ([n_pos, hd/2] each) for positions pos_start.., as the reference's entry points
        receive them (rope_cos / rope_sin, cos_table / sin_table)."""
        c = np.ascontiguousarray(cos_rows, dtype=np.float32).reshape(-1, self.cfg["hd"] // 2)
        s = np.ascontiguousarray(sin_rows, dtype=np.float32).reshape(-1, self.cfg["hd"] // 2)
        if c.shape != s.shape:
            raise ValueError("cos and sin rows differ in shape")
        _check(self._lib.oxb_hip_model_set_rope_rows(self.id, pos_start, c.shape[0], c.ctypes.data_as(_lib.f32p),
                                                     s.ctypes.data_as(_lib.f32p)))

    def prefill(self, hidden, pos_start: int = 0, seq: int = 0, want_logits: bool = True):
        """Batched prefill of one sequence (try_cuda_prefill, gpu_backend/cuda_prefill/try_apis.rs:42, 318).
        hidden: [n_tokens, h] embedding rows for positions pos_start.. -> (last-token logits [vocab] or None,
        greedy token of the last position).  Decode continues at pos_start + n_tokens."""
        hv = np.ascontiguousarray(hidden, dtype=np.float32).reshape(-1, self.cfg["h"])
        logits = np.empty(self.cfg["vocab"], dtype=np.float32) if want_logits else None
        token = np.empty(1, dtype=np.uint32)
        _check(self._lib.oxb_hip_prefill(self.id, seq, hv.ctypes.data_as(_lib.f32p), hv.shape[0], pos_start,
                                         logits.ctypes.data_as(_lib.f32p) if want_logits else None,
                                         token.ctypes.data_as(_lib.u32p) if self._has_lm else None))
        return logits, (int(token[0]) if self._has_lm else None)

    def generate(self, embedding: Embedding, tokens, pos, n_steps: int) -> np.ndarray:
        """Greedy decode of n_steps tokens per sequence without a host round trip per token: tokens [batch] are fed
        at pos [batch], every further step feeds the previous argmax -> ids [n_steps, batch]."""
        tv = np.ascontiguousarray(np.broadcast_to(np.asarray(tokens, dtype=np.uint32), (self.batch,)))
        pv = np.ascontiguousarray(np.broadcast_to(np.asarray(pos, dtype=np.uint32), (self.batch,)))
        out = np.empty((n_steps, self.batch), dtype=np.uint32)
        _check(self._lib.oxb_hip_decode_tokens(self.id, embedding.id, tv.ctypes.data_as(_lib.u32p), pv.ctypes.data_as(_lib.u32p),
                                               n_steps, out.ctypes.data_as(_lib.u32p)))
        return out

    def generate_sampled(self, embedding: Embedding, tokens, pos, n_steps: int, temperature: float, top_k: int, top_p: float,
                         rng_state):
        """generate() with Sampler::sample instead of the argmax -> (ids [n_steps, batch], advanced rng states [batch])."""
        tv = np.ascontiguousarray(np.broadcast_to(np.asarray(tokens, dtype=np.uint32), (self.batch,)))
        pv = np.ascontiguousarray(np.broadcast_to(np.asarray(pos, dtype=np.uint32), (self.batch,)))
        st = np.ascontiguousarray(np.broadcast_to(np.asarray(rng_state, dtype=np.uint64), (self.batch,))).copy()
        out = np.empty((n_steps, self.batch), dtype=np.uint32)
        sp = Sampling(temperature, top_k, top_p)
        _check(self._lib.oxb_hip_decode_tokens_sampled(self.id, embedding.id, tv.ctypes.data_as(_lib.u32p), pv.ctypes.data_as(_lib.u32p),
                                                       n_steps, C.byref(sp), st.ctypes.data_as(_lib.u64p), out.ctypes.data_as(_lib.u32p)))
        return out, st

    def prefill_tokens(self, embedding: Embedding, ids, pos_start: int = 0, seq: int = 0, want_logits: bool = True):
        """prefill() with the embedding rows gathered on the device from token ids."""
        iv = np.ascontiguousarray(ids, dtype=np.uint32).reshape(-1)
        logits = np.empty(self.cfg["vocab"], dtype=np.float32) if want_logits else None
        token = np.empty(1, dtype=np.uint32)
        _check(self._lib.oxb_hip_prefill_tokens(self.id, embedding.id, seq, iv.ctypes.data_as(_lib.u32p), iv.size, pos_start,
                                                logits.ctypes.data_as(_lib.f32p) if want_logits else None,
                                                token.ctypes.data_as(_lib.u32p)))
        return logits, int(token[0])

    def uses_graph(self) -> bool:
        return bool(self._lib.oxb_hip_model_uses_graph(self.id))

    def set_attention(self, kv_dtype: int = KV_F16, window_size: int = 0, sink_tokens: int = 0, page_size: int = 0,
                      n_pages: int = 0):
        """Long-context options of the attention kernels; changing kv_dtype or the paging replaces the cache (start
        again at 0)."""
        opt = AttentionOptions(kv_dtype, window_size, sink_tokens, page_size, n_pages)
        _check(self._lib.oxb_hip_model_set_attention(self.id, C.byref(opt)))

    def kv_reserve(self, seq: int, n_tokens: int):
        """PagedKvCache::ensure_capacity: pages for positions 0 .. n_tokens - 1 of a sequence slot."""
        _check(self._lib.oxb_hip_model_kv_reserve(self.id, seq, n_tokens))

    def kv_release(self, seq: int):
        """PagedKvCache::drop_sequence: the slot's pages return to the pool."""
        _check(self._lib.oxb_hip_model_kv_release(self.id, seq))

    def kv_pool(self) -> KvPoolInfo:
        info = KvPoolInfo()
        _check(self._lib.oxb_hip_model_kv_pool(self.id, C.byref(info)))
        return info

    def kv_capacity(self, seq: int) -> int:
        n = C.c_uint32(0)
        _check(self._lib.oxb_hip_model_kv_capacity(self.id, seq, C.byref(n)))
        return int(n.value)

    def attention(self) -> AttentionOptions:
        opt = AttentionOptions()
        _check(self._lib.oxb_hip_model_get_attention(self.id, C.byref(opt)))
        return opt

    def read_kv(self, layer: int, kv_head: int, pos: int, n_pos: int, seq: int = 0):
        """Cache rows as stored -> (k, v, k_scales, v_scales): fp16 rows (scales 1.0) or uint8 codes with row scales."""
        dt = np.float16 if self.attention().kv_dtype == KV_F16 else np.uint8
        hd = self.cfg["hd"]
        k, v = np.empty((n_pos, hd), dtype=dt), np.empty((n_pos, hd), dtype=dt)
        ks, vs = np.empty(n_pos, dtype=np.float32), np.empty(n_pos, dtype=np.float32)
        _check(self._lib.oxb_hip_model_read_kv(self.id, seq, layer, kv_head, pos, n_pos, k.ctypes.data, v.ctypes.data,
                                               ks.ctypes.data_as(_lib.f32p), vs.ctypes.data_as(_lib.f32p)))
        return k, v, ks, vs

    def reset(self):
        _check(self._lib.oxb_hip_model_reset(self.id))

    def close(self):
        if self.id:
            _check(self._lib.oxb_hip_model_destroy(self.id))
            self.id = 0
            for h in self._mats:
                self.be.free_weights(h)
            for v in self._vecs:
                _check(self._lib.oxb_hip_free_f32(v))
            self._mats, self._vecs = [], []


def batch_ffn_phase(backend: NativeHipBackend, fmt: int, hidden, attn_out, norm_weight, norm_eps: float,
                    attn_proj_handle: int, gate_up_handle: int, down_handle: int, h: int, intermediate: int,
                    attn_proj_k: int) -> np.ndarray:
    """GpuBackendTrait::batch_ffn_phase (gpu_backend/mod.rs:519): returns the updated hidden vector."""
    hv = np.array(hidden, dtype=np.float32, copy=True)
    av = np.ascontiguousarray(attn_out, dtype=np.float32)
    nv = np.ascontiguousarray(norm_weight, dtype=np.float32)
    if hv.size < h or av.size < attn_proj_k or nv.size < h:
        raise GpuError(5, "invalid argument: buffer shorter than its dimension")
    _check(_lib.lib().oxb_hip_ffn_phase(fmt, hv.ctypes.data_as(_lib.f32p), av.ctypes.data_as(_lib.f32p),
                                        nv.ctypes.data_as(_lib.f32p), norm_eps, int(attn_proj_handle),
                                        int(gate_up_handle), int(down_handle), h, intermediate, attn_proj_k))
    return hv


def batch_attn_phase(backend: NativeHipBackend, fmt: int, hidden, norm_weight, norm_eps: float, qkv_handle: int,
                     q_rows: int, k_rows: int, h: int):
    """GpuBackendTrait::batch_attn_phase (gpu_backend/mod.rs:501): RMSNorm + fused QKV product -> (q, k, v)."""
    hv = np.ascontiguousarray(hidden, dtype=np.float32)
    nv = np.ascontiguousarray(norm_weight, dtype=np.float32)
    if hv.size < h or nv.size < h:
        raise GpuError(5, "invalid argument: buffer shorter than its dimension")
    q, k, v = (np.empty(n, dtype=np.float32) for n in (q_rows, k_rows, k_rows))
    _check(_lib.lib().oxb_hip_attn_phase(fmt, hv.ctypes.data_as(_lib.f32p), nv.ctypes.data_as(_lib.f32p), norm_eps,
                                         int(qkv_handle), q_rows, k_rows, h, q.ctypes.data_as(_lib.f32p),
                                         k.ctypes.data_as(_lib.f32p), v.ctypes.data_as(_lib.f32p)))
    return q, k, v
