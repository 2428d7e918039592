"""ctypes front end of the CPU oracle (``liboxb_oracle.so``).

TEST INFRASTRUCTURE ONLY.  Imported by ``tests/``, by ``__graft_entry__.smoke``
and by the ``cpu_baseline`` leg of ``bench.py``; the shipped package never
imports it.  Every function maps 1:1 onto a C function of ``oxb_oracle.h`` /
``oxb_simd.cpp``, whose comments cite the reference source they restate.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboxb_oracle.so")
_lib = None

OK, NOT_BLOCK_ALIGNED, DIMENSION_MISMATCH, BUFFER_TOO_SMALL = 0, 1, 2, 3
Q1_BYTES, TQ2_BYTES, QK = 18, 34, 128


class OracleError(Exception):
    def __init__(self, code: int):
        super().__init__({1: "NotBlockAligned", 2: "DimensionMismatch", 3: "BufferTooSmall"}.get(code, str(code)))
        self.code = code


def build() -> None:
    subprocess.check_call(["make", "-s", "-C", _HERE])


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = C.CDLL(_LIB_PATH)
        u8p, f32p, sz = C.POINTER(C.c_uint8), C.POINTER(C.c_float), C.c_size_t
        L.oxb_f16_to_f32.restype = C.c_float
        L.oxb_f16_to_f32.argtypes = [C.c_uint16]
        L.oxb_f32_to_f16.restype = C.c_uint16
        L.oxb_f32_to_f16.argtypes = [C.c_float]
        for n in ("oxb_dequant_q1", "oxb_dequant_tq2"):
            getattr(L, n).argtypes = [u8p, sz, f32p, sz]
        for n in ("oxb_gemv_q1", "oxb_gemv_tq2"):
            getattr(L, n).argtypes = [u8p, sz, f32p, sz, f32p, sz, sz, sz]
        for n in ("oxb_gemm_q1", "oxb_gemm_tq2"):
            getattr(L, n).argtypes = [u8p, sz, f32p, sz, f32p, sz, sz, sz, sz]
        L.oxb_rms_norm.argtypes = [f32p, f32p, f32p, sz, C.c_float]
        L.oxb_rms_norm.restype = None
        L.oxb_silu.argtypes = [C.c_float]
        L.oxb_silu.restype = C.c_float
        L.oxb_swiglu.argtypes = [f32p, f32p, f32p, sz]
        L.oxb_swiglu.restype = None
        L.oxb_softmax.argtypes = [f32p, sz]
        L.oxb_softmax.restype = None
        L.oxb_rope_table.argtypes = [f32p, f32p, sz, sz, C.c_float]
        L.oxb_rope_table.restype = None
        L.oxb_rope_apply.argtypes = [f32p, f32p, f32p, f32p, sz]
        L.oxb_rope_apply.restype = None
        L.oxb_attention_head.argtypes = [f32p, f32p, f32p, f32p, sz, sz]
        L.oxb_attention_head.restype = None
        for n in ("oxb_argmax_last", "oxb_argmax_first"):
            getattr(L, n).argtypes = [f32p, sz]
            getattr(L, n).restype = C.c_uint32
        L.oxb_state_new.restype = C.c_void_p
        L.oxb_state_cache.restype = C.c_void_p
        L.oxb_state_cache.argtypes = [C.c_void_p, C.c_int]
        L.oxb_state_load_rows.argtypes = [C.c_void_p, C.c_void_p, sz, sz, sz, sz, f32p, f32p]
        L.oxb_state_load_rows.restype = None
        L.oxb_state_freeze.argtypes = [C.c_void_p, C.c_int]
        L.oxb_state_freeze.restype = None
        L.oxb_in_window.argtypes = [sz, sz, sz, sz]
        L.oxb_attention_head_windowed.argtypes = [f32p, f32p, f32p, f32p, sz, sz, sz, sz]
        L.oxb_attention_head_windowed.restype = None
        for n in ("oxb_fp8_e4m3_encode", "oxb_fp8_e5m2_encode"):
            getattr(L, n).argtypes = [C.c_float]
            getattr(L, n).restype = C.c_uint8
        for n in ("oxb_fp8_e4m3_decode", "oxb_fp8_e5m2_decode"):
            getattr(L, n).argtypes = [C.c_uint8]
            getattr(L, n).restype = C.c_float
        L.oxb_kv_quantize_row.argtypes = [C.c_int, f32p, sz, u8p, C.POINTER(C.c_float)]
        L.oxb_kv_dequantize_row.argtypes = [C.c_int, u8p, sz, C.c_float, f32p]
        L.oxb_oracle_set_threads.argtypes = [C.c_int]
        L.oxb_oracle_set_threads.restype = None
        L.oxb_sample.restype = C.c_uint32
        L.oxb_sample.argtypes = [f32p, sz, C.c_float, sz, C.c_float, C.POINTER(C.c_uint64), C.POINTER(C.c_uint32), f32p, sz,
                                 C.POINTER(sz), f32p]
        L.oxb_state_new.argtypes = [C.c_void_p]
        L.oxb_state_free.argtypes = [C.c_void_p]
        L.oxb_state_free.restype = None
        L.oxb_forward_ex.argtypes = [C.c_void_p, C.c_void_p, f32p, sz, f32p, f32p]
        L.oxb_simd_tier.restype = C.c_int
        L.oxb_simd_set_tier.argtypes = [C.c_int]
        L.oxb_simd_set_tier.restype = C.c_int
        L.oxb_simd_threads.restype = C.c_int
        L.oxb_simd_set_threads.argtypes = [C.c_int]
        L.oxb_simd_set_threads.restype = None
        L.oxb_simd_gemv.argtypes = [C.c_int, u8p, sz, f32p, sz, f32p, sz, sz, sz]
        L.oxb_simd_gemm.argtypes = [C.c_int, u8p, sz, f32p, sz, f32p, sz, sz, sz, sz]
        L.oxb_simd_gemm_x4.argtypes = [C.c_int, u8p, sz, f32p, sz, f32p, sz, sz, sz, sz]
        L.oxb_forward_batch.argtypes = [C.c_void_p, C.c_void_p, f32p, sz, sz, f32p, f32p]
        _lib = L
    return _lib


def _u8(a):
    return a.ctypes.data_as(C.POINTER(C.c_uint8))


def _f32(a):
    return a.ctypes.data_as(C.POINTER(C.c_float))


def _bytes(a) -> np.ndarray:
    return np.ascontiguousarray(np.frombuffer(a, dtype=np.uint8) if not isinstance(a, np.ndarray) else a, dtype=np.uint8)


def _vec(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.float32)


def _check(rc: int) -> None:
    if rc != 0:
        raise OracleError(rc)


def f16_to_f32(h: int) -> float:
    return float(lib().oxb_f16_to_f32(int(h)))


def f32_to_f16(f: float) -> int:
    return int(lib().oxb_f32_to_f16(float(f)))


def dequant(fmt: int, blocks) -> np.ndarray:
    b = _bytes(blocks)
    bb = Q1_BYTES if fmt == 0 else TQ2_BYTES
    n = b.size // bb
    out = np.empty(n * QK, dtype=np.float32)
    fn = lib().oxb_dequant_q1 if fmt == 0 else lib().oxb_dequant_tq2
    _check(fn(_u8(b), n, _f32(out), out.size))
    return out


def gemv(fmt: int, blocks, x, n_rows: int, k: int, y_len: int | None = None) -> np.ndarray:
    """Scalar reference GEMV.  Buffer lengths are passed as they are, so the
    reference's validation errors can be provoked."""
    b, xv = _bytes(blocks), _vec(x)
    bb = Q1_BYTES if fmt == 0 else TQ2_BYTES
    y = np.zeros(n_rows if y_len is None else y_len, dtype=np.float32)
    fn = lib().oxb_gemv_q1 if fmt == 0 else lib().oxb_gemv_tq2
    _check(fn(_u8(b), b.size // bb, _f32(xv), xv.size, _f32(y), y.size, n_rows, k))
    return y


def gemm(fmt: int, blocks, x, m: int, n_rows: int, k: int) -> np.ndarray:
    b, xv = _bytes(blocks), _vec(x).reshape(-1)
    bb = Q1_BYTES if fmt == 0 else TQ2_BYTES
    y = np.zeros(m * n_rows, dtype=np.float32)
    fn = lib().oxb_gemm_q1 if fmt == 0 else lib().oxb_gemm_tq2
    _check(fn(_u8(b), b.size // bb, _f32(xv), xv.size, _f32(y), y.size, m, n_rows, k))
    return y.reshape(m, n_rows)


def simd_gemv(fmt: int, blocks, x, n_rows: int, k: int, out: np.ndarray | None = None) -> np.ndarray:
    b, xv = _bytes(blocks), _vec(x)
    bb = Q1_BYTES if fmt == 0 else TQ2_BYTES
    y = np.zeros(n_rows, dtype=np.float32) if out is None else out
    _check(lib().oxb_simd_gemv(fmt, _u8(b), b.size // bb, _f32(xv), xv.size, _f32(y), y.size, n_rows, k))
    return y


def simd_gemm(fmt: int, blocks, x, m: int, n_rows: int, k: int, x4: bool = False) -> np.ndarray:
    """x4: the route for long prompts (four token rows share each decoded weight chunk; the same bits)."""
    b, xv = _bytes(blocks), _vec(x).reshape(-1)
    bb = Q1_BYTES if fmt == 0 else TQ2_BYTES
    y = np.zeros(m * n_rows, dtype=np.float32)
    fn = lib().oxb_simd_gemm_x4 if x4 else lib().oxb_simd_gemm
    _check(fn(fmt, _u8(b), b.size // bb, _f32(xv), xv.size, _f32(y), y.size, m, n_rows, k))
    return y.reshape(m, n_rows)


SIMD_TIERS = {0: "scalar", 1: "avx2+fma", 2: "avx512"}


def simd_tier() -> str:
    return SIMD_TIERS[lib().oxb_simd_tier()]


def simd_set_tier(tier: int) -> int:
    """Lower (or restore) the SIMD tier of the CPU baseline: 0 scalar, 1 AVX2+FMA, 2 AVX-512.  Returns the tier in use,
    -1 when the host CPU lacks the requested one."""
    return lib().oxb_simd_set_tier(int(tier))


def set_threads(n: int) -> None:
    """Threads for the row loops of the scalar kernels (0 = all cores); results do not depend on it."""
    lib().oxb_oracle_set_threads(n)


def simd_threads() -> int:
    return lib().oxb_simd_threads()


def rms_norm(x, w, eps: float) -> np.ndarray:
    xv, wv = _vec(x), _vec(w)
    out = np.empty_like(xv)
    lib().oxb_rms_norm(_f32(xv), _f32(wv), _f32(out), xv.size, eps)
    return out


def silu(x: float) -> float:
    return float(lib().oxb_silu(float(x)))


def swiglu(gate, up) -> np.ndarray:
    g, u = _vec(gate), _vec(up)
    out = np.empty_like(g)
    lib().oxb_swiglu(_f32(g), _f32(u), _f32(out), g.size)
    return out


def softmax(v) -> np.ndarray:
    a = _vec(v).copy()
    lib().oxb_softmax(_f32(a), a.size)
    return a


def rope_table(head_dim: int, max_seq: int, base: float):
    half = head_dim // 2
    c = np.empty((max_seq, half), dtype=np.float32)
    s = np.empty((max_seq, half), dtype=np.float32)
    lib().oxb_rope_table(_f32(c), _f32(s), head_dim, max_seq, base)
    return c, s


def rope_apply(v, cos_row, sin_row) -> np.ndarray:
    a, c, s = _vec(v), _vec(cos_row), _vec(sin_row)
    out = np.empty_like(a)
    lib().oxb_rope_apply(_f32(a), _f32(out), _f32(c), _f32(s), a.size // 2)
    return out


def attention_head(q, keys, values, seq_len: int, head_dim: int) -> np.ndarray:
    qv, kv, vv = _vec(q), _vec(keys).reshape(-1), _vec(values).reshape(-1)
    out = np.empty(head_dim, dtype=np.float32)
    lib().oxb_attention_head(_f32(qv), _f32(kv), _f32(vv), _f32(out), seq_len, head_dim)
    return out


def in_window(key: int, query: int, window: int, sinks: int) -> bool:
    """is_in_window (crates/oxibonsai-model/src/layers/sliding_window.rs:173-189)."""
    return bool(lib().oxb_in_window(key, query, window, sinks))


def attention_head_windowed(q, keys, values, seq_len: int, head_dim: int, window: int, sinks: int) -> np.ndarray:
    qv, kv, vv = _vec(q), _vec(keys).reshape(-1), _vec(values).reshape(-1)
    out = np.empty(head_dim, dtype=np.float32)
    lib().oxb_attention_head_windowed(_f32(qv), _f32(kv), _f32(vv), _f32(out), seq_len, head_dim, window, sinks)
    return out


KV_F32, KV_F16, KV_I8, KV_FP8_E4M3, KV_FP8_E5M2 = range(5)


def fp8_encode(x, e5m2: bool = False) -> np.ndarray:
    """fp8_e4m3_encode / fp8_e5m2_encode (crates/oxibonsai-core/src/quant_fp8.rs:47-160, 208-301), elementwise."""
    a = _vec(x)
    f = lib().oxb_fp8_e5m2_encode if e5m2 else lib().oxb_fp8_e4m3_encode
    return np.array([f(float(v)) for v in a], dtype=np.uint8)


def fp8_decode(codes, e5m2: bool = False) -> np.ndarray:
    f = lib().oxb_fp8_e5m2_decode if e5m2 else lib().oxb_fp8_e4m3_decode
    return np.array([f(int(c)) for c in np.asarray(codes, dtype=np.uint8).reshape(-1)], dtype=np.float32)


def kv_quantize_row(mode: int, row):
    """quantize_row_i8 / quantize_row_fp8 (crates/oxibonsai-model/src/kv_cache_quant.rs:46-62, 519-540) -> (codes, scale)."""
    a = _vec(row)
    codes = np.empty(a.size, dtype=np.uint8)
    scale = C.c_float(0.0)
    _check(lib().oxb_kv_quantize_row(mode, _f32(a), a.size, _u8(codes), C.byref(scale)))
    return codes, np.float32(scale.value)


def kv_dequantize_row(mode: int, codes, scale) -> np.ndarray:
    c = np.ascontiguousarray(codes, dtype=np.uint8).reshape(-1)
    out = np.empty(c.size, dtype=np.float32)
    _check(lib().oxb_kv_dequantize_row(mode, _u8(c), c.size, float(scale), _f32(out)))
    return out


def argmax_last(v) -> int:
    a = _vec(v)
    return int(lib().oxb_argmax_last(_f32(a), a.size))


def sample(logits, temperature: float, top_k: int, top_p: float, rng_state: int):
    """Sampler::sample (crates/oxibonsai-runtime/src/sampling.rs:84-177) -> (token, new rng state, candidate ids,
    candidate probabilities, random draw); the last three are empty / None for the greedy branch."""
    a = _vec(logits)
    st = C.c_uint64(rng_state)
    cap = a.size
    ci, cp = np.zeros(cap, dtype=np.uint32), np.zeros(cap, dtype=np.float32)
    nc, r = C.c_size_t(0), C.c_float(0.0)
    tok = lib().oxb_sample(_f32(a), a.size, temperature, top_k, top_p, C.byref(st), ci.ctypes.data_as(C.POINTER(C.c_uint32)),
                           _f32(cp), cap, C.byref(nc), C.byref(r))
    return int(tok), int(st.value), ci[:nc.value].copy(), cp[:nc.value].copy(), (float(r.value) if nc.value else None)


def argmax_first(v) -> int:
    a = _vec(v)
    return int(lib().oxb_argmax_first(_f32(a), a.size))


# ---------------------------------------------------------------------------
# Whole-model decode (oxb_forward_ex).  The ctypes structs mirror oxb_oracle.h.
# ---------------------------------------------------------------------------
class _Linear(C.Structure):
    _fields_ = [("blocks", C.POINTER(C.c_uint8)), ("n_rows", C.c_size_t), ("k", C.c_size_t)]


class _Layer(C.Structure):
    _fields_ = [("attn_norm", C.POINTER(C.c_float)), ("q_norm", C.POINTER(C.c_float)),
                ("k_norm", C.POINTER(C.c_float)), ("ffn_norm", C.POINTER(C.c_float)),
                ("q", _Linear), ("k", _Linear), ("v", _Linear), ("o", _Linear),
                ("gate", _Linear), ("up", _Linear), ("down", _Linear)]


class _Model(C.Structure):
    _fields_ = [("fmt", C.c_int)] + [(n, C.c_size_t) for n in
                                      ("n_layers", "h", "inter", "nq", "nkv", "hd", "vocab", "max_seq")] + \
               [("eps", C.c_float), ("rope_theta", C.c_float), ("layers", C.POINTER(_Layer)),
                ("final_norm", C.POINTER(C.c_float)), ("lm_head", _Linear), ("kv_mode", C.c_int),
                ("window", C.c_size_t), ("sinks", C.c_size_t)]


class OracleModel:
    """CPU decode of a synthetic Qwen3-shaped model held as reference AoS blocks.

    ``weights`` is the dict produced by ``oxibonsai_amd.synth.make_model``:
    per layer ``attn_norm, q_norm, k_norm, ffn_norm`` (f32 arrays) and
    ``q, k, v, o, gate, up, down`` (uint8 AoS block arrays), plus
    ``final_norm`` and ``lm_head``.
    """

    def __init__(self, cfg: dict, weights: dict, kv_f16: bool = False, dot_f64: bool = False, kv_mode: int = None,
                 window: int = 0, sinks: int = 0, simd: bool = False):
        """dot_f64: every linear layer sums in double (not the reference's arithmetic; a yardstick for how far the
        fp32 summation order moves the result at a given model size).  simd: the linear layers run on the CPU SIMD
        tier (the reference's AVX-512 / AVX2 kernels as restated in oxb_simd.cpp, which the tests hold to the scalar
        kernels) - what makes prompts of thousands of tokens at the 8B shape affordable.  kv_mode: one of KV_* (default f32, or f16 with
        kv_f16); window / sinks: sliding-window attention (window 0 = every earlier position is visible)."""
        if kv_mode is None:
            kv_mode = KV_F16 if kv_f16 else KV_F32
        self.kv_mode = kv_mode
        self.cfg = cfg
        self._keep = []
        assert not (dot_f64 and simd)
        fmt = cfg["fmt"] + (2 if dot_f64 else 0) + (4 if simd else 0)
        h, inter, nq, nkv, hd = cfg["h"], cfg["inter"], cfg["nq"], cfg["nkv"], cfg["hd"]

        def lin(arr, n_rows, k):
            a = _bytes(arr)
            self._keep.append(a)
            return _Linear(_u8(a), n_rows, k)

        def vec(arr):
            a = _vec(arr)
            self._keep.append(a)
            return _f32(a)

        layers = (_Layer * cfg["n_layers"])()
        for i, lw in enumerate(weights["layers"]):
            layers[i] = _Layer(vec(lw["attn_norm"]), vec(lw["q_norm"]), vec(lw["k_norm"]), vec(lw["ffn_norm"]),
                               lin(lw["q"], nq * hd, h), lin(lw["k"], nkv * hd, h), lin(lw["v"], nkv * hd, h),
                               lin(lw["o"], h, nq * hd), lin(lw["gate"], inter, h), lin(lw["up"], inter, h),
                               lin(lw["down"], h, inter))
        self._layers = layers
        self._model = _Model(fmt, cfg["n_layers"], h, inter, nq, nkv, hd, cfg["vocab"], cfg["max_seq"],
                             cfg["eps"], cfg["rope_theta"], layers, vec(weights["final_norm"]),
                             lin(weights["lm_head"], cfg["vocab"], h), kv_mode, window, sinks)
        self._state = lib().oxb_state_new(C.byref(self._model))

    def forward(self, hidden, pos: int, want_normed: bool = False, want_logits: bool = True):
        hv = _vec(hidden)
        logits = np.empty(self.cfg["vocab"], dtype=np.float32) if want_logits else None
        normed = np.empty(self.cfg["h"], dtype=np.float32)
        _check(lib().oxb_forward_ex(C.byref(self._model), self._state, _f32(hv), pos,
                                    _f32(logits) if want_logits else None, _f32(normed)))
        return (logits, normed) if want_normed else logits

    def forward_batch(self, hidden, pos_start: int, want_logits: bool = True):
        """n consecutive positions of the sequence at once (hidden [n][h]), layer by layer: the values of n forward
        calls in a row.  Returns the last position's logits (or None)."""
        hv = np.ascontiguousarray(hidden, dtype=np.float32).reshape(-1, self.cfg["h"])
        logits = np.empty(self.cfg["vocab"], dtype=np.float32) if want_logits else None
        _check(lib().oxb_forward_batch(C.byref(self._model), self._state, _f32(hv), pos_start, hv.shape[0],
                                       _f32(logits) if want_logits else None, None))
        return logits

    def cache(self):
        """K and V as attention reads them, [layer][kv_head][max_seq][hd] f32; for a quantised cache also the codes
        (uint8, same shape) and the scales [layer][kv_head][max_seq]: (k, v, k_codes, v_codes, k_scale, v_scale)."""
        c = self.cfg
        shape = (c["n_layers"], c["nkv"], c["max_seq"], c["hd"])
        n = int(np.prod(shape))
        def view(which, ctype, count, dtype, shp):
            ptr = lib().oxb_state_cache(self._state, which)
            if not ptr:
                return None
            return np.ctypeslib.as_array(C.cast(ptr, C.POINTER(ctype)), shape=(count,)).view(dtype).reshape(shp).copy()

        return (view(0, C.c_float, n, np.float32, shape), view(1, C.c_float, n, np.float32, shape),
                view(2, C.c_uint8, n, np.uint8, shape), view(3, C.c_uint8, n, np.uint8, shape),
                view(4, C.c_float, n // c["hd"], np.float32, shape[:3]), view(5, C.c_float, n // c["hd"], np.float32, shape[:3]))

    def cache_rows(self, layer: int, kv_head: int, pos0: int, n: int):
        """Rows pos0 .. pos0 + n - 1 of one (layer, kv head) as attention reads them -> (k, v), f32 [n][hd] copies
        (cache() copies the whole cache, which at a context of 32 768 is gigabytes)."""
        c = self.cfg
        assert pos0 + n <= c["max_seq"]
        off = ((layer * c["nkv"] + kv_head) * c["max_seq"] + pos0) * c["hd"]
        out = []
        for which in (0, 1):
            base = lib().oxb_state_cache(self._state, which)
            ptr = C.cast(base + off * 4, C.POINTER(C.c_float))
            out.append(np.ctypeslib.as_array(ptr, shape=(n * c["hd"],)).reshape(n, c["hd"]).copy())
        return out[0], out[1]

    def load_rows(self, layer: int, kv_head: int, pos0: int, k_rows, v_rows):
        """Cache rows as attention shall read them (f32 [n][hd]), e.g. the rows another implementation stored."""
        k = np.ascontiguousarray(k_rows, dtype=np.float32)
        v = np.ascontiguousarray(v_rows, dtype=np.float32)
        assert k.shape == v.shape and k.shape[1] == self.cfg["hd"] and pos0 + k.shape[0] <= self.cfg["max_seq"]
        lib().oxb_state_load_rows(C.byref(self._model), self._state, layer, kv_head, pos0, k.shape[0], _f32(k), _f32(v))

    def freeze(self, frozen: bool = True):
        """While frozen a forward stores nothing: attention runs over the rows given by load_rows."""
        lib().oxb_state_freeze(self._state, 1 if frozen else 0)

    def reset(self):
        lib().oxb_state_free(self._state)
        self._state = lib().oxb_state_new(C.byref(self._model))

    def __del__(self):
        try:
            if self._state:
                lib().oxb_state_free(self._state)
                self._state = None
        except Exception:
            pass
