"""Shared builders for the tests: reference-style blocks and the reference's own test generators."""
from __future__ import annotations

import numpy as np

Q1, TQ2 = 0, 1


def f16_bits(v: float) -> int:
    return int(np.array([v], dtype=np.float32).astype(np.float16).view(np.uint16)[0])


def q1_block(scale: float, bits) -> np.ndarray:
    """make_block / make_q1_block of the reference tests: [d f16 LE][16 B]
    (crates/oxibonsai-kernels/src/gemv.rs:94-99, tests/gpu_backend_tests.rs:282-290)."""
    b = np.zeros(18, dtype=np.uint8)
    h = f16_bits(scale)
    b[0], b[1] = h & 0xFF, h >> 8
    b[2:] = np.asarray(bits, dtype=np.uint8) if np.ndim(bits) else np.full(16, bits, dtype=np.uint8)
    return b


def tq2_block(scale: float, qs) -> np.ndarray:
    """make_g128_block of the reference tests: [32 B codes][d f16 LE]
    (crates/oxibonsai-kernels/src/gemv_ternary.rs:196-203)."""
    b = np.zeros(34, dtype=np.uint8)
    b[:32] = np.asarray(qs, dtype=np.uint8) if np.ndim(qs) else np.full(32, qs, dtype=np.uint8)
    h = f16_bits(scale)
    b[32], b[33] = h & 0xFF, h >> 8
    return b


def block(fmt: int, scale: float, pattern) -> np.ndarray:
    return q1_block(scale, pattern) if fmt == Q1 else tq2_block(scale, pattern)


def cross_tier_q1(n_rows: int, k: int) -> np.ndarray:
    """Generator of crates/oxibonsai-kernels/tests/cross_tier.rs:18-27:
    block i has scale 0.3 + 0.02 i and bits[j] = (37 i + 13 j + 7) & 0xFF."""
    n = n_rows * (k // 128)
    out = np.zeros((n, 18), dtype=np.uint8)
    for i in range(n):
        out[i] = q1_block(0.3 + 0.02 * i, [(37 * i + 13 * j + 7) & 0xFF for j in range(16)])
    return out.reshape(-1)


def simd_parity_tq2(n_rows: int, k: int):
    """Generator of the reference's SIMD-vs-scalar TQ2 test (crates/oxibonsai-kernels/src/simd_avx2.rs:1147-1160):
    qs = (17 r + 29 b + 11 i) & 0xFF, d = 0.25 + 0.01 r, x = ((7 i % 23) * 0.125) - 1.5."""
    bpr = k // 128
    out = np.zeros((n_rows * bpr, 34), dtype=np.uint8)
    for r in range(n_rows):
        for b in range(bpr):
            out[r * bpr + b] = tq2_block(0.25 + 0.01 * r, [(17 * r + 29 * b + 11 * i) & 0xFF for i in range(32)])
    x = np.array([((7 * i) % 23) * 0.125 - 1.5 for i in range(k)], dtype=np.float32)
    return out.reshape(-1), x


def metal_tq2(n_rows: int, k: int) -> np.ndarray:
    """Codes from the base-3 digits of 31 r + 17 b + byte, as the reference's Metal GEMV test builds them
    (crates/oxibonsai-kernels/src/gpu_backend/metal_graph/tests.rs:481-500); scale 0.01 (1 + (r + b) % 7)."""
    bpr = k // 128
    out = np.zeros((n_rows * bpr, 34), dtype=np.uint8)
    for r in range(n_rows):
        for b in range(bpr):
            qs = []
            for byte in range(32):
                v = 31 * r + 17 * b + byte
                code = 0
                for lane in range(4):
                    code |= (v % 3) << (2 * lane)
                    v //= 3
                qs.append(code)
            out[r * bpr + b] = tq2_block(0.01 * (1 + (r + b) % 7), qs)
    return out.reshape(-1)


def dense_f64(fmt: int, blocks: np.ndarray, n_rows: int, k: int) -> np.ndarray:
    """Independent float64 decode straight from the format definition (not through the oracle)."""
    bpr = k // 128
    if fmt == Q1:
        b = blocks.reshape(n_rows * bpr, 18)
        d = b[:, 0:2].copy().view(np.float16).astype(np.float64).reshape(-1, 1)
        bits = np.unpackbits(b[:, 2:], axis=1, bitorder="little").astype(np.float64)
        w = d * (2.0 * bits - 1.0)
    else:
        b = blocks.reshape(n_rows * bpr, 34)
        d = b[:, 32:34].copy().view(np.float16).astype(np.float64).reshape(-1, 1)
        codes = np.stack([(b[:, :32] >> s) & 3 for s in (0, 2, 4, 6)], axis=-1).reshape(-1, 128)
        w = d * np.array([-1.0, 0.0, 1.0, 0.0])[codes]
    return w.reshape(n_rows, k)


def rel_err(a: np.ndarray, b: np.ndarray) -> np.ndarray:
    """The reference's parity formula |a-b| / max(|a|, |b|, 1e-3)
    (crates/oxibonsai-model/tests/metal_prefill_ternary_parity_tests.rs:297-298)."""
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    return np.abs(a - b) / np.maximum(np.maximum(np.abs(a), np.abs(b)), 1e-3)


def parity_violations(a: np.ndarray, b: np.ndarray, tol: float = 1e-3) -> int:
    """Number of elements failing the reference's gate `abs_err < tol || rel_err < tol`
    (crates/oxibonsai-model/tests/metal_prefill_ternary_parity_tests.rs:294-308)."""
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    abs_err = np.abs(a - b)
    return int(np.count_nonzero(~((abs_err < tol) | (rel_err(a, b) < tol)) | ~np.isfinite(a) | ~np.isfinite(b)))


from oxibonsai_amd.gguf import GGUF_F16, GGUF_F32, GGUF_MAGIC, GGUF_Q1, GGUF_TQ2, gguf_bytes, model_gguf  # noqa: E402,F401


class DeviceBuffer:
    """A device allocation made through the HIP runtime the library itself links (libamdhip64.so.7), for the
    entry points that take device pointers; no second runtime (torch ships its own) enters the process."""
    _hip = None

    @classmethod
    def hip(cls):
        if cls._hip is None:
            import ctypes as C
            h = C.CDLL("libamdhip64.so.7")
            h.hipMalloc.argtypes = [C.POINTER(C.c_void_p), C.c_size_t]
            h.hipFree.argtypes = [C.c_void_p]
            h.hipMemcpy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int]
            h.hipMemset.argtypes = [C.c_void_p, C.c_int, C.c_size_t]
            h.hipDeviceSynchronize.argtypes = []
            h.hipMemGetInfo.argtypes = [C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)]
            cls._hip = h
        return cls._hip

    def __init__(self, nbytes: int):
        import ctypes as C
        p = C.c_void_p(0)
        assert self.hip().hipMalloc(C.byref(p), max(int(nbytes), 16)) == 0, "hipMalloc failed"
        self.ptr, self.nbytes = p.value, int(nbytes)

    @classmethod
    def from_numpy(cls, a: np.ndarray) -> "DeviceBuffer":
        a = np.ascontiguousarray(a)
        b = cls(a.nbytes)
        assert cls.hip().hipMemcpy(b.ptr, a.ctypes.data, a.nbytes, 1) == 0       # hipMemcpyHostToDevice
        return b

    def fill(self, byte: int) -> None:
        assert self.hip().hipMemset(self.ptr, byte, self.nbytes) == 0
        assert self.hip().hipDeviceSynchronize() == 0

    def to_numpy(self, dtype, shape) -> np.ndarray:
        out = np.empty(shape, dtype=dtype)
        assert out.nbytes <= self.nbytes
        assert self.hip().hipDeviceSynchronize() == 0
        assert self.hip().hipMemcpy(out.ctypes.data, self.ptr, out.nbytes, 2) == 0     # hipMemcpyDeviceToHost
        return out

    def free(self) -> None:
        if self.ptr:
            self.hip().hipFree(self.ptr)
            self.ptr = 0
