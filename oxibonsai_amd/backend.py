"""Host-side mirror of the reference's GPU backend interface for the sub-2-bit path.

``NativeHipBackend`` carries the method names, argument meaning and error
behaviour of ``GpuBackendTrait`` (crates/oxibonsai-kernels/src/gpu_backend/mod.rs:358-534)
as the reference's ``NativeCudaBackend`` implements it
(gpu_backend/cuda_graph/nativecudabackend_traits.rs:29-188); every method is a
thin call into the C ABI of ``liboxb_hip.so``.  A Rust ``impl GpuBackendTrait``
would make exactly these calls through ``extern "C"``.
"""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import _lib
from .synth import BLOCK_BYTES, Q1, QK, TQ2

_STATUS_NAMES = {1: "NotAvailable", 2: "OutOfMemory", 3: "KernelLaunch", 4: "SyncFailed",
                 5: "InvalidArgument", 6: "WeightNotFound"}


class GpuError(Exception):
    """GpuError (gpu_backend/mod.rs:317-342); ``kind`` is the enum variant's name."""

    def __init__(self, code: int, message: str):
        self.code = code
        self.kind = _STATUS_NAMES.get(code, f"Status{code}")
        super().__init__(f"{self.kind}: {message}")


def _check(rc: int) -> None:
    if rc != 0:
        raise GpuError(rc, _lib.last_error())


def _u8(a: np.ndarray):
    return a.ctypes.data_as(_lib.u8p)


def _f32(a: np.ndarray):
    return a.ctypes.data_as(_lib.f32p)


def _as_bytes(b) -> np.ndarray:
    if isinstance(b, np.ndarray):
        return np.ascontiguousarray(b.reshape(-1).view(np.uint8))
    return np.frombuffer(bytes(b), dtype=np.uint8)


class GpuWeightHandle(int):
    """Opaque u64 id of a resident weight (crates/oxibonsai-kernels/src/weight_cache.rs:13-21)."""

    def id(self) -> int:
        return int(self)


class NativeHipBackend:
    """MI355X tier behind the reference's backend trait."""

    def __init__(self, device: int = 0):
        self._lib = _lib.lib()
        _check(self._lib.oxb_hip_init(device))
        self._device = device

    # -- identity -----------------------------------------------------------
    def name(self) -> str:
        return "native-hip"

    def is_accelerated(self) -> bool:
        return True

    def device_count(self) -> int:
        return int(self._lib.oxb_hip_device_count())

    def device_name(self) -> str:
        buf = C.create_string_buffer(256)
        _check(self._lib.oxb_hip_device_info(buf, 256, None, None))
        return buf.value.decode()

    def synchronize(self, device_id: int = 0) -> None:
        _check(self._lib.oxb_hip_synchronize())

    def memory_info(self, device_id: int = 0) -> tuple[int, int]:
        """(free, total) bytes."""
        f, t = C.c_size_t(0), C.c_size_t(0)
        _check(self._lib.oxb_hip_device_info(None, 0, C.byref(f), C.byref(t)))
        return int(f.value), int(t.value)

    # -- uncached -------------------------------------------------------------
    def gemv_q1_g128(self, block_bytes, input, n_rows: int, k: int) -> np.ndarray:
        return self._oneshot(self._lib.oxb_hip_gemv_q1_g128, block_bytes, input, n_rows, k)

    def gemv_tq2_g128(self, block_bytes, input, n_rows: int, k: int) -> np.ndarray:
        return self._oneshot(self._lib.oxb_hip_gemv_tq2_g128, block_bytes, input, n_rows, k)

    def _oneshot(self, fn, block_bytes, input, n_rows, k):
        b = _as_bytes(block_bytes)
        x = np.ascontiguousarray(input, dtype=np.float32)
        y = np.zeros(n_rows, dtype=np.float32)
        _check(fn(_u8(b), b.size, _f32(x), x.size, _f32(y), y.size, n_rows, k))
        return y

    def gemm_q1_g128(self, block_bytes, input, m: int, n_rows: int, k: int, exact: bool | None = None) -> np.ndarray:
        """[m x k] inputs -> [m x n_rows] (mod.rs:425-440).  m > 16 runs the fp16 matrix-core prefill GEMM
        (activations rounded to fp16); m <= 16 or ``exact=True`` streams the weights once per two input rows
        through the GEMV kernel with fp32-exact products, like the reference's per-row loop."""
        return self._oneshot_gemm(Q1, block_bytes, input, m, n_rows, k, exact)

    def gemm_tq2_g128(self, block_bytes, input, m: int, n_rows: int, k: int, exact: bool | None = None) -> np.ndarray:
        return self._oneshot_gemm(TQ2, block_bytes, input, m, n_rows, k, exact)

    def _oneshot_gemm(self, fmt, block_bytes, input, m, n_rows, k, exact=None):
        x = np.ascontiguousarray(input, dtype=np.float32).reshape(-1)
        if k % QK != 0:
            raise GpuError(5, f"invalid argument: k={k} is not a multiple of 128")
        if x.size < m * k:
            raise GpuError(5, f"invalid argument: input holds {x.size} values, {m * k} needed")
        h = self._upload(fmt, block_bytes, n_rows, k)
        try:
            if exact is None:
                exact = m <= 16
            if exact:
                return self._gemv_cached(h, x[:m * k], n_rows, k, m)
            return self.gemm_cached(h, x[:m * k], m, n_rows, k)
        finally:
            self.free_weights(h)

    def gemm_cached(self, handle: int, input, m: int, n_rows: int, k: int) -> np.ndarray:
        """Prefill GEMM on a resident weight: fp16 matrix cores, fp32 accumulation."""
        x = np.ascontiguousarray(input, dtype=np.float32).reshape(-1)
        if x.size != m * k:
            raise GpuError(5, f"invalid argument: input holds {x.size} values, {m * k} needed")
        y = np.empty((m, n_rows), dtype=np.float32)
        _check(self._lib.oxb_hip_gemm(int(handle), _f32(x), _f32(y), m, n_rows, k))
        return y

    # -- resident weights -------------------------------------------------------
    def upload_weights_raw(self, block_bytes, n_rows: int | None = None, k: int | None = None,
                           handle_id: int = 0) -> GpuWeightHandle:
        """Q1_0_g128 AoS bytes -> resident handle (GpuBackendTrait::upload_weights_raw, gpu_backend/mod.rs:445).
        As in the reference the bytes are enough: the shape then comes with the first cached GEMV / GEMM call or
        with the model that names the handle.  Giving (n_rows, k) here binds it at once."""
        return self._upload(Q1, block_bytes, n_rows, k, handle_id)

    def upload_weights_ternary(self, blocks, n_rows: int | None = None, k: int | None = None,
                               handle_id: int = 0) -> GpuWeightHandle:
        """TQ2_0_g128 blocks (struct byte order [qs 32][d]) -> resident handle (upload_weights_ternary,
        gpu_backend/mod.rs:472); the shape is optional as in upload_weights_raw."""
        return self._upload(TQ2, blocks, n_rows, k, handle_id)

    def _upload(self, fmt, block_bytes, n_rows, k, handle_id=0):
        b = _as_bytes(block_bytes)
        hid = C.c_uint64(handle_id)
        if n_rows is None and k is None:
            fn = self._lib.oxb_hip_upload_q1_raw if fmt == Q1 else self._lib.oxb_hip_upload_tq2_raw
            _check(fn(C.byref(hid), _u8(b), b.size))
            return GpuWeightHandle(hid.value)
        if n_rows is None or k is None:
            raise GpuError(5, "invalid argument: give both n_rows and k, or neither")
        fn = self._lib.oxb_hip_upload_q1 if fmt == Q1 else self._lib.oxb_hip_upload_tq2
        _check(fn(C.byref(hid), _u8(b), b.size, n_rows, k))
        return GpuWeightHandle(hid.value)

    def free_weights(self, handle: int) -> None:
        _check(self._lib.oxb_hip_free_weight(int(handle)))

    def gemv_q1_g128_cached(self, handle: int, input, n_rows: int, k: int) -> np.ndarray:
        return self._gemv_cached(handle, input, n_rows, k, 1)[0]

    def gemv_tq2_g128_cached(self, handle: int, input, n_rows: int, k: int) -> np.ndarray:
        return self._gemv_cached(handle, input, n_rows, k, 1)[0]

    def gemv_cached_batch(self, handle: int, inputs, n_rows: int, k: int) -> np.ndarray:
        """[batch x k] -> [batch x n_rows] on resident weights."""
        x = np.ascontiguousarray(inputs, dtype=np.float32)
        return self._gemv_cached(handle, x.reshape(-1), n_rows, k, x.size // k)

    def _gemv_cached(self, handle, input, n_rows, k, batch):
        x = np.ascontiguousarray(input, dtype=np.float32).reshape(-1)
        if x.size < batch * k:
            raise GpuError(5, f"invalid argument: input holds {x.size} values, {batch * k} needed")
        y = np.zeros((batch, n_rows), dtype=np.float32)
        _check(self._lib.oxb_hip_gemv(int(handle), _f32(x), _f32(y), n_rows, k, batch))
        return y

    def dequant(self, handle: int) -> np.ndarray:
        """fp32 [n_rows x k] decoded on the device from the resident layout."""
        fmt, nr, k, nb = C.c_int(0), C.c_uint32(0), C.c_uint32(0), C.c_size_t(0)
        _check(self._lib.oxb_hip_weight_info(int(handle), C.byref(fmt), C.byref(nr), C.byref(k), C.byref(nb)))
        out = np.empty((nr.value, k.value), dtype=np.float32)
        _check(self._lib.oxb_hip_dequant(int(handle), _f32(out), out.size))
        return out


# -- host-only repack (no GPU needed) -------------------------------------------
def repack(fmt: int, block_bytes, n_rows: int, k: int) -> tuple[np.ndarray, np.ndarray]:
    """AoS blocks -> (codes, scales) sections of the resident layout, as uint8 arrays."""
    L = _lib.lib()
    b = _as_bytes(block_bytes)
    cb, sb = C.c_size_t(0), C.c_size_t(0)
    _check(L.oxb_hip_repack_sizes(fmt, n_rows, k, C.byref(cb), C.byref(sb)))
    codes = np.zeros(cb.value, dtype=np.uint8)
    scales = np.zeros(sb.value, dtype=np.uint8)
    _check(L.oxb_hip_repack(fmt, _u8(b), b.size, n_rows, k, _u8(codes), codes.size, _u8(scales), scales.size))
    return codes, scales


def unpack(fmt: int, codes: np.ndarray, scales: np.ndarray, n_rows: int, k: int) -> np.ndarray:
    L = _lib.lib()
    out = np.zeros(n_rows * (k // QK) * BLOCK_BYTES[fmt], dtype=np.uint8)
    _check(L.oxb_hip_unpack(fmt, _u8(codes), codes.size, _u8(scales), scales.size, n_rows, k, _u8(out), out.size))
    return out
