"""The allocation-free GEMM entry point (oxb_hip_gemm_dev_static) against oxb_hip_gemm_dev, through the C ABI.

Same kernels and launch plan, so the results must be equal bit for bit; the second call of each pair is smaller than
the first and runs on the scratch the first call left behind."""
import ctypes as C

import numpy as np
import pytest

from helpers import Q1, TQ2, DeviceBuffer
from oxibonsai_amd import _lib, synth

pytestmark = pytest.mark.gpu


def _both(L, h, x, m, n, k):
    d_x = DeviceBuffer.from_numpy(x)
    d_y = DeviceBuffer(m * n * 4)
    outs = []
    try:
        for fn in (L.oxb_hip_gemm_dev, L.oxb_hip_gemm_dev_static):
            d_y.fill(0xFF)                              # NaN patterns: every output must be written by the call
            rc = fn(int(h), d_x.ptr, d_y.ptr, m, n, k)
            assert rc == 0, _lib.last_error()
            assert L.oxb_hip_synchronize() == 0
            outs.append(d_y.to_numpy(np.float32, (m, n)))
    finally:
        d_x.free()
        d_y.free()
    return outs


@pytest.mark.parametrize("fmt,shapes", [
    (TQ2, [(512, 2560, 9728), (130, 250, 1152)]),      # wide kernel with a K split, then a ragged small case
    (Q1, [(300, 4096, 4096), (20, 4100, 1152)]),       # wide kernel, then the narrow (few token rows) kernel
    (Q1, [(64, 333, 640), (1, 16, 128)]),
])
def test_static_scratch_gemm_equals_the_allocating_entry_point(backend, fmt, shapes):
    L = _lib.lib()
    for i, (m, n, k) in enumerate(shapes):             # two calls in a row, the second one smaller
        a = synth.make_blocks(fmt, 50 + i + n, n, k)
        x = synth.normal_f32(60 + i + k, m * k).reshape(m, k)
        h = backend.upload_weights_raw(a, n, k) if fmt == Q1 else backend.upload_weights_ternary(a, n, k)
        try:
            want, got = _both(L, h, x, m, n, k)
        finally:
            backend.free_weights(h)
        assert np.all(np.isfinite(want))
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (fmt, m, n, k)


def test_static_scratch_gemm_rejects_what_does_not_fit(backend):
    L = _lib.lib()
    n, k, m = 256, 4096, 4096                           # packed activations alone: 32 * 16 * 4096 * 16 B = 32 MiB + the rest
    a = synth.make_blocks(Q1, 9, n, k)
    h = backend.upload_weights_raw(a, n, k)
    d_x = d_y = None
    try:
        d_x, d_y = DeviceBuffer(m * k * 4), DeviceBuffer(m * n * 4)
        d_x.fill(0)
        rc = L.oxb_hip_gemm_dev_static(int(h), d_x.ptr, d_y.ptr, m, n, k)
        assert rc == 5 and "allocation-free entry point holds" in _lib.last_error()
        assert L.oxb_hip_gemm_dev(int(h), d_x.ptr, d_y.ptr, m, n, k) == 0     # the allocating one takes it
        assert L.oxb_hip_synchronize() == 0
        assert L.oxb_hip_gemm_dev_static(int(h), d_x.ptr, d_y.ptr, 16, n, k) == 0   # and small shapes still run
        assert L.oxb_hip_synchronize() == 0
    finally:
        for b in (d_x, d_y):
            if b is not None:
                b.free()
        backend.free_weights(h)


def _free_bytes() -> int:
    hip = DeviceBuffer.hip()
    free, total = C.c_size_t(0), C.c_size_t(0)
    assert hip.hipMemGetInfo(C.byref(free), C.byref(total)) == 0
    return free.value


def test_static_scratch_gemm_allocates_nothing(backend):
    """What the entry point exists for: the device's free memory is the same before and after a call, also for a
    shape larger than any the entry point has seen in this process (a fallback to the library's growing workspace
    would show here: the probe is first shown to see an allocation of the size in question)."""
    L = _lib.lib()
    n, k, m = 1040, 8192, 900                           # packed activations: 8192 x 1024 halves = 16 MiB of the 32
    a = synth.make_blocks(TQ2, 77, n, k)
    x = synth.normal_f32(78, m * k).reshape(m, k)
    h = backend.upload_weights_ternary(a, n, k)
    d_x, d_y = DeviceBuffer.from_numpy(x), DeviceBuffer(m * n * 4)
    try:
        assert L.oxb_hip_synchronize() == 0
        before = _free_bytes()
        probe = DeviceBuffer(16 << 20)
        assert _free_bytes() < before                   # hipMemGetInfo notices 16 MiB
        probe.free()
        assert _free_bytes() == before
        d_y.fill(0xFF)
        assert L.oxb_hip_gemm_dev_static(int(h), d_x.ptr, d_y.ptr, m, n, k) == 0, _lib.last_error()
        assert L.oxb_hip_synchronize() == 0
        assert _free_bytes() == before
        got = d_y.to_numpy(np.float32, (m, n))
        d_y.fill(0xFF)
        assert L.oxb_hip_gemm_dev(int(h), d_x.ptr, d_y.ptr, m, n, k) == 0, _lib.last_error()
        assert np.array_equal(got.view(np.uint32), d_y.to_numpy(np.float32, (m, n)).view(np.uint32))
    finally:
        d_x.free()
        d_y.free()
        backend.free_weights(h)
