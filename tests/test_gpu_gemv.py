"""GPU parity of the native-hip GEMV path against the CPU oracle, through the C ABI.

Tolerances: decode bit-exact; GEMV within 1e-3 relative under the reference's own gate
(abs_err < 1e-3 || |a-b| / max(|a|, |b|, 1e-3) < 1e-3), tightened here by a bound of
1e-5 of the output scale and by a comparison with the float64 product."""
import numpy as np
import pytest

import oxibonsai_amd as ox
from helpers import (Q1, TQ2, block, cross_tier_q1, dense_f64, metal_tq2, parity_violations, q1_block, rel_err,
                     simd_parity_tq2, tq2_block)
from kernel_model import gemv_f4 as model_gemv_f4
from oracle import oracle
from oxibonsai_amd import synth

pytestmark = pytest.mark.gpu
GEMV_REL_TOL = 1e-3


def _upload(be, fmt, a, n, k):
    return be.upload_weights_raw(a, n, k) if fmt == Q1 else be.upload_weights_ternary(a, n, k)


def _gemv(be, fmt, h, x, n, k):
    return be.gemv_q1_g128_cached(h, x, n, k) if fmt == Q1 else be.gemv_tq2_g128_cached(h, x, n, k)


def test_backend_identity(backend):
    assert backend.name() == "native-hip" and backend.is_accelerated()
    assert backend.device_count() >= 1
    assert "gfx950" in backend.device_name()
    free, total = backend.memory_info()
    assert 0 < free <= total and total > 200 * 2**30
    backend.synchronize()


@pytest.mark.parametrize("fmt", [Q1, TQ2])
@pytest.mark.parametrize("shape", [(1, 128), (16, 512), (17, 640), (100, 2048), (250, 1152)])
def test_dequant_bit_exact(backend, fmt, shape):
    n, k = shape
    a = synth.make_blocks(fmt, 300 + n, n, k)
    h = _upload(backend, fmt, a, n, k)
    try:
        got = backend.dequant(h)
    finally:
        backend.free_weights(h)
    want = oracle.dequant(fmt, a).reshape(n, k)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_dequant_bit_exact_special_codes_and_scales(backend):
    # all 256 code bytes (incl. the reserved 0b11 lanes) and awkward scales (subnormal, max, negative)
    qs = np.arange(256, dtype=np.uint8).reshape(8, 32)
    scales = [1.0, 6e-8, 65504.0, -0.375, 0.0, 3.1e-5, 0.1, 7.0]
    a = np.concatenate([tq2_block(s, qs[i]) for i, s in enumerate(scales)])
    h = backend.upload_weights_ternary(a, 2, 512)
    got = backend.dequant(h)
    backend.free_weights(h)
    assert np.array_equal(got.view(np.uint32), oracle.dequant(TQ2, a).reshape(2, 512).view(np.uint32))
    a = np.concatenate([q1_block(s, qs[i][:16]) for i, s in enumerate(scales)])
    h = backend.upload_weights_raw(a, 4, 256)
    got = backend.dequant(h)
    backend.free_weights(h)
    assert np.array_equal(got.view(np.uint32), oracle.dequant(Q1, a).reshape(4, 256).view(np.uint32))


def test_reference_kats_through_the_abi(backend):
    ones = np.ones(128, np.float32)
    # crates/oxibonsai-kernels/src/gemv.rs:101-150, gpu_backend/mod.rs:1353-1398
    assert abs(backend.gemv_q1_g128(q1_block(1.0, 0xFF), np.arange(128, dtype=np.float32), 1, 128)[0] - 8128.0) < 1.0
    assert abs(backend.gemv_q1_g128(q1_block(2.0, 0x00), ones, 1, 128)[0] + 256.0) < 1.0
    two = np.concatenate([q1_block(1.0, 0xFF), q1_block(1.0, 0x00)])
    y = backend.gemv_q1_g128(two, ones, 2, 128)
    assert abs(y[0] - 128.0) < 1.0 and abs(y[1] + 128.0) < 1.0
    # two blocks per row (tests/gpu_backend_tests.rs:282-376)
    row = np.concatenate([q1_block(0.5, 0xFF), q1_block(0.25, 0x00)])
    assert abs(backend.gemv_q1_g128(row, np.ones(256, np.float32), 1, 256)[0] - (64.0 - 32.0)) < 1e-3
    # crates/oxibonsai-kernels/src/gemv_ternary.rs:212-324
    y = backend.gemv_tq2_g128(np.concatenate([tq2_block(1.0, 0xAA)] * 2), ones, 2, 128)
    assert abs(y[0] - 128.0) < 0.5 and abs(y[1] - 128.0) < 0.5
    y = backend.gemv_tq2_g128(np.concatenate([tq2_block(1.0, 0x00)] * 2), ones, 2, 128)
    assert abs(y[0] + 128.0) < 0.5 and abs(y[1] + 128.0) < 0.5
    assert abs(backend.gemv_tq2_g128(tq2_block(1.0, 0x46), ones, 1, 128)[0]) < 1e-4
    assert abs(backend.gemv_tq2_g128(tq2_block(1.0, 0xFF), ones, 1, 128)[0]) < 1e-4
    y = backend.gemv_tq2_g128(np.concatenate([tq2_block(1.0, 0xAA)] * 8), np.ones(256, np.float32), 4, 256)
    assert np.all(np.abs(y - 256.0) < 1.0)


def test_reference_generators(backend):
    n, k = 128, 1024
    a = cross_tier_q1(n, k)
    x = np.array([(i % 17) * 0.25 - 2.0 for i in range(k)], dtype=np.float32)
    got = backend.gemv_q1_g128(a, x, n, k)
    assert np.max(np.abs(got - oracle.gemv(Q1, a, x, n, k))) < 1.0              # cross_tier.rs tolerance
    assert np.max(rel_err(got, dense_f64(Q1, a, n, k) @ x.astype(np.float64))) < GEMV_REL_TOL
    a, x = simd_parity_tq2(64, 128)
    assert np.mean((backend.gemv_tq2_g128(a, x, 64, 128) - oracle.gemv(TQ2, a, x, 64, 128)) ** 2) < 1e-6
    a = metal_tq2(64, 512)
    x = np.array([((i * 7 + 3) % 19) * 0.1 - 0.9 for i in range(512)], dtype=np.float32)
    assert np.max(np.abs(backend.gemv_tq2_g128(a, x, 64, 512) - oracle.gemv(TQ2, a, x, 64, 512))) < 1e-3


# BASELINE configs 0 and 1 at full size, plus ragged / tiny / very wide shapes.
SHAPES = [
    (TQ2, 12288, 2048), (Q1, 6144, 4096), (Q1, 24576, 4096), (Q1, 4096, 12288),
    (TQ2, 6144, 4096), (TQ2, 4096, 12288),
    (Q1, 1, 128), (TQ2, 1, 128), (Q1, 37, 640), (TQ2, 250, 1152), (Q1, 1000, 2560), (TQ2, 333, 9728),
    (Q1, 48, 12800), (Q1, 40, 20480), (TQ2, 24, 17408),
]


@pytest.mark.parametrize("fmt,n,k", SHAPES)
def test_gemv_matches_oracle(backend, fmt, n, k):
    a = synth.make_blocks(fmt, 1000 + n + k, n, k)
    x = synth.normal_f32(77 + k, k)
    h = _upload(backend, fmt, a, n, k)
    try:
        got = _gemv(backend, fmt, h, x, n, k)
    finally:
        backend.free_weights(h)
    want = oracle.gemv(fmt, a, x, n, k)
    assert parity_violations(got, want, GEMV_REL_TOL) == 0
    scale = np.max(np.abs(want))
    assert np.max(np.abs(got - want)) < 1e-5 * scale                      # far below the gate
    if n * k <= 2**25:                                                     # float64 truth where it is cheap
        truth = dense_f64(fmt, a, n, k) @ x.astype(np.float64)
        assert np.max(np.abs(got - truth)) <= 2 * np.max(np.abs(want - truth)) + 1e-7 * scale


@pytest.mark.parametrize("fmt,n,k", [(Q1, 6144, 4096), (Q1, 4096, 12288), (TQ2, 12288, 2048), (Q1, 50, 384)])
@pytest.mark.parametrize("batch", [2, 5, 8])
def test_gemv_batched_matches_oracle(backend, fmt, n, k, batch):
    a = synth.make_blocks(fmt, 2000 + n, n, k)
    xs = synth.normal_f32(5, batch * k).reshape(batch, k)
    xs[1] *= 1e-3                       # vectors of very different magnitude share a launch
    if batch > 4:
        xs[4] *= 250.0
    h = _upload(backend, fmt, a, n, k)
    try:
        got = backend.gemv_cached_batch(h, xs, n, k)
    finally:
        backend.free_weights(h)
    want = oracle.gemm(fmt, a, xs, batch, n, k)
    for b in range(batch):
        scale = max(np.max(np.abs(want[b])), 1e-30)
        assert np.max(np.abs(got[b] - want[b])) < 1e-5 * scale + 1e-6, b


@pytest.fixture
def packed_from_two():
    """Every batch above one through the route that quantises the vectors in a launch of their own (by default it
    starts at five vectors); the default comes back afterwards."""
    from oxibonsai_amd import _lib
    assert _lib.lib().oxb_hip_set_gemv_packed_min_batch(2) == 0
    yield
    assert _lib.lib().oxb_hip_set_gemv_packed_min_batch(1) == 0


PACKED_SHAPES = [
    (Q1, 24576, 4096), (Q1, 4096, 12288), (Q1, 6144, 4096), (TQ2, 12288, 2048), (TQ2, 2048, 6144),   # the model shapes
    (Q1, 1, 128), (TQ2, 17, 128), (Q1, 37, 640), (TQ2, 250, 1152), (Q1, 1000, 2560), (TQ2, 333, 9728),
    (Q1, 5000, 8192),                      # two superblocks per wave and several tile groups per workgroup
    (TQ2, 4100, 10240),                    # three superblocks per wave, two tiles per workgroup
    (Q1, 48, 12800), (TQ2, 24, 17408),     # K beyond one launch: the following launches accumulate
]


@pytest.mark.parametrize("fmt,n,k", PACKED_SHAPES)
def test_gemv_packed_route_matches_oracle(backend, packed_from_two, fmt, n, k):
    """Two to eight vectors (and nineteen: 8 + 8 + 3) quantised once per GEMV and multiplied in one pass over the
    weights; vectors of very different magnitude share a launch, one vector is all zeros, one ends in a run of
    zeros (a whole superblock without a non-zero value)."""
    a = synth.make_blocks(fmt, 2100 + n, n, k)
    h = _upload(backend, fmt, a, n, k)
    try:
        for batch in (2, 3, 4, 5, 7, 8, 19):
            xs = synth.normal_f32(50 + batch, batch * k).reshape(batch, k)
            xs[1] *= 1e-3
            xs[batch - 1] *= 250.0
            if batch > 2:
                xs[2] = 0.0
            if k >= 1024:
                xs[0, -600:] = 0.0
            got = backend.gemv_cached_batch(h, xs, n, k)
            want = oracle.gemm(fmt, a, xs, batch, n, k)
            for b in range(batch):
                scale = max(np.max(np.abs(want[b])), 1e-30)
                assert np.max(np.abs(got[b] - want[b])) < 1e-5 * scale + 1e-6, (batch, b)
            if batch > 2:
                assert not np.any(got[2])
    finally:
        backend.free_weights(h)


@pytest.mark.parametrize("fmt", [Q1, TQ2])
def test_gemv_packed_route_properties(backend, packed_from_two, fmt):
    n, k = 777, 3072
    a = synth.make_blocks(fmt, 31, n, k)
    h = _upload(backend, fmt, a, n, k)
    try:
        x = np.stack([synth.normal_f32(10 + i, k) for i in range(8)])
        y = backend.gemv_cached_batch(h, x, n, k)
        truth = x.astype(np.float64) @ dense_f64(fmt, a, n, k).T
        assert np.max(np.abs(y - truth)) < 1e-6 * np.max(np.abs(truth))
        assert np.array_equal(backend.gemv_cached_batch(h, x, n, k), y)                       # deterministic
        # a vector's result depends neither on its place in the batch nor on its companions
        perm = [5, 2, 7, 0, 3, 6, 1, 4]
        assert np.array_equal(backend.gemv_cached_batch(h, x[perm], n, k), y[perm])
        assert np.array_equal(backend.gemv_cached_batch(h, x[:3], n, k), y[:3])
        for s in (-100, 66):                                                                  # power-of-two scaling is exact
            xs = x.copy()
            xs[6] = np.ldexp(x[6], s)
            ys = backend.gemv_cached_batch(h, xs, n, k)
            assert np.array_equal(ys[6], np.ldexp(y[6], s).astype(np.float32)), s
            assert np.array_equal(np.delete(ys, 6, 0), np.delete(y, 6, 0))
        # an infinity or a NaN makes every output of its own vector NaN and leaves the other vectors alone
        xb = x.copy()
        xb[1, 5], xb[6, 3000] = np.nan, np.inf
        yb = backend.gemv_cached_batch(h, xb, n, k)
        assert np.all(np.isnan(yb[1])) and np.all(np.isnan(yb[6]))
        assert np.array_equal(np.delete(yb, [1, 6], 0), np.delete(y, [1, 6], 0))
        # both routes are exact up to their fp32 joins: the four-vector route must agree to the last few bits
        from oxibonsai_amd import _lib
        assert _lib.lib().oxb_hip_set_gemv_packed_min_batch(0) == 0
        y4 = backend.gemv_cached_batch(h, x, n, k)
        assert np.max(np.abs(y4 - y)) < 2e-6 * np.max(np.abs(y))
    finally:
        backend.free_weights(h)


@pytest.mark.parametrize("fmt", [Q1, TQ2])
def test_gemv_properties(backend, fmt):
    n, k = 777, 3072
    a = synth.make_blocks(fmt, 31, n, k)
    h = _upload(backend, fmt, a, n, k)
    try:
        x1, x2 = synth.normal_f32(1, k), synth.normal_f32(2, k)
        y1, y2 = _gemv(backend, fmt, h, x1, n, k), _gemv(backend, fmt, h, x2, n, k)
        y12 = _gemv(backend, fmt, h, x1 + x2, n, k)
        assert np.max(np.abs(y12 - (y1 + y2))) < 1e-4                              # linearity
        assert np.array_equal(_gemv(backend, fmt, h, x1, n, k), y1)                # deterministic
        assert np.all(_gemv(backend, fmt, h, np.zeros(k, np.float32), n, k) == 0.0)  # zero input
        for s in (-100, 66):                                                       # power-of-two scaling is exact
            xs = np.ldexp(x1, s).astype(np.float32)
            assert np.array_equal(_gemv(backend, fmt, h, xs, n, k), np.ldexp(y1, s).astype(np.float32)), s
        xbad = x1.copy()
        xbad[5] = np.nan
        assert np.all(np.isnan(_gemv(backend, fmt, h, xbad, n, k)))                 # NaN in -> NaN out
        xo = x1.copy()
        xo[100] = 5000.0                                                            # one massive outlier
        want = dense_f64(fmt, a, n, k) @ xo.astype(np.float64)
        assert np.max(np.abs(_gemv(backend, fmt, h, xo, n, k) - want)) < 1e-6 * np.max(np.abs(want))
        yb = backend.gemv_cached_batch(h, np.stack([x1, x2]), n, k)[1]
        # one vector takes the fp4 route, two and more the int8 route; both are exact up to their fp32 joins
        assert np.max(np.abs(yb - y2)) < 2e-6 * np.max(np.abs(y2))
        yb3 = backend.gemv_cached_batch(h, np.stack([x2, x1, x2]), n, k)
        assert np.array_equal(yb3[0], yb) and np.array_equal(yb3[2], yb)            # a batch row does not depend on its place
    finally:
        backend.free_weights(h)
    zero = a.copy().reshape(-1, 18 if fmt == Q1 else 34)
    zero[:, (0 if fmt == Q1 else 32):(2 if fmt == Q1 else 34)] = 0
    h = _upload(backend, fmt, zero.reshape(-1), n, k)
    assert np.all(_gemv(backend, fmt, h, x1, n, k) == 0.0)                          # zero scale -> 0
    backend.free_weights(h)


def test_error_paths(backend):
    b = q1_block(1.0, 0xFF)
    ones = np.ones(128, np.float32)
    for call in (lambda: backend.gemv_q1_g128(b, np.ones(100, np.float32), 1, 100),   # k % 128
                 lambda: backend.gemv_q1_g128(b, np.ones(64, np.float32), 1, 128),    # short input
                 lambda: backend.gemv_q1_g128(b, ones, 2, 128),                        # short weights
                 lambda: backend.gemv_tq2_g128(tq2_block(1.0, 0xAA), ones, 2, 128),
                 lambda: backend.upload_weights_raw(b, 1, 100)):
        with pytest.raises(ox.GpuError) as e:
            call()
        assert e.value.kind == "InvalidArgument"
    with pytest.raises(ox.GpuError) as e:
        backend.gemv_q1_g128_cached(0xDEAD, ones, 1, 128)
    assert e.value.kind == "WeightNotFound"
    h = backend.upload_weights_raw(b, 1, 128)
    with pytest.raises(ox.GpuError) as e:
        backend.gemv_q1_g128_cached(h, np.ones(256, np.float32), 1, 256)              # shape differs from upload
    assert e.value.kind == "InvalidArgument"
    assert abs(backend.gemv_q1_g128_cached(h, ones, 1, 128)[0] - 128.0) < 1e-3        # still usable afterwards
    backend.free_weights(h)
    with pytest.raises(ox.GpuError) as e:
        backend.free_weights(h)
    assert e.value.kind == "WeightNotFound"


def test_caller_chosen_handle_ids_and_replacement(backend):
    a1, a2 = synth.make_blocks(Q1, 1, 32, 256), synth.make_blocks(Q1, 2, 32, 256)
    x = synth.normal_f32(3, 256)
    h = backend.upload_weights_raw(a1, 32, 256, handle_id=4_000_000)
    assert h == 4_000_000
    y1 = backend.gemv_q1_g128_cached(h, x, 32, 256)
    assert backend.upload_weights_raw(a2, 32, 256, handle_id=4_000_000) == 4_000_000   # replaces
    y2 = backend.gemv_q1_g128_cached(h, x, 32, 256)
    assert np.max(np.abs(y1 - oracle.gemv(Q1, a1, x, 32, 256))) < 1e-5
    assert np.max(np.abs(y2 - oracle.gemv(Q1, a2, x, 32, 256))) < 1e-5
    backend.free_weights(h)


def test_tq2_single_vector_on_an_lm_head_sized_matrix(backend):
    """From 32 row tiles per CU on the single-vector kernel runs two workgroups per CU; ternary weights at that size:
    bit-equal to the numpy model of that route on the tiles compared (the model walks every block in Python), every
    row within 1e-5 of the scalar oracle; power-of-two scaling stays exact; ragged last tile, K of two superblocks
    with the second one partial."""
    n, k = 16 * 32 * 256 + 5, 640
    a = synth.make_blocks(TQ2, 77, n, k)
    x = synth.normal_f32(78, k)
    h = backend.upload_weights_ternary(a, n, k)
    try:
        y = backend.gemv_tq2_g128_cached(h, x, n, k)
        y2 = backend.gemv_tq2_g128_cached(h, np.ldexp(x, 9).astype(np.float32), n, k)
    finally:
        backend.free_weights(h)
    want = oracle.gemv(TQ2, a, x, n, k)
    assert parity_violations(y, want, GEMV_REL_TOL) == 0
    assert np.max(np.abs(y - want)) < 1e-5                      # outputs are O(1): the scalar oracle's own order effects
    assert np.array_equal(y2, np.ldexp(y, 9).astype(np.float32))
    # the model on the first 40, some middle and the last rows: same blocks, row tiles are independent
    nblk = k // 128
    blocks = a.reshape(n, nblk * 34)
    for r0, r1 in ((0, 40), (65536, 65536 + 48), (n - 21, n)):
        sub = np.ascontiguousarray(blocks[r0:r1]).reshape(-1)
        codes, scales = ox.repack(TQ2, sub, r1 - r0, k)
        m = model_gemv_f4(codes, scales, r1 - r0, k, x, TQ2)
        assert np.array_equal(y[r0:r1].view(np.uint32), m.view(np.uint32)), (r0, r1)
