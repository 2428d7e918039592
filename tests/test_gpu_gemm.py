"""GPU parity of the native-hip prefill GEMM (fp16 matrix cores, fp32 accumulation) through the C ABI.

Tolerance: 1e-2 relative under the reference's gate form (abs_err < tol || |a-b| / max(|a|, |b|, 1e-3) < tol),
tightened by the bound the arithmetic implies: weights and products are exact, so an output differs from the
float64 product by at most 2^-11 * sum_k |w_k x_k| (activation rounding to fp16) plus fp32 summation error.
Inputs that are exact in fp16 must give bit-exact results, which pins the k order of both operands."""
import numpy as np
import pytest

from helpers import Q1, TQ2, dense_f64, parity_violations, q1_block, tq2_block
from oracle import oracle
from oxibonsai_amd import GpuError, synth

pytestmark = pytest.mark.gpu
GEMM_REL_TOL = 1e-2


def _upload(be, fmt, a, n, k):
    return be.upload_weights_raw(a, n, k) if fmt == Q1 else be.upload_weights_ternary(a, n, k)


def _gemm(be, fmt, a, x, m, n, k):
    h = _upload(be, fmt, a, n, k)
    try:
        return be.gemm_cached(h, x, m, n, k)
    finally:
        be.free_weights(h)


def _check_against_truth(got, w64, x, extra=0.0):
    """|got - W x| <= 2^-11 sum|w x| + fp32 summation slack, element by element."""
    x64 = x.astype(np.float64)
    truth = x64 @ w64.T
    bound = 2.0 ** -11 * (np.abs(x64) @ np.abs(w64).T)
    slack = 4e-6 * (np.abs(x64) @ np.abs(w64).T) + 1e-30 + extra
    err = np.abs(got.astype(np.float64) - truth)
    bad = err > bound + slack
    assert not bad.any(), f"{int(bad.sum())} outputs beyond the fp16-rounding bound, worst ratio {np.max(err / (bound + slack)):.3f}"
    return truth


@pytest.mark.parametrize("fmt", [Q1, TQ2])
@pytest.mark.parametrize("shape", [(1, 16, 128), (17, 40, 256), (33, 100, 640), (128, 256, 1024), (130, 250, 1152),
                                   (300, 70, 2048), (16, 1, 512), (15, 17, 384), (129, 333, 128),
                                   # few token rows (decode batches): 1, 2 and 4 row tiles per workgroup, K runs
                                   # that do not divide by the eight waves, one and two token tiles
                                   (8, 8200, 256), (32, 16400, 128), (9, 16400, 256), (20, 4100, 1152), (5, 48, 12288), (31, 9000, 1536),
                                   # the one-launch packer of up to 64 rows: its longest row (eight items per thread), one
                                   # block more (two-kernel route), item counts between its instantiations, 64 rows
                                   (5, 100, 16384), (8, 48, 16512), (31, 50, 8576), (64, 33, 6144), (3, 16, 2176)])
def test_gemm_matches_oracle(backend, fmt, shape):
    m, n, k = shape
    a = synth.make_blocks(fmt, 900 + m + n, n, k)
    x = synth.normal_f32(77 + k, m * k).reshape(m, k)
    got = _gemm(backend, fmt, a, x, m, n, k)
    want = oracle.gemm(fmt, a, x, m, n, k)
    assert got.shape == (m, n)
    assert parity_violations(got, want, GEMM_REL_TOL) == 0
    _check_against_truth(got, dense_f64(fmt, a, n, k), x)


@pytest.mark.parametrize("fmt", [Q1, TQ2])
@pytest.mark.parametrize("m,n", [(48, 64), (24, 64), (9, 8208)])
def test_gemm_is_bit_exact_on_fp16_representable_inputs(backend, fmt, m, n):
    # integer activations below 2048 and power-of-two scales: every product and every partial sum is an exact
    # fp32 number, so any disagreement in the k order of the two MFMA operands shows as a wrong integer
    k = 640
    rng = np.random.default_rng(5)
    bpr = k // 128
    blocks = []
    for i in range(n * bpr):
        scale = float(2.0 ** rng.integers(-3, 3))
        blocks.append(q1_block(scale, rng.integers(0, 256, 16, dtype=np.uint8)) if fmt == Q1
                      else tq2_block(scale, rng.integers(0, 256, 32, dtype=np.uint8)))
    a = np.concatenate(blocks)
    x = rng.integers(-2047, 2048, size=(m, k)).astype(np.float32)
    x[:, 0] = 16384.0  # fixes every row's scaling exponent
    got = _gemm(backend, fmt, a, x, m, n, k)
    truth = x.astype(np.float64) @ dense_f64(fmt, a, n, k).T
    assert np.array_equal(got.astype(np.float64), truth)


@pytest.mark.parametrize("fmt", [Q1, TQ2])
def test_gemm_row_scaling_is_exact(backend, fmt):
    m, n, k = 20, 48, 512
    a = synth.make_blocks(fmt, 31, n, k)
    x = synth.normal_f32(32, m * k).reshape(m, k)
    base = _gemm(backend, fmt, a, x, m, n, k)
    exps = np.array([-100, -30, -14, -1, 0, 1, 5, 14, 15, 16, 17, 30, 60, 100, -60, 3, 2, -2, -3, 7])
    scaled = np.ldexp(x, exps[:, None]).astype(np.float32)
    got = _gemm(backend, fmt, a, scaled, m, n, k)
    assert np.array_equal(got, np.ldexp(base, exps[:, None]).astype(np.float32))


@pytest.mark.parametrize("fmt", [Q1, TQ2])
def test_gemm_outlier_and_zero_rows(backend, fmt):
    m, n, k = 18, 32, 1024
    a = synth.make_blocks(fmt, 41, n, k)
    x = synth.normal_f32(42, m * k).reshape(m, k).copy()
    x[3] = 0.0
    x[5, 100] = 5000.0     # small elements of this row lose relative precision, within the bound
    x[7] = 1e-30
    got = _gemm(backend, fmt, a, x, m, n, k)
    assert np.all(got[3] == 0.0)
    _check_against_truth(got, dense_f64(fmt, a, n, k), x)
    assert parity_violations(got, oracle.gemm(fmt, a, x, m, n, k), GEMM_REL_TOL) == 0


@pytest.mark.parametrize("fmt", [Q1, TQ2])
def test_gemm_non_finite_rows_give_nan_rows_only(backend, fmt):
    m, n, k = 20, 32, 256
    a = synth.make_blocks(fmt, 51, n, k)
    x = synth.normal_f32(52, m * k).reshape(m, k).copy()
    clean = _gemm(backend, fmt, a, x, m, n, k)
    x[2, 7] = np.nan
    x[17, 255] = np.inf
    x[18, 0] = -np.inf
    got = _gemm(backend, fmt, a, x, m, n, k)
    for r in (2, 17, 18):
        assert np.all(np.isnan(got[r]))
    keep = [r for r in range(m) if r not in (2, 17, 18)]
    assert np.array_equal(got[keep], clean[keep])


def test_gemm_special_codes_and_scales(backend):
    # every code byte (incl. the reserved 0b11 lanes) with ordinary, large and negative scales
    qs = np.arange(256, dtype=np.uint8).reshape(8, 32)
    scales = [1.0, 0.007, 65504.0, -0.375, 0.0, 3.1e-4, 0.1, 7.0]
    m = 16
    x = synth.normal_f32(61, m * 512).reshape(m, 512)
    a = np.concatenate([tq2_block(s, qs[i]) for i, s in enumerate(scales)])
    got = _gemm(backend, TQ2, a, x, m, 2, 512)
    _check_against_truth(got, dense_f64(TQ2, a, 2, 512), x)
    x = x[:, :256]
    a = np.concatenate([q1_block(s, qs[i][:16]) for i, s in enumerate(scales)])
    got = _gemm(backend, Q1, a, np.ascontiguousarray(x), m, 4, 256)
    _check_against_truth(got, dense_f64(Q1, a, 4, 256), x)


@pytest.mark.parametrize("name,n,k", [("qkv", 5120, 2560), ("gate_up", 19456, 2560), ("down", 2560, 9728)])
def test_gemm_prefill_shapes_qwen3_4b_ternary(backend, name, n, k):
    """M = 512 tokens at the Qwen3-4B matrix shapes: a sample of token rows against the CPU restatement, all rows
    against the bound-free property that the GEMM of a row equals the GEMM of the same row placed elsewhere."""
    m = 512
    a = synth.make_blocks(TQ2, 7000 + n, n, k)
    x = synth.normal_f32(7001 + k, m * k).reshape(m, k).copy()
    x[300] = x[10]  # the same token row at two positions of different token tiles
    x[511] = x[129]
    got = _gemm(backend, TQ2, a, x, m, n, k)
    rows = [0, 10, 127, 128, 255, 256, 400, 511]
    want = oracle.simd_gemm(TQ2, a, np.ascontiguousarray(x[rows]), len(rows), n, k)
    assert parity_violations(got[rows], want, GEMM_REL_TOL) == 0
    # the fp16 rounding model: error rms about 2^-11/sqrt(3) of |w||x| rms, far inside the gate
    scale = np.sqrt(np.mean(want.astype(np.float64) ** 2))
    assert np.max(np.abs(got[rows] - want)) < 3e-3 * scale
    assert np.array_equal(got[300], got[10]) and np.array_equal(got[511], got[129])
    assert np.all(np.isfinite(got))


@pytest.mark.parametrize("m,n,k", [(32, 24576, 8192), (9, 24556, 6656), (17, 24576, 512)])
def test_gemm_few_rows_six_row_tiles_per_workgroup(backend, m, n, k):
    """Q1 matrices of 1536 row tiles and more at up to 32 token rows take six row tiles per workgroup.  K of 8192 and
    6656: a wave's K slice is two superblocks, so the weights of the next one are requested in place of the one just
    prepared (no second register set), the second with a last slice that is shorter than the others and a last
    workgroup that is not full; K of 512: seven of the eight waves have no slice at all."""
    a = synth.make_blocks(Q1, 8200 + m, n, k)
    x = synth.normal_f32(8201 + m, m * k).reshape(m, k)
    got = _gemm(backend, Q1, a, x, m, n, k)
    want = oracle.simd_gemm(Q1, a, x, m, n, k, x4=True)
    assert parity_violations(got, want, GEMM_REL_TOL) == 0
    assert np.max(np.abs(got - want)) < 3e-3 * np.sqrt(np.mean(want.astype(np.float64) ** 2))


def test_gemm_prefill_shape_q1_8b_gate_up(backend):
    m, n, k = 256, 24576, 4096
    a = synth.make_blocks(Q1, 8000, n, k)
    x = synth.normal_f32(8001, m * k).reshape(m, k)
    got = _gemm(backend, Q1, a, x, m, n, k)
    rows = [0, 31, 128, 255]
    want = oracle.simd_gemm(Q1, a, np.ascontiguousarray(x[rows]), len(rows), n, k)
    assert parity_violations(got[rows], want, GEMM_REL_TOL) == 0
    assert np.max(np.abs(got[rows] - want)) < 3e-3 * np.sqrt(np.mean(want.astype(np.float64) ** 2))


@pytest.mark.parametrize("fmt", [Q1, TQ2])
def test_gemm_prefill_shape_8b_qkv_2048_tokens(backend, fmt):
    """6144 x 4096 at 2048 tokens: the shape the planner gives three row tiles per wave, whose weight loads stay in
    flight across the block barrier.  A sample of rows against the CPU restatement, equal token rows in different
    token tiles and workgroups must give equal output rows, and the whole result is finite."""
    m, n, k = 2048, 6144, 4096
    a = synth.make_blocks(fmt, 8100 + fmt, n, k)
    x = synth.normal_f32(8101, m * k).reshape(m, k).copy()
    x[1999] = x[3]
    x[1024] = x[127]
    got = _gemm(backend, fmt, a, x, m, n, k)
    rows = [0, 3, 127, 128, 1023, 1500, 2047]
    want = oracle.simd_gemm(fmt, a, np.ascontiguousarray(x[rows]), len(rows), n, k)
    assert parity_violations(got[rows], want, GEMM_REL_TOL) == 0
    assert np.max(np.abs(got[rows] - want)) < 3e-3 * np.sqrt(np.mean(want.astype(np.float64) ** 2))
    assert np.array_equal(got[1999], got[3]) and np.array_equal(got[1024], got[127])
    assert np.all(np.isfinite(got))


def test_trait_gemm_paths(backend):
    # the trait-level call: m <= 16 takes the fp32-exact route, larger m the matrix cores
    n, k = 64, 512
    a = synth.make_blocks(Q1, 91, n, k)
    for m in (3, 40):
        x = synth.normal_f32(92 + m, m * k).reshape(m, k)
        got = backend.gemm_q1_g128(a, x, m, n, k)
        want = oracle.gemm(Q1, a, x, m, n, k)
        assert parity_violations(got, want, 1e-3 if m <= 16 else GEMM_REL_TOL) == 0
    a = synth.make_blocks(TQ2, 93, n, k)
    x = synth.normal_f32(94, 40 * k).reshape(40, k)
    exact = backend.gemm_tq2_g128(a, x, 40, n, k, exact=True)
    fast = backend.gemm_tq2_g128(a, x, 40, n, k)
    want = oracle.gemm(TQ2, a, x, 40, n, k)
    assert parity_violations(exact, want, 1e-3) == 0 and parity_violations(fast, want, GEMM_REL_TOL) == 0


def test_gemm_validation(backend):
    a = synth.make_blocks(Q1, 95, 16, 256)
    h = backend.upload_weights_raw(a, 16, 256)
    x = np.zeros((4, 256), dtype=np.float32)
    try:
        with pytest.raises(GpuError) as e:
            backend.gemm_cached(h, x, 4, 16, 384)
        assert e.value.kind == "InvalidArgument"
        with pytest.raises(GpuError) as e:
            backend.gemm_cached(h, x[:0], 0, 16, 256)
        assert e.value.kind == "InvalidArgument"
        with pytest.raises(GpuError) as e:
            backend.gemm_cached(h + 12345, x, 4, 16, 256)
        assert e.value.kind == "WeightNotFound"
    finally:
        backend.free_weights(h)


@pytest.mark.parametrize("fmt", [Q1, TQ2])
def test_gemm_subnormal_fp16_scales(backend, fmt):
    # block scales below the smallest normal fp16 number (6.1e-5) are still exact operands
    m, n, k = 16, 16, 256
    rng = np.random.default_rng(9)
    mk = (lambda s: q1_block(s, rng.integers(0, 256, 16, dtype=np.uint8))) if fmt == Q1 else \
         (lambda s: tq2_block(s, rng.integers(0, 256, 32, dtype=np.uint8)))
    a = np.concatenate([mk(float(s)) for s in rng.choice([6e-8, 3e-6, 5.9e-5, 1.2e-7], n * 2)])
    x = synth.normal_f32(10, m * k).reshape(m, k)
    got = _gemm(backend, fmt, a, x, m, n, k)
    _check_against_truth(got, dense_f64(fmt, a, n, k), x)
    assert np.count_nonzero(got) == got.size
