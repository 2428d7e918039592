"""Pins the CPU oracle: the reference's own known-answer tests, the IEEE definition of f16,
and an independent float64 decode.  No GPU involved."""
import numpy as np
import pytest

from helpers import Q1, TQ2, block, cross_tier_q1, dense_f64, metal_tq2, q1_block, simd_parity_tq2, tq2_block
from oracle import oracle
from oxibonsai_amd import synth


# ---- f16 <-> f32 against numpy for every bit pattern ---------------------------------------------
def test_f16_to_f32_all_patterns():
    h = np.arange(65536, dtype=np.uint16)
    want = h.view(np.float16).astype(np.float32)
    got = np.array([oracle.f16_to_f32(int(v)) for v in h], dtype=np.float32)
    nan = np.isnan(want)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))
    assert np.all(np.isnan(got[nan]))


def test_f32_to_f16_round_to_nearest_even():
    rng = np.random.default_rng(1)
    vals = np.concatenate([
        rng.standard_normal(20000).astype(np.float32) * np.float32(10.0) ** rng.integers(-8, 5, 20000).astype(np.float32),
        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e-8, 5.9604645e-8, 2.9802322e-8, 2.98023224e-8 * 1.0000001,
                  6.1035156e-5, 6.0975552e-5, np.inf, -np.inf], dtype=np.float32),
        # exact ties between neighbouring f16 values
        (np.arange(1024, 2048, dtype=np.float32) + 0.5) * np.float32(2.0 ** -10),
    ])
    with np.errstate(over="ignore"):
        want = vals.astype(np.float16).view(np.uint16)
    got = np.array([oracle.f32_to_f16(float(v)) for v in vals], dtype=np.uint16)
    assert np.array_equal(got, want)


# ---- dequant KATs: core/src/tensor.rs:161-190, kernels/src/dequant.rs:51-99 -----------------------
def test_dequant_q1_patterns():
    assert np.all(oracle.dequant(Q1, q1_block(2.0, 0xFF)) == 2.0)
    assert np.all(oracle.dequant(Q1, q1_block(2.0, 0x00)) == -2.0)
    w = oracle.dequant(Q1, q1_block(1.5, 0xAA))  # 10101010: bit0 = 0 -> -d, bit1 = 1 -> +d
    assert np.all(w[0::2] == -1.5) and np.all(w[1::2] == 1.5)
    w = oracle.dequant(Q1, q1_block(1.5, 0x55))
    assert np.all(w[0::2] == 1.5) and np.all(w[1::2] == -1.5)


# kernels/src/dequant_ternary.rs:127-218, core/src/quant_ternary.rs:518-546
def test_dequant_tq2_patterns():
    assert np.all(oracle.dequant(TQ2, tq2_block(1.0, 0xAA)) == 1.0)
    assert np.all(oracle.dequant(TQ2, tq2_block(1.0, 0x00)) == -1.0)
    assert np.all(oracle.dequant(TQ2, tq2_block(1.0, 0x55)) == 0.0)
    assert np.all(oracle.dequant(TQ2, tq2_block(1.0, 0xFF)) == 0.0)  # reserved 0b11 -> 0
    # 0x9C = 0b10_01_11_00: lanes (LSB first) 00 -> -1, 11 -> 0, 01 -> 0, 10 -> +1
    w = oracle.dequant(TQ2, tq2_block(0.5, 0x9C)).reshape(32, 4)
    assert np.array_equal(w[0], np.array([-0.5, 0.0, 0.0, 0.5], dtype=np.float32))
    # 0b10_01_00_10: lanes +1, -1, 0, +1 (dequant_ternary.rs:177-218)
    w = oracle.dequant(TQ2, tq2_block(2.0, 0b10010010)).reshape(32, 4)
    assert np.array_equal(w[5], np.array([2.0, -2.0, 0.0, 2.0], dtype=np.float32))


def test_dequant_brute_force_all_bytes_all_scales():
    # every code byte x every lane
    for byte in range(256):
        w = oracle.dequant(TQ2, tq2_block(1.0, byte))[:4]
        want = [{0: -1.0, 1: 0.0, 2: 1.0, 3: 0.0}[(byte >> (2 * l)) & 3] for l in range(4)]
        assert list(w) == want
        wq = oracle.dequant(Q1, q1_block(1.0, byte))[:8]
        assert list(wq) == [1.0 if (byte >> i) & 1 else -1.0 for i in range(8)]
    # every finite f16 scale
    h = np.arange(65536, dtype=np.uint16)
    h = h[np.isfinite(h.view(np.float16))]
    blocks = np.zeros((h.size, 18), dtype=np.uint8)
    blocks[:, 0:2] = h.view(np.uint8).reshape(-1, 2)
    blocks[:, 2] = 0x01
    w = oracle.dequant(Q1, blocks.reshape(-1)).reshape(-1, 128)
    d = h.view(np.float16).astype(np.float32)
    assert np.array_equal(w[:, 0].view(np.uint32), d.view(np.uint32))
    assert np.array_equal(w[:, 1].view(np.uint32), (-d).view(np.uint32))


# ---- GEMV KATs: kernels/src/gemv.rs:101-170, gemv_ternary.rs:212-324 -------------------------------
def test_gemv_q1_reference_kats():
    x = np.arange(128, dtype=np.float32)
    assert oracle.gemv(Q1, q1_block(1.0, 0xFF), x, 1, 128)[0] == 8128.0
    assert oracle.gemv(Q1, q1_block(2.0, 0x00), np.ones(128, np.float32), 1, 128)[0] == -256.0
    two = np.concatenate([q1_block(1.0, 0xFF), q1_block(1.0, 0x00)])
    assert list(oracle.gemv(Q1, two, np.ones(128, np.float32), 2, 128)) == [128.0, -128.0]


def test_gemv_tq2_reference_kats():
    ones = np.ones(128, np.float32)
    two = np.concatenate([tq2_block(1.0, 0xAA)] * 2)
    assert list(oracle.gemv(TQ2, two, ones, 2, 128)) == [128.0, 128.0]
    two = np.concatenate([tq2_block(1.0, 0x00)] * 2)
    assert list(oracle.gemv(TQ2, two, ones, 2, 128)) == [-128.0, -128.0]
    assert oracle.gemv(TQ2, tq2_block(1.0, 0x46), ones, 1, 128)[0] == 0.0  # +1, 0, -1, 0 canary
    eight = np.concatenate([tq2_block(1.0, 0xAA)] * 8)
    assert list(oracle.gemv(TQ2, eight, np.ones(256, np.float32), 4, 256)) == [256.0] * 4


@pytest.mark.parametrize("fmt", [Q1, TQ2])
def test_gemv_validation_errors(fmt):
    b = block(fmt, 1.0, 0xAA)
    with pytest.raises(oracle.OracleError) as e:
        oracle.gemv(fmt, b, np.ones(100, np.float32), 1, 100)
    assert e.value.code == oracle.NOT_BLOCK_ALIGNED
    with pytest.raises(oracle.OracleError) as e:
        oracle.gemv(fmt, b, np.ones(64, np.float32), 1, 128)  # input too short
    assert e.value.code == oracle.DIMENSION_MISMATCH
    with pytest.raises(oracle.OracleError) as e:
        oracle.gemv(fmt, b, np.ones(128, np.float32), 2, 128, y_len=1)  # output too short
    assert e.value.code == oracle.BUFFER_TOO_SMALL
    with pytest.raises(oracle.OracleError) as e:
        oracle.gemv(fmt, b, np.ones(128, np.float32), 2, 128)  # one block for two rows
    # gemv.rs:52-58 reports BufferTooSmall, gemv_ternary.rs:76-81 DimensionMismatch
    assert e.value.code == (oracle.BUFFER_TOO_SMALL if fmt == Q1 else oracle.DIMENSION_MISMATCH)


# ---- against an independent float64 decode, on the reference's own generators ---------------------
def test_gemv_q1_cross_tier_generator():
    n, k = 128, 1024
    blocks = cross_tier_q1(n, k)
    x = np.array([(i % 17) * 0.25 - 2.0 for i in range(k)], dtype=np.float32)
    want = dense_f64(Q1, blocks, n, k) @ x.astype(np.float64)
    got = oracle.gemv(Q1, blocks, x, n, k)
    assert np.max(np.abs(got - want)) < 1e-3 * np.max(np.abs(want))
    simd = oracle.simd_gemv(Q1, blocks, x, n, k)
    assert np.max(np.abs(simd - got)) < 1.0  # cross_tier.rs:60-93 tolerance
    assert np.max(np.abs(simd - want)) < 1e-3 * np.max(np.abs(want))


def test_gemv_tq2_simd_parity_generator():
    blocks, x = simd_parity_tq2(64, 128)
    want = dense_f64(TQ2, blocks, 64, 128) @ x.astype(np.float64)
    got = oracle.gemv(TQ2, blocks, x, 64, 128)
    simd = oracle.simd_gemv(TQ2, blocks, x, 64, 128)
    assert np.mean((got - want) ** 2) < 1e-6          # simd_avx2.rs:1163-1180: MSE < 1e-6
    assert np.mean((simd - got) ** 2) < 1e-6


def test_gemv_tq2_metal_generator():
    n, k = 64, 512
    blocks = metal_tq2(n, k)
    x = np.array([((i * 7 + 3) % 19) * 0.1 - 0.9 for i in range(k)], dtype=np.float32)
    want = dense_f64(TQ2, blocks, n, k) @ x.astype(np.float64)
    assert np.max(np.abs(oracle.gemv(TQ2, blocks, x, n, k) - want)) < 1e-3  # metal_graph/tests.rs:468-535


@pytest.mark.parametrize("fmt", [Q1, TQ2])
def test_gemv_seeded_vs_float64_and_simd(fmt):
    n, k = 96, 2048
    blocks = synth.make_blocks(fmt, 42 + fmt, n, k)
    x = synth.normal_f32(7, k)
    want = dense_f64(fmt, blocks, n, k) @ x.astype(np.float64)
    got = oracle.gemv(fmt, blocks, x, n, k)
    simd = oracle.simd_gemv(fmt, blocks, x, n, k)
    scale = np.max(np.abs(want))
    assert np.max(np.abs(got - want)) < 2e-6 * scale
    assert np.max(np.abs(simd - want)) < 2e-6 * scale
    # dequant agrees bit for bit with the independent decode
    assert np.array_equal(oracle.dequant(fmt, blocks).astype(np.float64).reshape(n, k), dense_f64(fmt, blocks, n, k))


# ---- invariants: tests/proptest_kernels.rs:57-112, edge_cases.rs:109-230 ---------------------------
@pytest.mark.parametrize("fmt", [Q1, TQ2])
def test_gemv_invariants(fmt):
    n, k = 24, 512
    blocks = synth.make_blocks(fmt, 3, n, k)
    x1, x2 = synth.normal_f32(1, k), synth.normal_f32(2, k)
    y1, y2 = oracle.gemv(fmt, blocks, x1, n, k), oracle.gemv(fmt, blocks, x2, n, k)
    y12 = oracle.gemv(fmt, blocks, x1 + x2, n, k)
    assert np.max(np.abs(y12 - (y1 + y2))) < 1e-4                     # linearity
    assert np.all(oracle.gemv(fmt, blocks, np.zeros(k, np.float32), n, k) == 0.0)
    xs = np.stack([x1, x2, x1 - x2])
    Y = oracle.gemm(fmt, blocks, xs, 3, n, k)
    assert np.array_equal(Y[0], y1) and np.array_equal(Y[1], y2)       # gemm row = gemv
    zero = blocks.copy().reshape(-1, 18 if fmt == Q1 else 34)
    if fmt == Q1:
        zero[:, 0:2] = 0
    else:
        zero[:, 32:34] = 0
    assert np.all(oracle.gemv(fmt, zero.reshape(-1), x1, n, k) == 0.0)  # zero scale -> 0
    assert np.array_equal(oracle.simd_gemm(fmt, blocks, xs, 3, n, k), np.stack(
        [oracle.simd_gemv(fmt, blocks, xs[i], n, k) for i in range(3)]))


def test_gemv_large_k_edge_case():
    # k = 12 800 as in tests/edge_cases.rs
    k = 12800
    blocks = np.concatenate([q1_block(0.5, 0xFF)] * (k // 128))
    assert oracle.gemv(Q1, blocks, np.ones(k, np.float32), 1, k)[0] == 0.5 * k


# ---- every SIMD tier the host offers, forced in turn ---------------------------------------------
@pytest.mark.parametrize("tier", [0, 1, 2])
def test_each_simd_tier_against_the_scalar_oracle(tier):
    """The CPU baseline picks its tier by CPUID (dispatch.rs:143-175), so on an AVX-512 host the AVX2 kernels would
    never run: force each tier and hold it to the scalar oracle with the reference's own SIMD-vs-scalar gates
    (MSE < 1e-6 on the generator of simd_avx2.rs:1147-1180; < 1.0 absolute on cross_tier.rs:18-93) and to the
    float64 product."""
    best = oracle.lib().oxb_simd_tier()
    top = oracle.simd_set_tier(2)
    top = top if top >= 0 else (1 if oracle.simd_set_tier(1) >= 0 else 0)
    try:
        if tier > top:
            pytest.skip(f"host CPU offers no tier above {oracle.SIMD_TIERS[top]}")
        assert oracle.simd_set_tier(tier) == tier and oracle.lib().oxb_simd_tier() == tier
        blocks, x = simd_parity_tq2(64, 128)
        assert np.mean((oracle.simd_gemv(TQ2, blocks, x, 64, 128) - oracle.gemv(TQ2, blocks, x, 64, 128)) ** 2) < 1e-6
        n, k = 128, 1024
        blocks = cross_tier_q1(n, k)
        x = np.array([(i % 17) * 0.25 - 2.0 for i in range(k)], dtype=np.float32)
        assert np.max(np.abs(oracle.simd_gemv(Q1, blocks, x, n, k) - oracle.gemv(Q1, blocks, x, n, k))) < 1.0
        for fmt in (Q1, TQ2):
            # odd block counts (the AVX2 Q1 kernel takes two blocks per iteration and a tail), row counts on both
            # sides of the direct / threaded switch, and the batched entry point
            for n, k in ((5, 128), (33, 384), (300, 640), (70, 2048)):
                blocks = synth.make_blocks(fmt, 900 + n, n, k)
                x = synth.normal_f32(901 + k, k)
                want = dense_f64(fmt, blocks, n, k) @ x.astype(np.float64)
                got = oracle.simd_gemv(fmt, blocks, x, n, k)
                scale = np.max(np.abs(want))
                assert np.max(np.abs(got - want)) < 2e-6 * scale, (tier, fmt, n, k)
                assert np.max(np.abs(got - oracle.gemv(fmt, blocks, x, n, k))) < 4e-6 * scale
            m, n, k = 5, 40, 256
            blocks = synth.make_blocks(fmt, 77, n, k)
            xs = synth.normal_f32(78, m * k).reshape(m, k)
            got = oracle.simd_gemm(fmt, blocks, xs, m, n, k)
            want = xs.astype(np.float64) @ dense_f64(fmt, blocks, n, k).T
            assert np.max(np.abs(got - want)) < 2e-6 * np.max(np.abs(want))
        assert oracle.simd_set_tier(3) == -1 and oracle.lib().oxb_simd_tier() == tier      # an unknown tier changes nothing
    finally:
        oracle.simd_set_tier(best)
