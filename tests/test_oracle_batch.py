"""The oracle's aids for long prompts, held to what is already pinned.  No GPU involved.

  oxb_simd_gemm_x4    four token rows share each decoded weight chunk: must equal oxb_simd_gemm bit for bit (that one is
                      held to the scalar kernels in test_oracle.py)
  oxb_forward_batch   n positions layer by layer: must equal n calls of the token-by-token forward bit for bit (logits
                      and every cache row), which is the property the reference's own prefill parity test checks
                      (crates/oxibonsai-model/tests/metal_prefill_ternary_parity_tests.rs:226-366)
  OracleModel(simd=True)   linear layers on the SIMD tier: within the reference's 1e-3 gate of the scalar forward"""
import numpy as np
import pytest

from helpers import Q1, TQ2, parity_violations
from oracle import oracle
from oxibonsai_amd import synth

TINY = dict(n_layers=2, h=256, inter=384, nq=4, nkv=2, hd=32, vocab=96, max_seq=48, eps=1e-6, rope_theta=1e6)


@pytest.mark.parametrize("fmt", [Q1, TQ2])
@pytest.mark.parametrize("m,n,k", [(1, 40, 256), (4, 33, 128), (7, 1100, 384), (37, 70, 1024)])
def test_gemm_x4_is_the_simd_gemm_bit_for_bit(fmt, m, n, k):
    a = synth.make_blocks(fmt, 11 + m, n, k)
    x = synth.normal_f32(5 + n, m * k).reshape(m, k)
    x[0, 3] = -0.0
    if m > 2:
        x[2, 7] = np.inf                                         # infinities and NaNs must come out the same way too
    want = oracle.simd_gemm(fmt, a, x, m, n, k)
    got = oracle.simd_gemm(fmt, a, x, m, n, k, x4=True)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    one = oracle.simd_gemv(fmt, a, x[m - 1], n, k)
    assert np.array_equal(got[m - 1].view(np.uint32), one.view(np.uint32))


def test_gemm_x4_on_every_tier():
    top = oracle.simd_set_tier(2) if oracle.simd_set_tier(2) >= 0 else oracle.lib().oxb_simd_tier()
    a = synth.make_blocks(Q1, 3, 48, 256)
    x = synth.normal_f32(4, 9 * 256).reshape(9, 256)
    try:
        for tier in range(top + 1):
            assert oracle.simd_set_tier(tier) == tier
            assert np.array_equal(oracle.simd_gemm(Q1, a, x, 9, 48, 256, x4=True), oracle.simd_gemm(Q1, a, x, 9, 48, 256))
    finally:
        oracle.simd_set_tier(top)


@pytest.mark.parametrize("fmt", [Q1, TQ2])
@pytest.mark.parametrize("simd", [False, True])
@pytest.mark.parametrize("kv_mode", [oracle.KV_F32, oracle.KV_F16, oracle.KV_I8, oracle.KV_FP8_E4M3])
def test_forward_batch_is_the_token_by_token_forward(fmt, simd, kv_mode):
    cfg = dict(TINY, fmt=fmt)
    w = synth.make_model(cfg, 21 + fmt)
    rows = synth.embedding_rows(0x51, range(23), cfg["h"]) * 50.0
    seq = oracle.OracleModel(cfg, w, kv_mode=kv_mode, simd=simd)
    bat = oracle.OracleModel(cfg, w, kv_mode=kv_mode, simd=simd)
    for pos in range(23):
        want = seq.forward(rows[pos], pos)
        if pos == 8:
            got = bat.forward_batch(rows[:9], 0)                 # a first run of nine positions ...
            assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
        if pos == 21:
            got = bat.forward_batch(rows[9:22], 9)               # ... a second one behind it ...
            assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    got = bat.forward(rows[22], 22)                              # ... and a decode step on the cache they left
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    for a, b in zip(seq.cache(), bat.cache()):
        assert (a is None and b is None) or np.array_equal(a, b)


def test_forward_batch_window_and_errors():
    cfg = dict(TINY, fmt=Q1)
    w = synth.make_model(cfg, 5)
    rows = synth.embedding_rows(0x52, range(20), cfg["h"]) * 50.0
    seq = oracle.OracleModel(cfg, w, kv_f16=True, window=6, sinks=2)
    bat = oracle.OracleModel(cfg, w, kv_f16=True, window=6, sinks=2)
    for pos in range(20):
        want = seq.forward(rows[pos], pos)
    assert np.array_equal(bat.forward_batch(rows, 0), want)
    with pytest.raises(oracle.OracleError):
        bat.forward_batch(rows, cfg["max_seq"] - 3)              # runs past the cache
    bat.freeze()
    with pytest.raises(oracle.OracleError):
        bat.forward_batch(rows[:2], 20)                          # a frozen cache takes no rows


@pytest.mark.parametrize("fmt", [Q1, TQ2])
def test_simd_forward_within_the_gate_of_the_scalar_forward(fmt):
    cfg = dict(TINY, fmt=fmt)
    w = synth.make_model(cfg, 31 + fmt)
    rows = synth.embedding_rows(0x53, range(12), cfg["h"]) * 50.0
    a, b = oracle.OracleModel(cfg, w, kv_f16=True), oracle.OracleModel(cfg, w, kv_f16=True, simd=True)
    for pos in range(12):
        want, got = a.forward(rows[pos], pos), b.forward(rows[pos], pos)
        assert parity_violations(got, want, 1e-3) == 0, pos
