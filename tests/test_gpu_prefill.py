"""GPU parity of the batched prefill pipeline (prefill GEMMs on the matrix cores, causal attention, KV store)
against the CPU oracle's token-by-token forward, through the C ABI.

The oracle is run with K/V rounded through f16 like the GPU cache.  The prefill projections round their
activations to fp16, so logits are held to 1e-2 under the reference's gate form
(abs < tol or |a-b| / max(|a|, |b|, 1e-3) < tol, metal_prefill_ternary_parity_tests.rs:294-308, which the
reference applies to its own batched-prefill-vs-sequential comparison at :254-311); greedy tokens must agree
wherever the oracle's top-2 margin exceeds that tolerance.  Decode steps that follow a prefill read the
cache the prefill wrote, which checks the stored keys and values."""
import numpy as np
import pytest

from helpers import Q1, TQ2, parity_violations
from oracle import oracle
from oxibonsai_amd import GpuError, synth
from oxibonsai_amd.model import HipModel

pytestmark = pytest.mark.gpu
PREFILL_TOL = 1e-2

TINY = dict(n_layers=2, h=128, inter=256, nq=4, nkv=2, hd=32, vocab=32, max_seq=64, eps=1e-6, rope_theta=1e6)
SMALL = dict(n_layers=3, h=512, inter=1536, nq=8, nkv=2, hd=64, vocab=1000, max_seq=400, eps=1e-6, rope_theta=1e6)
MID = dict(n_layers=2, h=512, inter=1024, nq=8, nkv=4, hd=128, vocab=512, max_seq=700, eps=1e-6, rope_theta=1e6)
WIDE = dict(n_layers=1, h=256, inter=512, nq=2, nkv=2, hd=256, vocab=64, max_seq=96, eps=1e-6, rope_theta=1e4)
# groups of four and eight q heads per kv head: the attention workgroup shares K and V between its waves
G4_HD32 = dict(n_layers=2, h=128, inter=256, nq=4, nkv=1, hd=32, vocab=64, max_seq=200, eps=1e-6, rope_theta=1e4)
G4_HD256 = dict(n_layers=1, h=1024, inter=512, nq=4, nkv=1, hd=256, vocab=64, max_seq=96, eps=1e-6, rope_theta=1e6)
G8_HD128 = dict(n_layers=1, h=1024, inter=512, nq=8, nkv=1, hd=128, vocab=64, max_seq=160, eps=1e-6, rope_theta=1e6)
# an FFN wide enough (392 gate tiles x 4 token tiles of 128) for the gate || up GEMM to take three row tiles per wave, gate
# and up tiles in different waves; 392 = 65 x 6 + 2 and 500 = 3 x 128 + 116: the last workgroups are partly empty
LONG_FFN = dict(n_layers=1, h=256, inter=6272, nq=4, nkv=2, hd=64, vocab=64, max_seq=520, eps=1e-6, rope_theta=1e6)


def _rows(seed, n, h):
    return synth.embedding_rows(seed, [(7 * i + 3) % 211 for i in range(n)], h) * 50.0   # O(1) activations


def _oracle_logits(cpu, rows, pos0=0):
    out = None
    for i, r in enumerate(rows):
        last = i == len(rows) - 1
        out = cpu.forward(r, pos0 + i, want_logits=last)
    return out


def _check(got, want, tok):
    assert parity_violations(got, want, PREFILL_TOL) == 0, f"max abs {np.max(np.abs(got - want)):.3e}"
    top2 = np.sort(want)[-2:]
    if top2[1] - top2[0] > 2 * PREFILL_TOL * max(1.0, abs(top2[1])):
        assert tok == oracle.argmax_first(want)
    assert tok == int(np.argmax(got))


@pytest.mark.parametrize("fmt", [TQ2, Q1])
@pytest.mark.parametrize("cfg,n", [(TINY, 8), (TINY, 17), (TINY, 33), (SMALL, 130), (MID, 70), (WIDE, 40),
                                   (G4_HD32, 97), (G4_HD32, 32), (G4_HD256, 50), (G8_HD128, 100), (SMALL, 1), (SMALL, 65),
                                   (LONG_FFN, 500)])
def test_prefill_matches_sequential_oracle(backend, fmt, cfg, n):
    cfg = dict(cfg, fmt=fmt)
    w = synth.make_model(cfg, 100 + n)
    cpu = oracle.OracleModel(cfg, w, kv_f16=True)
    gpu = HipModel(backend, cfg, w, batch=1)
    try:
        rows = _rows(5, n, cfg["h"])
        got, tok = gpu.prefill(rows)
        _check(got, _oracle_logits(cpu, rows), tok)
        # decode continues on the cache the prefill wrote
        for step in range(3):
            r = _rows(6 + step, 1, cfg["h"])[0]
            want = cpu.forward(r, n + step)
            g, t = gpu.forward(r, n + step)
            _check(g[0], want, int(t[0]))
    finally:
        gpu.close()


def test_chunked_prefill_equals_one_prefill(backend):
    # the reference's chunked 4 + 4 = 8 test (metal_prefill_ternary_parity_tests.rs:427-473), at tile-crossing sizes
    cfg = dict(SMALL, fmt=TQ2)
    w = synth.make_model(cfg, 77)
    rows = _rows(8, 150, cfg["h"])
    a = HipModel(backend, cfg, w)
    b = HipModel(backend, cfg, w)
    try:
        whole, tok_w = a.prefill(rows)
        b.prefill(rows[:49], want_logits=False)
        b.prefill(rows[49:128], pos_start=49, want_logits=False)
        parts, tok_p = b.prefill(rows[128:], pos_start=128)
        # same arithmetic per token row; only the attention's key-block boundaries move with the chunking
        assert parity_violations(parts, whole, 1e-3) == 0
        cpu = oracle.OracleModel(cfg, w, kv_f16=True)
        _check(parts, _oracle_logits(cpu, rows), tok_p)
    finally:
        a.close()
        b.close()


def test_prefill_then_long_greedy_decode_tracks_oracle(backend):
    cfg = dict(SMALL, fmt=Q1)
    w = synth.make_model(cfg, 55)
    cpu = oracle.OracleModel(cfg, w, kv_f16=True)
    gpu = HipModel(backend, cfg, w)
    try:
        n = 40
        rows = _rows(9, n, cfg["h"])
        got, tok = gpu.prefill(rows)
        want = _oracle_logits(cpu, rows)
        _check(got, want, tok)
        agree = decided = 0
        for step in range(64):      # free-running: the GPU's token feeds both sides
            r = synth.embedding_rows(9, [tok], cfg["h"])[0] * 50.0
            want = cpu.forward(r, n + step)
            g, t = gpu.forward(r, n + step)
            assert parity_violations(g[0], want, PREFILL_TOL) == 0
            top2 = np.sort(want)[-2:]
            if top2[1] - top2[0] > 2 * PREFILL_TOL * max(1.0, abs(top2[1])):
                decided += 1
                agree += int(t[0] == oracle.argmax_first(want))
            tok = int(t[0])
        assert agree == decided and decided > 32
    finally:
        gpu.close()


def test_prefill_into_one_sequence_of_a_batch(backend):
    cfg = dict(TINY, fmt=TQ2)
    w = synth.make_model(cfg, 3)
    gpu = HipModel(backend, cfg, w, batch=2)
    solo = HipModel(backend, cfg, w, batch=1)
    try:
        rows0, rows1 = _rows(1, 20, cfg["h"]), _rows(2, 20, cfg["h"])
        l0, _ = gpu.prefill(rows0, seq=0)
        l1, _ = gpu.prefill(rows1, seq=1)
        s0, _ = solo.prefill(rows0)
        assert np.array_equal(l0, s0)
        s1, _ = solo.prefill(rows1)
        assert np.array_equal(l1, s1)
        # one batched decode step over both caches
        step = np.stack([_rows(3, 1, cfg["h"])[0], _rows(4, 1, cfg["h"])[0]])
        got, _ = gpu.forward(step, [20, 20])
        solo.prefill(rows0)
        w0, _ = solo.forward(step[0], 20)
        assert parity_violations(got[0], w0[0], 1e-3) == 0
    finally:
        gpu.close()
        solo.close()


def test_prefill_validation(backend):
    cfg = dict(TINY, fmt=Q1)
    gpu = HipModel(backend, cfg, synth.make_model(cfg, 4))
    try:
        rows = _rows(1, 10, cfg["h"])
        with pytest.raises(GpuError) as e:
            gpu.prefill(rows, pos_start=60)          # 60 + 10 > max_seq 64
        assert e.value.kind == "InvalidArgument"
        with pytest.raises(GpuError) as e:
            gpu.prefill(rows, seq=1)
        assert e.value.kind == "InvalidArgument"
        with pytest.raises(GpuError) as e:
            gpu.prefill(rows[:0])
        assert e.value.kind == "InvalidArgument"
    finally:
        gpu.close()
