"""The benchmark configurations at their real sizes, through the C ABI, against the CPU oracle.

  configs[1]  Q1_0_g128 GEMV at the Qwen3-8B shapes, batch 8 (batch 1 is in test_gpu_gemv.py)
  configs[3]  random-init ternary Qwen3-1.7B, KV context 4096: a seeded prompt, then 128 free-running greedy steps
  configs[4]  random-init Qwen3-8B-shape Q1 model: the 2048-token prefill followed by greedy steps, decode at batch 8
              and 32, one step at a context of ~32 000, and batch 8 with a KV context of 32 768 whose last sequence is
              filled to ~32 000 positions (cache offsets beyond 2^32 elements)

Greedy tokens follow the reference's parity test (crates/oxibonsai-model/tests/metal_prefill_ternary_parity_tests.rs:
317-366): the token must equal the oracle's wherever the oracle's own top-2 margin exceeds the logit tolerance; the
margin of every step is reported.  Tolerances at these sizes are those of test_gpu_model.test_full_size_shapes_match_oracle."""
import sys
import time

import numpy as np
import pytest

from helpers import Q1, TQ2
from oracle import oracle
from oxibonsai_amd import synth
from oxibonsai_amd.model import HipModel

pytestmark = pytest.mark.gpu

C3 = dict(fmt=TQ2, n_layers=28, h=2048, inter=6144, nq=16, nkv=8, hd=128, vocab=151936, max_seq=4096, eps=1e-6, rope_theta=1e6)
C4 = dict(fmt=Q1, n_layers=36, h=4096, inter=12288, nq=32, nkv=8, hd=128, vocab=151936, max_seq=32768, eps=1e-6, rope_theta=1e6)


def _row(seed, tok, h):
    return synth.embedding_rows(seed, [int(tok)], h)[0] * 50.0       # O(1) activations


@pytest.mark.parametrize("shape", [(24576, 4096), (6144, 4096), (4096, 12288)])
def test_config1_q1_gemv_batch8(backend, shape):
    n, k = shape
    a = synth.make_q1_blocks(0xB0A5A10100 + n, n * (k // 128), 0.01, 0.1)
    xs = synth.normal_f32(0xB0A5A10180 + k, 8 * k).reshape(8, k)
    h = backend.upload_weights_raw(a, n, k)
    try:
        got = backend.gemv_cached_batch(h, xs, n, k)
    finally:
        backend.free_weights(h)
    want = oracle.gemm(Q1, a, xs, 8, n, k)
    for b in range(8):
        scale = float(np.max(np.abs(want[b])))
        assert np.max(np.abs(got[b] - want[b])) < 1e-5 * scale, b          # the north star asks for 1e-3 relative


def test_config3_ternary_1p7b_greedy_128_steps(backend):
    cfg = C3
    w = synth.make_model(cfg, 0xB0A5A103)
    cpu = oracle.OracleModel(cfg, w, kv_f16=True)
    gpu = HipModel(backend, cfg, w, batch=1)
    try:
        prompt = [int(t) for t in synth.token_ids(0xB0A5A1C3, 8, cfg["vocab"])]
        # the prompt goes in token by token on both sides (fp32-exact products), so that the comparison of the
        # generated tokens is not blurred by the fp16 activations of the batched prefill
        for pos, t in enumerate(prompt):
            r = _row(0xE3B, t, cfg["h"])
            last = pos == len(prompt) - 1
            want = cpu.forward(r, pos, want_logits=last)
            got, tok = gpu.forward(r, pos, want_logits=last)
        margins, undecided, worst = [], 0, 0.0
        for step in range(128):
            tol = 5e-4 * float(np.max(np.abs(want)))
            err = float(np.max(np.abs(got[0] - want)))
            worst = max(worst, err / tol)
            assert err < tol, (step, err, tol)
            top2 = np.sort(want)[-2:]
            margins.append(float(top2[1] - top2[0]))
            if margins[-1] > 2 * tol:
                assert int(tok[0]) == oracle.argmax_first(want), (step, margins[-1])
            else:
                undecided += 1
            assert int(tok[0]) == int(np.argmax(got[0]))
            if step == 127:
                break
            pos = len(prompt) + step
            r = _row(0xE3B, tok[0], cfg["h"])                      # free-running: the GPU's token feeds both sides
            want = cpu.forward(r, pos)
            got, tok = gpu.forward(r, pos)
        print(f"config 3: 128 greedy steps, top-2 margin min {min(margins):.4f} median {np.median(margins):.4f}, "
              f"{undecided} steps inside the tolerance of a tie, worst logit error {worst:.2f} of the tolerance")
        assert undecided <= 12                                      # the comparison must decide nearly every step
        assert gpu.uses_graph()
    finally:
        gpu.close()


@pytest.fixture(scope="module")
def c4_model():
    w = synth.make_model(C4, 0xB0A5A104)
    yield w


@pytest.fixture(scope="module")
def c4_table():
    """Embedding rows of 5000 token ids, O(1) activations."""
    return synth.embedding_rows(0xC4E, range(5000), C4["h"]) * 50.0


N_DISTINCT = 4


@pytest.fixture(scope="module")
def c4_oracle_steps(c4_model):
    """Three decode steps from position 0 of four different sequences, on the oracle: logits [seq][step]."""
    cfg = dict(C4, max_seq=64)
    out = []
    for s in range(N_DISTINCT):
        cpu = oracle.OracleModel(cfg, c4_model, kv_f16=True)
        out.append([cpu.forward(_row(0xC40 + s, 1000 * s + step, cfg["h"]), step) for step in range(3)])
    return out


@pytest.mark.parametrize("B", [8, 12, 32])
def test_config4_q1_8b_batched_decode(backend, c4_model, c4_oracle_steps, B):
    """Batch 8 and 32 at the 8B shape (and 12: one token tile on the matrix-core route): sequence b carries the inputs
    of sequence b % 4, each of the four is held to its own oracle, and sequences with equal inputs must agree with each
    other.  Batches of nine and more run their projections as fp16 matrix-core GEMMs - gate || up and the LM head with
    six row tiles per workgroup, which only shapes of this size select: prefill tolerance.  Batch 8 takes the fp32-exact
    packed GEMV and is held to the same bar."""
    cfg = dict(C4, max_seq=64)
    gpu = HipModel(backend, cfg, c4_model, batch=B)
    try:
        for step in range(3):
            rows = [_row(0xC40 + s, 1000 * s + step, cfg["h"]) for s in range(N_DISTINCT)]
            got, toks = gpu.forward(np.stack([rows[b % N_DISTINCT] for b in range(B)]), np.full(B, step, dtype=np.uint32))
            for s in range(N_DISTINCT):
                want = c4_oracle_steps[s][step]
                # eight sequences take the fp32-exact route: the batch-1 decode bar; more run on fp16 activations
                tol = (5e-4 if B <= 8 else 5e-3) * float(np.max(np.abs(want)))
                err = float(np.max(np.abs(got[s] - want)))
                assert err < tol, (B, step, s, err, tol)
                top2 = np.sort(want)[-2:]
                if top2[1] - top2[0] > 2 * tol:
                    assert int(toks[s]) == oracle.argmax_first(want), (B, step, s)
                for b in range(s, B, N_DISTINCT):
                    assert np.allclose(got[b], got[s], rtol=0, atol=1e-4), (B, step, b)
                    assert int(toks[b]) == int(np.argmax(got[b]))
        assert gpu.uses_graph()
    finally:
        gpu.close()


def test_config4_q1_8b_decode_at_context_32000(backend, c4_model, c4_table):
    """KV context 32 768 at the 8B shape: a prompt of 31 990 positions goes in through the batched prefill, then decode
    steps follow.  The oracle cannot walk 32 000 positions of a 36-layer model in test time, so it reads the device's
    own cache rows (every layer and kv head) and is held frozen over them: its forward of the new position then shows
    whether attention over the whole context, the projections and the LM head agree."""
    cfg = C4
    n = 31990
    gpu = HipModel(backend, cfg, c4_model, batch=1)
    try:
        ids = synth.token_ids(0xB0A5A1C4, n, 5000)
        table = c4_table
        for p0 in range(0, n, 4096):                                  # chunked prefill, 4096 positions per call
            gpu.prefill(table[ids[p0:p0 + 4096]], pos_start=p0, want_logits=False)
        steps = []
        for step in range(2):
            r = _row(0xC4F, step, cfg["h"])
            got, tok = gpu.forward(r, n + step)
            steps.append((r, got[0].copy(), int(tok[0])))
        cpu = oracle.OracleModel(cfg, c4_model, kv_f16=True)
        for L in range(cfg["n_layers"]):
            for hh in range(cfg["nkv"]):
                k, v, _, _ = gpu.read_kv(L, hh, 0, n + 2)
                cpu.load_rows(L, hh, 0, k.astype(np.float32), v.astype(np.float32))
        cpu.freeze()
        for step, (r, got, tok) in enumerate(steps):
            want = cpu.forward(r, n + step)
            tol = 5e-4 * float(np.max(np.abs(want)))
            err = float(np.max(np.abs(got - want)))
            assert err < tol, (step, err, tol)
            top2 = np.sort(want)[-2:]
            if top2[1] - top2[0] > 2 * tol:
                assert tok == oracle.argmax_first(want), step
        assert gpu.uses_graph()
    finally:
        gpu.close()


def _say(capsys, msg):
    """A progress line past pytest's capture: the long tests below must not look hung to whoever watches the output."""
    with capsys.disabled():
        print(msg, file=sys.stderr, flush=True)


N_PROMPT = 2048
N_GREEDY = 32   # greedy steps behind the prompt (the oracle's SIMD-tier forward takes ~40 ms each)


@pytest.mark.timeout(900)
def test_config4_q1_8b_prefill_2048_then_greedy(backend, c4_model, c4_table, capsys):
    """configs[4] as quoted: 2048 random token ids through the batched prefill (try_cuda_prefill,
    gpu_backend/cuda_prefill/try_apis.rs:42 -> the LM head of encode_q1.rs:881), then greedy decode on the cache it
    wrote, at the 8B shape with a KV context of 32 768.  The oracle runs the same 2048 positions layer by layer with
    its linear layers on the CPU SIMD tier (bit-equal to its token-by-token forward, tests/test_oracle_batch.py; the
    tier is held to the scalar kernels in tests/test_oracle.py).  Every GEMM tile of the prefill is full here (16
    token tiles of 128 at the real N and K), which the 8-token prefill of test_full_size_shapes_match_oracle never
    reaches.  Tolerance: the prefill's (fp16 activations), 5e-3 of the largest logit; the rows of the first layer
    within one fp16 step plus 2^-11 of the row's scale of the oracle's, those of the last layer within 2e-2 in the root mean square
    (single elements of a head with a small norm lie up to 4e-2 of the row's scale off after 36 layers)."""
    cfg = C4
    ids = synth.token_ids(0xB0A5A1C5, N_PROMPT, 5000)
    rows = c4_table[ids]
    gpu = HipModel(backend, cfg, c4_model, batch=1)
    try:
        got, tok = gpu.prefill(rows, pos_start=0)
        _say(capsys, f"config 4: device prefill of {N_PROMPT} tokens done, oracle running")
        cpu = oracle.OracleModel(cfg, c4_model, kv_f16=True, simd=True)
        t0 = time.time()
        want = cpu.forward_batch(rows[:N_PROMPT // 2], 0, want_logits=False)
        _say(capsys, f"config 4: oracle at position {N_PROMPT // 2} after {time.time() - t0:.0f} s")
        want = cpu.forward_batch(rows[N_PROMPT // 2:], N_PROMPT // 2)
        _say(capsys, f"config 4: oracle prefill done after {time.time() - t0:.0f} s")
        tol = 5e-3 * float(np.max(np.abs(want)))
        err = float(np.max(np.abs(got - want)))
        assert err < tol, ("prefill logits", err, tol)
        top2 = np.sort(want)[-2:]
        if top2[1] - top2[0] > 2 * tol:
            assert tok == oracle.argmax_first(want)
        assert tok == int(np.argmax(got))
        # what the prefill left in the cache
        deep = []
        for L, bar in ((0, None), (cfg["n_layers"] - 1, 2e-2)):
            for hh in (0, cfg["nkv"] - 1):
                k, v, _, _ = gpu.read_kv(L, hh, 0, N_PROMPT)
                wk, wv = cpu.cache_rows(L, hh, 0, N_PROMPT)
                for a, b, name in ((k, wk, "K"), (v, wv, "V")):
                    a = a.astype(np.float32)
                    if bar is None:        # one fp16 step of the value plus the GEMM's fp16 activations (2^-11 of the row's scale)
                        step = (np.spacing(np.maximum(np.abs(a), np.abs(b)).astype(np.float16)).astype(np.float32)
                                + 2.0 ** -11 * np.max(np.abs(b), axis=1, keepdims=True))
                        assert np.all(np.abs(a - b) <= step), (L, hh, name, float(np.max(np.abs(a - b) / step)))
                    else:                  # 36 layers of fp16 activations later: the rows as a whole (root mean square)
                        rms = float(np.sqrt(np.mean((a - b) ** 2) / np.mean(b ** 2)))
                        rel = np.abs(a - b) / np.max(np.abs(b), axis=1, keepdims=True)
                        at = np.unravel_index(int(np.argmax(rel)), rel.shape)
                        deep.append((L, hh, name, round(rms, 5), round(float(rel[at]), 5), tuple(int(i) for i in at),
                                     int(np.count_nonzero(rel > 2e-2))))
                        assert rms <= bar, deep[-1]
        # greedy decode on that cache; the device's token feeds both sides
        worst, undecided = err / tol, 0
        for step in range(N_GREEDY):
            r = _row(0xC4D, tok, cfg["h"])
            want = cpu.forward(r, N_PROMPT + step)
            g, t = gpu.forward(r, N_PROMPT + step)
            tol = 5e-3 * float(np.max(np.abs(want)))
            err = float(np.max(np.abs(g[0] - want)))
            worst = max(worst, err / tol)
            assert err < tol, (step, err, tol)
            top2 = np.sort(want)[-2:]
            if top2[1] - top2[0] > 2 * tol:
                assert int(t[0]) == oracle.argmax_first(want), step
            else:
                undecided += 1
            assert int(t[0]) == int(np.argmax(g[0]))
            tok = int(t[0])
        _say(capsys, f"config 4: prefill {N_PROMPT} + {N_GREEDY} greedy steps, worst logit error {worst:.2f} of the tolerance, "
                     f"{undecided} steps inside the tolerance of a tie, oracle {time.time() - t0:.0f} s; last-layer rows "
                     f"(layer, head, K/V, rms error, worst element / row scale, its (position, dimension), elements beyond 2e-2): {deep}")
        assert gpu.uses_graph()
    finally:
        gpu.close()


@pytest.mark.parametrize("B", [8, 32])
def test_config4_q1_8b_prefill_and_decode_repeat_bit_for_bit(backend, c4_model, c4_table, B):
    """The 2048-token prefill and decode steps of eight (fp32-exact GEMVs) and 32 sequences (fp16 GEMMs) behind it, twice from a cleared cache: every logit
    and every cache row of the first and the last layer must come out bit for bit the same (the reference holds its
    fused path to the same property on a small model, cuda_full_layer/encode_ternary.rs:966-1149).  No oracle is
    involved: this is the check that an unordered sum or a read that overtakes a write would fail some of the time."""
    cfg = dict(C4, max_seq=2304)
    ids = synth.token_ids(0xB0A5A1C6, N_PROMPT, 5000)
    rows = c4_table[ids]
    gpu = HipModel(backend, cfg, c4_model, batch=B)
    try:
        runs = []
        for _ in range(2):
            gpu.reset()
            logits, tok = gpu.prefill(rows, pos_start=0, seq=B - 1)
            kv = [gpu.read_kv(L, hh, 0, N_PROMPT, seq=B - 1)[:2] for L in (0, cfg["n_layers"] - 1) for hh in (0, cfg["nkv"] - 1)]
            steps = []
            for step in range(3):                    # the last sequence continues behind its prompt, the others start at 0
                hidden = np.stack([_row(0xC4E + b, step, cfg["h"]) for b in range(B)])
                pos = np.array([step] * (B - 1) + [N_PROMPT + step], dtype=np.uint32)
                g, t = gpu.forward(hidden, pos)
                steps.append((g.copy(), t.copy()))
            runs.append((logits.copy(), int(tok), kv, steps))
        a, b = runs
        assert np.array_equal(a[0].view(np.uint32), b[0].view(np.uint32)) and a[1] == b[1]
        for (ka, va), (kb, vb) in zip(a[2], b[2]):
            assert np.array_equal(ka, kb) and np.array_equal(va, vb)
        for (ga, ta), (gb, tb) in zip(a[3], b[3]):
            assert np.array_equal(ga.view(np.uint32), gb.view(np.uint32)) and np.array_equal(ta, tb)
    finally:
        gpu.close()


@pytest.mark.timeout(600)
def test_config4_q1_8b_batch8_at_kv_context_32768(backend, c4_model, c4_oracle_steps, c4_table, capsys):
    """Batch 8 with a KV context of 32 768, as configs[4] quotes it: the last of the eight sequences is filled to
    31 990 positions, so its cache rows lie beyond 2^32 elements from the start of the allocation (the reference
    indexes its cache with u32 element counts, gpu_backend/cuda_full_layer/mod.rs:128-130: the case a 64-bit offset
    exists for).  Sequences 0-6 decode from position 0 with the inputs of c4_oracle_steps; sequence 7 is held to the
    oracle frozen over the device's own cache rows, as in the batch-1 test above.  Batches of five and more run
    their projections as fp16 matrix-core GEMMs: prefill tolerance."""
    cfg, B, n = C4, 8, 31990
    assert (B - 1) * cfg["n_layers"] * cfg["nkv"] * cfg["max_seq"] * cfg["hd"] > 2 ** 32
    gpu = HipModel(backend, cfg, c4_model, batch=B)
    try:
        ids = synth.token_ids(0xB0A5A1C6, n, 5000)
        table = c4_table
        for p0 in range(0, n, 4096):
            gpu.prefill(table[ids[p0:p0 + 4096]], pos_start=p0, seq=B - 1, want_logits=False)
        _say(capsys, "config 4, batch 8: sequence 7 filled")
        steps = []
        for step in range(2):
            deep = _row(0xC4F, 7 + step, cfg["h"])
            hidden = np.stack([_row(0xC40 + b % N_DISTINCT, 1000 * (b % N_DISTINCT) + step, cfg["h"]) for b in range(B - 1)] + [deep])
            pos = np.array([step] * (B - 1) + [n + step], dtype=np.uint32)
            got, toks = gpu.forward(hidden, pos)
            steps.append((deep, got.copy(), toks.copy()))
            for b in range(B - 1):
                want = c4_oracle_steps[b % N_DISTINCT][step]
                tol = 5e-3 * float(np.max(np.abs(want)))
                err = float(np.max(np.abs(got[b] - want)))
                assert err < tol, (step, b, err, tol)
                top2 = np.sort(want)[-2:]
                if top2[1] - top2[0] > 2 * tol:
                    assert int(toks[b]) == oracle.argmax_first(want), (step, b)
                if b >= N_DISTINCT:
                    assert np.allclose(got[b], got[b - N_DISTINCT], rtol=0, atol=1e-4), (step, b)
        # no other sequence's rows were touched by the deep one's (and the other way round)
        k0, v0, _, _ = gpu.read_kv(0, 0, 0, 4, seq=0)
        k4, v4, _, _ = gpu.read_kv(0, 0, 0, 4, seq=N_DISTINCT)
        assert np.array_equal(k0[:2], k4[:2]) and np.array_equal(v0[:2], v4[:2]) and not np.any(k0[2:]) and not np.any(v0[2:])
        cpu = oracle.OracleModel(cfg, c4_model, kv_f16=True, simd=True)
        for L in range(cfg["n_layers"]):
            for hh in range(cfg["nkv"]):
                k, v, _, _ = gpu.read_kv(L, hh, 0, n + 2, seq=B - 1)
                cpu.load_rows(L, hh, 0, k.astype(np.float32), v.astype(np.float32))
        cpu.freeze()
        _say(capsys, "config 4, batch 8: oracle holds the deep sequence's rows")
        for step, (deep, got, toks) in enumerate(steps):
            want = cpu.forward(deep, n + step)
            tol = 5e-3 * float(np.max(np.abs(want)))
            err = float(np.max(np.abs(got[B - 1] - want)))
            assert err < tol, (step, err, tol)
            top2 = np.sort(want)[-2:]
            if top2[1] - top2[0] > 2 * tol:
                assert int(toks[B - 1]) == oracle.argmax_first(want), step
        assert gpu.uses_graph()
    finally:
        gpu.close()
