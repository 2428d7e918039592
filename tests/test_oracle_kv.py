"""Pins for the oracle's long-context attention options: sliding window with sinks, INT8 / FP8 KV rows.

Known answers come from the reference's own unit tests (crates/oxibonsai-model/src/layers/sliding_window.rs:191-328,
crates/oxibonsai-core/src/quant_fp8.rs:603-800, crates/oxibonsai-model/tests/kv_cache_quant_tests.rs,
fp8_kv_cache_tests.rs); what those leave open is fixed by torch's float8 types (an independent implementation of
the same two formats), by a float64 nearest-value search over the code table, and by float64 numpy restatements.
"""
import numpy as np
import pytest
import torch

from oracle import oracle
from test_oracle_layers import _f64_forward


# ---- sliding window ----------------------------------------------------------------------------------------
def _positions(pos, seq_len, window, sinks):
    """attention_range's list, from the closed form (sliding_window.rs:53-98 returns nothing for window 0)."""
    eff = min(seq_len, pos + 1)
    return [t for t in range(eff) if oracle.in_window(t, pos, window, sinks)]


def test_window_positions_of_the_reference_unit_tests():
    assert _positions(4, 5, 8, 2) == [0, 1, 2, 3, 4]          # small_sequence_within_window
    assert _positions(10, 11, 4, 2) == [0, 1, 9, 10]          # window_slides_past_beginning
    assert {0, 1} <= set(_positions(100, 101, 4, 2))          # sink_tokens_always_included
    assert _positions(10, 11, 3, 0) == [8, 9, 10]             # window_with_no_sinks
    assert _positions(0, 0, 4096, 4) == []                    # empty_sequence
    assert _positions(5, 6, 3, 1) == [0, 4, 5]                # mask_application / eviction
    assert len(_positions(1000, 1001, 4, 2)) <= 4             # window_total_count_bounded
    # is_in_window_basic
    assert oracle.in_window(0, 100, 4, 2) and oracle.in_window(1, 100, 4, 2)
    assert oracle.in_window(100, 100, 4, 2) and oracle.in_window(99, 100, 4, 2)
    assert not oracle.in_window(98, 100, 4, 2)
    assert not any(oracle.in_window(t, 2, 0, 0) for t in range(3))   # zero_window_masks_everything
    assert not oracle.in_window(7, 5, 8, 0)                          # a key after the query


def test_window_closed_form_equals_the_range_construction():
    """attention_range builds the list from sinks + a recent run; is_in_window is the per-key form.  Both must
    describe the same set (brute force over small cases, the list rebuilt here from the reference's description)."""
    for window in range(1, 9):
        for sinks in range(0, 10):
            for pos in range(0, 20):
                eff = pos + 1
                if window >= eff:
                    want = list(range(eff))
                else:
                    sc = min(sinks, eff)
                    budget = max(window - sc, 0)
                    start = max(pos + 1 - budget, sc) if pos + 1 > budget else sc
                    want = list(range(sc)) + list(range(start, pos + 1))
                assert _positions(pos, eff, window, sinks) == want, (window, sinks, pos)


def test_windowed_attention_matches_float64_softmax_over_the_visible_keys():
    rng = np.random.default_rng(11)
    hd, T = 32, 90
    q = rng.standard_normal(hd).astype(np.float32)
    K, V = rng.standard_normal((T, hd)).astype(np.float32), rng.standard_normal((T, hd)).astype(np.float32)
    for window, sinks in ((16, 4), (5, 0), (3, 7), (200, 4), (1, 0)):
        vis = np.array([oracle.in_window(t, T - 1, window, sinks) for t in range(T)])
        sc = (K.astype(np.float64) @ q) / np.sqrt(hd)
        p = np.where(vis, np.exp(sc - sc[vis].max()), 0.0)
        want = (p / p.sum()) @ V.astype(np.float64)
        got = oracle.attention_head_windowed(q, K, V, T, hd, window, sinks)
        assert np.max(np.abs(got - want)) < 1e-5, (window, sinks)
    # window 0 in the attention call means "no window": the plain attention
    assert np.array_equal(oracle.attention_head_windowed(q, K, V, T, hd, 0, 0), oracle.attention_head(q, K, V, T, hd))


# ---- FP8 codes ---------------------------------------------------------------------------------------------
FORMATS = ((False, torch.float8_e4m3fn, 448.0), (True, torch.float8_e5m2, 57344.0))


def test_fp8_known_answers_of_the_reference():
    e4 = lambda v: int(oracle.fp8_encode([v])[0])
    e5 = lambda v: int(oracle.fp8_encode([v], True)[0])
    assert e4(0.0) == 0x00 and e4(-0.0) == 0x80 and e4(np.nan) == 0x7f
    assert e4(np.inf) == 0x7e and e4(-np.inf) == 0xfe and e4(448.0) == 0x7e and e4(-448.0) == 0xfe
    assert e4(2.0 ** -9) == 0x01 and e4(1000.0) == 0x7e
    assert e5(0.0) == 0x00 and e5(-0.0) == 0x80 and e5(np.inf) == 0x7c and e5(-np.inf) == 0xfc and e5(np.nan) == 0x7e
    assert e5(57344.0) == 0x7b and e5(1e6) == 0x7c            # beyond the largest finite value: infinity
    d4, d5 = oracle.fp8_decode(np.arange(256, dtype=np.uint8)), oracle.fp8_decode(np.arange(256, dtype=np.uint8), True)
    assert np.isnan(d4[0x7f]) and np.isnan(d4[0xff]) and d4[0x7e] == 448.0 and d4[0x00] == 0.0
    assert d4[0x80] == 0.0 and np.signbit(d4[0x80]) and d4[0x01] == 2.0 ** -9
    assert d5[0x7c] == np.inf and d5[0xfc] == -np.inf and np.isnan(d5[0x7e]) and d5[0x7b] == 57344.0
    for v in (0.0, 0.5, 1.0, -1.0, 2.0, -2.0, 100.0, 448.0, -448.0, 0.125):   # e4m3_round_trip_values
        assert abs(float(oracle.fp8_decode(oracle.fp8_encode([v]))[0]) - v) <= max(1.0, abs(v)) * 0.25


@pytest.mark.parametrize("e5m2,dtype,top", FORMATS)
def test_fp8_decode_equals_torch_for_every_byte(e5m2, dtype, top):
    b = np.arange(256, dtype=np.uint8)
    mine = oracle.fp8_decode(b, e5m2)
    ref = torch.from_numpy(b.copy()).view(dtype).float().numpy()
    fin = np.isfinite(ref)
    assert np.array_equal(mine[fin], ref[fin]) and np.array_equal(np.signbit(mine[fin]), np.signbit(ref[fin]))
    assert np.array_equal(np.isnan(mine), np.isnan(ref)) and np.array_equal(mine[np.isinf(ref)], ref[np.isinf(ref)])


@pytest.mark.parametrize("e5m2,dtype,top", FORMATS)
def test_fp8_encode_is_round_to_nearest_even(e5m2, dtype, top):
    table = oracle.fp8_decode(np.arange(128, dtype=np.uint8), e5m2).astype(np.float64)   # non-negative codes
    fin = np.isfinite(table)
    codes_fin, vals = np.arange(128)[fin], table[fin]
    rng = np.random.default_rng(5)
    mids = ((vals[:-1] + vals[1:]) / 2).astype(np.float32)
    x = np.concatenate([rng.normal(0, 1, 4000), rng.uniform(-top, top, 4000), rng.normal(0, 2e-3, 4000),
                        rng.normal(0, 2e-5, 4000), vals, -vals, mids, -mids,
                        np.nextafter(mids, np.float32(np.inf)), np.nextafter(mids, np.float32(0))]).astype(np.float32)
    x = x[np.abs(x) <= top]
    got = oracle.fp8_encode(x, e5m2)
    # torch converts with the same rounding inside the finite range
    assert np.array_equal(got, torch.from_numpy(x).to(dtype).view(torch.uint8).numpy())
    # and a float64 search over the table: nearest value, ties to the even code
    a = np.abs(x.astype(np.float64))
    d = np.abs(a[:, None] - vals[None, :])
    best = d.min(axis=1)
    for i in range(x.size):
        cand = codes_fin[d[i] == best[i]]
        want = cand[0] if cand.size == 1 else cand[cand % 2 == 0][0]
        assert (got[i] & 0x7f) == want and (got[i] >> 7) == int(np.signbit(x[i])), (x[i], hex(got[i]), hex(want))


# ---- rows ----------------------------------------------------------------------------------------------------
def test_int8_rows():
    codes, scale = oracle.kv_quantize_row(oracle.KV_I8, [127.0, -127.0, 0.0])      # quantize_row_exact_range
    assert abs(scale - 1.0) < 1e-5 and list(codes.view(np.int8)) == [127, -127, 0]
    codes, scale = oracle.kv_quantize_row(oracle.KV_I8, np.zeros(8))               # all-zero row: scale = f32::EPSILON
    assert scale == np.finfo(np.float32).eps and not codes.any()
    assert np.all(np.abs(oracle.kv_dequantize_row(oracle.KV_I8, codes, scale)) < 1e-5)
    row = (np.arange(64) * 0.1 - 3.2).astype(np.float32)                            # quantize_row_roundtrip_small_error
    codes, scale = oracle.kv_quantize_row(oracle.KV_I8, row)
    deq = oracle.kv_dequantize_row(oracle.KV_I8, codes, scale)
    assert np.mean(np.abs(deq - row)) < np.max(np.abs(row)) * 0.005
    rng = np.random.default_rng(2)
    for n in (1, 32, 128, 256):
        row = (rng.standard_normal(n) * rng.uniform(1e-3, 50)).astype(np.float32)
        codes, scale = oracle.kv_quantize_row(oracle.KV_I8, row)
        s = np.float32(max(np.float32(np.max(np.abs(row))) / np.float32(127.0), np.finfo(np.float32).eps))
        t = (row / s).astype(np.float32).astype(np.float64)
        want = np.clip(np.sign(t) * np.floor(np.abs(t) + 0.5), -127, 127).astype(np.int8)   # round half away from zero
        assert scale == s and np.array_equal(codes.view(np.int8), want)
        assert np.array_equal(oracle.kv_dequantize_row(oracle.KV_I8, codes, scale), want.astype(np.float32) * s)
        assert np.max(np.abs(codes.view(np.int8))) == 127                           # the largest value takes the top code


@pytest.mark.parametrize("e5m2,dtype,top", FORMATS)
def test_fp8_rows(e5m2, dtype, top):
    mode = oracle.KV_FP8_E5M2 if e5m2 else oracle.KV_FP8_E4M3
    codes, scale = oracle.kv_quantize_row(mode, np.zeros(16))
    assert scale == np.finfo(np.float32).eps and not codes.any()                    # all-zero row -> 0x00 bytes
    rng = np.random.default_rng(4)
    for n in (1, 32, 128, 256):
        row = (rng.standard_normal(n) * rng.uniform(1e-3, 50)).astype(np.float32)
        codes, scale = oracle.kv_quantize_row(mode, row)
        s = np.float32(max(np.float32(np.max(np.abs(row))) / np.float32(top), np.finfo(np.float32).eps))
        t = (row / s).astype(np.float32)
        assert scale == s
        inside = np.abs(t) <= top     # a quotient that rounds above the top value leaves the finite range (E5M2: infinity)
        assert np.array_equal(codes[inside], torch.from_numpy(t[inside]).to(dtype).view(torch.uint8).numpy())
        deq = oracle.kv_dequantize_row(mode, codes, scale)
        assert np.array_equal(deq, oracle.fp8_decode(codes, e5m2) * s)
        fin = np.isfinite(deq)
        assert np.max(np.abs(deq[fin] - row[fin])) <= np.max(np.abs(row)) * (0.13 if e5m2 else 0.07)


# ---- whole model ---------------------------------------------------------------------------------------------
BASE = dict(n_layers=2, h=128, inter=256, nq=4, nkv=2, hd=32, vocab=32, max_seq=16, eps=1e-6, rope_theta=1e6)


def _np_row(mode):
    top = {oracle.KV_I8: 127.0, oracle.KV_FP8_E4M3: 448.0, oracle.KV_FP8_E5M2: 57344.0}[mode]

    def f(row):
        r = row.astype(np.float32)
        s = np.float32(max(np.float32(np.max(np.abs(r))) / np.float32(top), np.finfo(np.float32).eps))
        t = (r / s).astype(np.float32)
        if mode == oracle.KV_I8:
            q = np.clip(np.sign(t) * np.floor(np.abs(t.astype(np.float64)) + 0.5), -127, 127)
        else:
            dt = torch.float8_e5m2 if mode == oracle.KV_FP8_E5M2 else torch.float8_e4m3fn
            q = torch.from_numpy(np.clip(t, -top, top)).to(dt).float().numpy().astype(np.float64)
        return q * np.float64(s)
    return f


def test_e5m2_rows_of_the_reference_can_hold_infinity():
    """quantize_row_fp8 divides by scale = max|x| / 57344 rounded to f32; where that quotient of the largest element
    rounds one ulp above 57344, fp8_e5m2_encode's `abs > FP8_E5M2_MAX` branch returns infinity (quant_fp8.rs:229-231)
    and attention over such a row is NaN.  E4M3 (>= 448 saturates) and INT8 (clamp) have no such case.  This is why
    the device path offers INT8 and E4M3 caches only."""
    rng = np.random.default_rng(9)
    hit = {oracle.KV_FP8_E5M2: 0, oracle.KV_FP8_E4M3: 0, oracle.KV_I8: 0}
    for _ in range(400):
        row = (rng.standard_normal(64) * rng.uniform(0.1, 10)).astype(np.float32)
        for mode in hit:
            codes, scale = oracle.kv_quantize_row(mode, row)
            hit[mode] += int(not np.all(np.isfinite(oracle.kv_dequantize_row(mode, codes, scale))))
    assert hit[oracle.KV_FP8_E5M2] > 10 and hit[oracle.KV_FP8_E4M3] == 0 and hit[oracle.KV_I8] == 0


@pytest.mark.parametrize("mode", [oracle.KV_I8, oracle.KV_FP8_E4M3])
def test_model_with_quantised_cache_matches_float64_numpy(mode):
    from oxibonsai_amd import synth
    cfg = dict(BASE, fmt=0)
    w = synth.make_model(cfg, 17)
    hiddens = [synth.embedding_rows(3, [t], cfg["h"])[0] * 50.0 for t in (5, 9, 2, 30, 11, 4, 8)]
    want = _f64_forward(cfg, w, hiddens, kv_round=_np_row(mode))
    plain = _f64_forward(cfg, w, hiddens)
    m = oracle.OracleModel(cfg, w, kv_mode=mode)
    worst = moved = 0.0
    for pos, hid in enumerate(hiddens):
        got = m.forward(hid, pos)
        worst = max(worst, float(np.max(np.abs(got - want[pos]))))
        moved = max(moved, float(np.max(np.abs(plain[pos] - want[pos]))))
    scale = max(float(np.max(np.abs(x))) for x in want)
    assert worst < 2e-4 * max(1.0, scale) and moved > 10 * worst     # the quantisation is visible, and followed exactly
    k, v, kc, vc, ks, vs = m.cache()
    n = len(hiddens)
    assert kc is not None and np.all(ks[:, :, :n] > 0) and np.all(ks[:, :, n:] == 0)
    for L in range(cfg["n_layers"]):
        for hh in range(cfg["nkv"]):
            for t in range(n):
                assert np.array_equal(k[L, hh, t], oracle.kv_dequantize_row(mode, kc[L, hh, t], ks[L, hh, t]))
                assert np.array_equal(v[L, hh, t], oracle.kv_dequantize_row(mode, vc[L, hh, t], vs[L, hh, t]))


@pytest.mark.parametrize("window,sinks", [(4, 1), (3, 0), (2, 3), (64, 4)])
def test_model_with_sliding_window_matches_float64_numpy(window, sinks):
    from oxibonsai_amd import synth
    cfg = dict(BASE, fmt=1)
    w = synth.make_model(cfg, 19)
    hiddens = [synth.embedding_rows(3, [t], cfg["h"])[0] * 50.0 for t in (5, 9, 2, 30, 11, 4, 8, 1, 0, 3)]

    def visible(key, query):   # the reference's rule restated (sliding_window.rs:173-189)
        return key < sinks or (key <= query and query - key < max(window - sinks, 0))
    want = _f64_forward(cfg, w, hiddens, visible=visible)
    plain = _f64_forward(cfg, w, hiddens)
    m = oracle.OracleModel(cfg, w, window=window, sinks=sinks)
    for pos, hid in enumerate(hiddens):
        got = m.forward(hid, pos)
        assert np.max(np.abs(got - want[pos])) < 2e-4 * max(1.0, np.max(np.abs(want[pos]))), pos
    moved = max(float(np.max(np.abs(a - b))) for a, b in zip(plain, want))
    assert (moved == 0.0) if window >= len(hiddens) else (moved > 1e-3)
