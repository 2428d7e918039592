"""Sampler::sample (crates/oxibonsai-runtime/src/sampling.rs:84-177): the CPU restatement against the reference's own
unit tests and what the mathematics fixes, then the device sampler against the restatement."""
import numpy as np
import pytest

from oracle import oracle
from oxibonsai_amd import synth


def _xorshift(x):
    m = (1 << 64) - 1
    x ^= (x << 13) & m
    x ^= x >> 7
    x ^= (x << 17) & m
    return x


def test_reference_unit_tests():
    # greedy_sampling (:195-204), argmax_basic (:219-222)
    assert oracle.sample([0.1, 0.5, 0.3, 0.9, 0.2], 0.0, 40, 0.9, 42)[0] == 3
    assert oracle.sample([1.0, 3.0, 2.0], 0.0, 40, 0.9, 1)[0] == 1 and oracle.sample([5.0], 0.0, 40, 0.9, 1)[0] == 0
    # sampling_returns_valid_index (:206-216): defaults, seed 12345, 50 draws over 100 equal logits
    st = 12345
    for _ in range(50):
        tok, st, *_ = oracle.sample(np.zeros(100, np.float32), 0.7, 40, 0.9, st)
        assert tok < 100
    # buffer_reuse_across_calls (:224-243): top_k = 5 over ascending logits -> only 195..199
    st, logits = 99, np.arange(200, dtype=np.float32) * np.float32(0.01)
    seen = set()
    for _ in range(20):
        tok, st, ids, p, r = oracle.sample(logits, 0.7, 5, 1.0, st)
        assert tok >= 195 and sorted(ids) == [195, 196, 197, 198, 199]
        seen.add(tok)
    assert len(seen) > 1


def test_generator_and_draw():
    # xorshift64 with shifts 13 / 7 / 17 (:73-80), r = (x as f64 / u64::MAX as f64) as f32 (:160)
    st = 42
    for _ in range(5):
        tok, new, ids, p, r = oracle.sample(np.zeros(8, np.float32), 1.0, 0, 1.0, st)
        assert new == _xorshift(st)
        assert r == np.float32(np.float64(new) / np.float64(2**64 - 1))
        st = new
    # a zero state stays zero: the draw is 0 and the first entry of the buffer wins - with top-k and top-p off the
    # buffer is still in index order (:98-104; no select, no sort), so that is token 0, not the most likely one
    tok, new, ids, *_ = oracle.sample([0.0, 5.0, 1.0], 1.0, 0, 1.0, 0)
    assert new == 0 and tok == 0 and list(ids) == [0, 1, 2]
    # top-p on: the stable descending sort (:136-137) puts the most likely token first
    tok, new, ids, *_ = oracle.sample([0.0, 5.0, 1.0], 1.0, 0, 0.999, 0)
    assert new == 0 and tok == 1 and list(ids) == [1, 2, 0]


def test_candidates_follow_the_definition():
    logits = synth.normal_f32(3, 500) * 3.0
    T, k, tp = 0.8, 50, 0.9
    tok, _, ids, p, r = oracle.sample(logits, T, k, tp, 777)
    scaled = (logits / np.float32(T)).astype(np.float64)
    order = np.argsort(-scaled, kind="stable")[:k]
    sm = np.exp(scaled[order] - scaled[order[0]])
    sm /= sm.sum()
    cut = int(np.argmax(np.cumsum(sm) > tp)) + 1
    assert list(ids) == list(order[:cut])
    assert np.allclose(p, sm[:cut] / sm[:cut].sum(), rtol=1e-5) and abs(float(p.sum()) - 1.0) < 1e-5
    assert tok == ids[int(np.argmax(np.cumsum(p) >= r))]
    # top_p that is never exceeded keeps everything; a tiny one keeps the best candidate only; low temperature -> argmax
    assert len(oracle.sample(logits, T, k, 1.5, 1)[2]) == k
    assert list(oracle.sample(logits, T, k, 1e-6, 1)[2]) == [order[0]]
    assert all(oracle.sample(logits, 1e-3, 40, 0.9, s)[0] == int(np.argmax(logits)) for s in (1, 2, 3))
    # frequencies of many draws follow the probabilities (top-p off)
    lg = np.array([2.0, 1.0, 0.0, -1.0], np.float32)
    want = np.exp(lg - 2.0) / np.exp(lg - 2.0).sum()
    st, counts = 0x9E3779B97F4A7C15, np.zeros(4)
    for _ in range(20000):
        tok, st, *_ = oracle.sample(lg, 1.0, 0, 1.0, st)
        counts[tok] += 1
    assert np.max(np.abs(counts / counts.sum() - want)) < 0.01


def test_unfiltered_path_follows_the_definition():
    """top_k = 0 (the Creative preset, presets.rs:57-63): softmax over the whole vocabulary summed in index order,
    stable descending sort for top-p, cumulative cut, renormalisation, pick - against numpy with the same f32 sums."""
    n, T, tp = 5000, 1.0, 0.95
    logits = (synth.normal_f32(11, n) * 2.0).astype(np.float32)
    logits[17] = logits[4000] = logits[3]                       # equal probabilities keep index order in the sort
    tok, new, ids, p, r = oracle.sample(logits, T, 0, tp, 0x9E3779B97F4A7C15)
    scaled = logits / np.float32(T)
    e = np.exp((scaled - scaled.max()).astype(np.float32)).astype(np.float32)
    s = np.float32(0.0)
    for v in e:
        s = np.float32(s + v)
    prob = (e / s).astype(np.float32)
    order = np.argsort(-prob.astype(np.float64), kind="stable")
    cum, cut = np.float32(0.0), n - 1
    for j, i in enumerate(order):
        cum = np.float32(cum + prob[i])
        if cum > np.float32(tp):
            cut = j
            break
    assert list(ids) == list(order[:cut + 1])
    s2 = np.float32(0.0)
    for i in order[:cut + 1]:
        s2 = np.float32(s2 + prob[i])
    want = (prob[order[:cut + 1]] / s2).astype(np.float32)
    assert np.max(np.abs(p - want)) <= 1.2e-7 * float(want.max())      # libm expf against numpy's exp: last place
    cum = np.float32(0.0)
    pick = ids[0]
    for i, q in zip(ids, p):
        cum = np.float32(cum + q)
        if r <= cum:
            pick = i
            break
    assert tok == pick
    # top-p off as well: index order throughout
    tok, _, ids, p, r = oracle.sample(logits, T, 0, 1.0, 777)
    assert list(ids) == list(range(n))
    cum, pick = np.float32(0.0), 0
    for i, q in enumerate(p):
        cum = np.float32(cum + q)
        if r <= cum:
            pick = i
            break
    assert tok == pick and pick != int(np.argmax(logits))       # an ordinary draw lands somewhere in the middle


# --------------------------------------------------------------------------- GPU
@pytest.mark.gpu
@pytest.mark.parametrize("n,T,k,tp", [(151936, 0.7, 40, 0.9), (5000, 1.0, 128, 1.0), (33, 0.5, 40, 0.95), (4096, 2.0, 1, 0.9),
                                      (2049, 0.7, 5, 1.0), (100000, 1e-3, 40, 0.9), (151936, 1.0, 128, 0.9), (151936, 0.9, 82, 1.0)])
def test_device_sampler_matches_restatement(backend, n, T, k, tp):
    from oxibonsai_amd.model import sample_logits
    rows = 6
    logits = (synth.normal_f32(n + k, rows * n) * 4.0).reshape(rows, n)
    logits[1, 7] = logits[1, 99 % n] = logits[1].max() + 1.0          # an exact tie at the top
    seeds = np.array([1, 42, 2**63 + 5, 12345, 99, 0], dtype=np.uint64)
    toks, states = sample_logits(logits, T, k, tp, seeds)
    for b in range(rows):
        tok, new, ids, p, r = oracle.sample(logits[b], T, k, tp, int(seeds[b]))
        assert int(states[b]) == new
        if int(toks[b]) != tok:
            # libm and device exp may differ in the last place: then the draw must sit on a cumulative boundary
            cum = np.cumsum(p.astype(np.float64))
            assert int(toks[b]) in ids and np.min(np.abs(cum - r)) < 1e-5, (b, int(toks[b]), tok)
    # a second call continues the generators
    toks2, states2 = sample_logits(logits, T, k, tp, states)
    for b in range(rows):
        assert int(states2[b]) == _xorshift(int(states[b]))


@pytest.mark.gpu
def test_device_sampler_orders_signs_zeros_ties_and_infinities(backend):
    # the selection compares the logits as integer keys: negative numbers, both zeros, -inf and long runs of equal
    # values must come out in the order the restatement's (value descending, index ascending) sort gives
    from oxibonsai_amd.model import sample_logits
    n, k = 6000, 64
    base = np.round(synth.normal_f32(3, 4 * n).reshape(4, n) * 3.0) / 2.0      # half-integers: many exact ties
    base[0, ::7] = -np.inf
    base[1] = -np.abs(base[1]) - 1.0                                             # all negative
    base[2, :] = 0.0
    base[2, 1::2] = -0.0                                                        # only zeros of both signs
    base[3, :] = -np.inf
    base[3, [5, 4097, 2048]] = [-2.0, -2.0, -7.5]                                # three finite candidates
    seeds = np.array([2**63 + 5, 12345678901234567, 0x9E3779B97F4A7C15, 42424242424242], dtype=np.uint64)
    toks, states = sample_logits(base.astype(np.float32), 1.0, k, 1.0, seeds)
    for b in range(4):
        tok, new, ids, p, r = oracle.sample(base[b].astype(np.float32), 1.0, k, 1.0, int(seeds[b]))
        assert int(states[b]) == new
        if int(toks[b]) != tok:
            cum = np.cumsum(p.astype(np.float64))
            assert int(toks[b]) in ids and np.min(np.abs(cum - r)) < 1e-5, (b, int(toks[b]), tok)


@pytest.mark.gpu
def test_device_sampler_statistics_and_errors(backend):
    from oxibonsai_amd import GpuError
    from oxibonsai_amd.model import sample_logits
    lg = np.tile(np.array([2.0, 1.0, 0.0, -1.0] + [-30.0] * 60, np.float32), (512, 1))
    want = np.exp(lg[0, :4] - 2.0) / np.exp(lg[0, :4] - 2.0).sum()
    st = (np.arange(512, dtype=np.uint64) + 1) * np.uint64(0x9E3779B97F4A7C15)
    counts = np.zeros(64)
    for _ in range(20):
        toks, st = sample_logits(lg, 1.0, 8, 1.0, st)
        counts += np.bincount(toks, minlength=64)
    assert counts[4:].sum() == 0 and np.max(np.abs(counts[:4] / counts.sum() - want)) < 0.02
    assert sample_logits([0.1, 0.5, 0.3, 0.9, 0.2], 0.0, 40, 0.9, 42)[0][0] == 3          # greedy_sampling
    for bad in ((-1.0, 40, 0.9), (0.7, 40, 0.0), (float("nan"), 40, 0.9)):
        with pytest.raises(GpuError) as e:
            sample_logits(lg[:2], *bad, [1, 2])
        assert e.value.kind == "InvalidArgument"


@pytest.mark.gpu
@pytest.mark.parametrize("n,T,tp,top_k", [(151936, 1.0, 0.95, 0), (151936, 0.7, 1.0, 0), (5000, 1.0, 0.95, 0), (5000, 2.0, 1.0, 0),
                                          (33, 0.5, 0.95, 40), (33, 0.5, 1.0, 40), (1, 1.0, 0.9, 0), (64, 1.0, 0.5, 0),
                                          (2049, 0.05, 0.9, 0),
                                          # a top-k beyond the selection kernels: whole-row sort, the first top_k entries
                                          (151936, 0.8, 0.95, 1000), (151936, 1.0, 1.0, 129), (5000, 1.0, 0.9, 300),
                                          (300, 1.0, 0.9, 299), (5000, 0.7, 1.0, 4999)])
def test_device_sampler_with_the_filter_off(backend, n, T, tp, top_k):
    """top_k = 0 (and top_k >= the vocabulary, which the reference treats alike): softmax, sort, cut and pick over the
    whole vocabulary with every sum taken in the reference's order.  The device must return the restatement's token;
    where they differ, the two tokens must be neighbours in the buffer and the draw must sit on their boundary (the
    device's exponential goes through double precision, libm's expf is not always the nearest f32)."""
    from oxibonsai_amd.model import sample_logits
    rows = 6
    spread = 4.0 if n < 100000 else 0.05                 # the large rows are nearly flat: 150 000 comparable probabilities
    logits = (synth.normal_f32(n + 7, rows * n) * spread).reshape(rows, n)
    if n > 100:
        logits[1, 7] = logits[1, 99] = logits[1].max() + 1.0       # equal probabilities: the sort keeps index order
        logits[2, 50:60] = 3.0 * spread + logits[2].max()            # a peaked row
    seeds = np.array([1, 42, 2**63 + 5, 0x9E3779B97F4A7C15, 99, 0], dtype=np.uint64)
    toks, states = sample_logits(logits, T, top_k, tp, seeds)
    differing = 0
    for b in range(rows):
        tok, new, ids, p, r = oracle.sample(logits[b], T, top_k, tp, int(seeds[b]))
        assert int(states[b]) == new
        if int(toks[b]) != tok:
            differing += 1
            ids = list(ids)
            assert int(toks[b]) in ids, (b, int(toks[b]), tok)
            a, c = sorted((ids.index(int(toks[b])), ids.index(tok)))
            cum = np.float32(0.0)
            for q in p[:a + 1]:
                cum = np.float32(cum + q)
            assert c - a == 1 and abs(float(cum) - float(r)) < 1e-6, (b, a, c, float(cum), float(r))
    assert differing <= 1


@pytest.mark.gpu
@pytest.mark.parametrize("T,k,tp", [(0.9, 20, 0.95), (1.0, 0, 0.95), (0.8, 0, 1.0), (0.9, 200, 0.9)])
def test_sampled_generation_loop(backend, tmp_path, T, k, tp):
    """Token loop with the sampler (top-k by selection, filter off with and without top-p, top-k by sorting): every
    step's token is the sampler's pick from that step's logits."""
    from helpers import GGUF_F16, TQ2, model_gguf
    from oxibonsai_amd.model import HipModel
    cfg = dict(fmt=TQ2, n_layers=2, h=512, inter=1024, nq=8, nkv=2, hd=64, vocab=300, max_seq=128, eps=1e-6, rope_theta=1e6)
    w = synth.make_model(cfg, 9)
    table = (synth.embedding_rows(3, range(cfg["vocab"]), cfg["h"]) * 50.0).astype(np.float16)
    (tmp_path / "m.gguf").write_bytes(model_gguf(cfg, w, GGUF_F16, table))
    a, emb, _ = HipModel.from_gguf(backend, str(tmp_path / "m.gguf"), batch=2)
    b = HipModel(backend, cfg, w, batch=2)
    try:
        seeds = np.array([7, 1234567], dtype=np.uint64)
        ids, states = a.generate_sampled(emb, [5, 17], [0, 0], 12, T, k, tp, seeds)
        toks, st = np.array([5, 17], dtype=np.uint32), [int(s) for s in seeds]
        for i in range(12):
            logits, _ = b.forward(table[toks].astype(np.float32), [i, i])
            for s in range(2):
                tok, st[s], cand, p, r = oracle.sample(logits[s], T, k, tp, st[s])
                if int(ids[i, s]) != tok:
                    cum = np.cumsum(p, dtype=np.float32)                # sequential f32, the sampler's own sums
                    assert int(ids[i, s]) in cand and np.min(np.abs(cum - r)) < 1e-5
            toks = ids[i].copy()                                       # follow the device's own tokens
        assert [int(s) for s in states] == st
        greedy = a.generate(emb, [5, 17], [0, 0], 4)
        same, _ = a.generate_sampled(emb, [5, 17], [0, 0], 4, 0.0, 40, 0.9, seeds)      # temperature 0 = the greedy loop
        assert np.array_equal(greedy, same)
    finally:
        a.close()
        b.close()
        emb.close()


@pytest.mark.gpu
def test_device_sum_in_order_is_bit_exact(backend):
    """The softmax denominator must be the reference's element-by-element f32 sum.  The device takes 256 elements at
    a time without a chain where it can prove the result (no rounding tie, binade not left) and one by one elsewhere:
    both routes and the switches between them against numpy's sequential cumsum."""
    from oxibonsai_amd.model import sum_in_order
    rng = np.random.default_rng(5)

    def ref(x):
        return np.cumsum(np.asarray(x, dtype=np.float32), dtype=np.float32)[-1]

    cases = {
        "softmax terms, flat": np.exp(rng.normal(0, 0.05, 151936)).astype(np.float32) * np.float32(0.9),
        "softmax terms, peaked": np.exp(rng.normal(0, 4.0, 151936) - 16).astype(np.float32),
        "many ties": np.concatenate([[np.float32(2.0**24)], rng.integers(1, 8, 100000).astype(np.float32)]),  # ulp 2 and up: odd terms tie
        "ties at every scale": np.ldexp(rng.integers(1, 4, 70000).astype(np.float32), rng.integers(-30, 2, 70000)).astype(np.float32),
        "one large element late": np.concatenate([np.full(5000, 1e-3, np.float32), [np.float32(900.0)], np.full(5000, 1e-3, np.float32)]),
        "zeros and subnormals": np.concatenate([np.zeros(300, np.float32), np.full(300, 1e-42, np.float32), np.ones(300, np.float32)]),
        "short": np.array([0.1, 0.2, 0.3], np.float32),
        "single": np.array([7.25], np.float32),
        "all zero": np.zeros(1000, np.float32),
        "crosses many binades": np.full(200000, 1.0, np.float32),
        "random magnitudes": np.exp(rng.normal(0, 6.0, 120001)).astype(np.float32),
        "odd length": np.exp(rng.normal(0, 1.0, 65537)).astype(np.float32),
    }
    for name, x in cases.items():
        got, want = sum_in_order(x), ref(x)
        assert got.tobytes() == want.tobytes(), (name, float(got), float(want))
