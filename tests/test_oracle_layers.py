"""Pins the oracle's layer math (RMSNorm, SiLU/SwiGLU, RoPE, softmax, attention, argmax) with the
reference's closed-form tests and float64 numpy.  No GPU involved."""
import numpy as np

from oracle import oracle


# model/src/layers/rms_norm.rs:62-96, tests/layer_correctness_tests.rs:61-79
def test_rms_norm_kats():
    x = np.array([1, 2, 3, 4], dtype=np.float32)
    out = oracle.rms_norm(x, np.ones(4, np.float32), 1e-6)
    assert np.allclose(out, x / np.sqrt(7.5), atol=1e-5)
    out = oracle.rms_norm(np.ones(4, np.float32), np.full(4, 2.0, np.float32), 1e-6)
    assert np.allclose(out, 2.0, atol=1e-5)
    rng = np.random.default_rng(0)
    x, w = rng.standard_normal(2048).astype(np.float32), rng.standard_normal(2048).astype(np.float32)
    want = w.astype(np.float64) * x / np.sqrt(np.mean(x.astype(np.float64) ** 2) + 1e-6)
    assert np.max(np.abs(oracle.rms_norm(x, w, 1e-6) - want)) < 1e-5


# model/src/layers/swiglu.rs:36-55
def test_silu_swiglu_kats():
    assert abs(oracle.silu(0.0)) < 1e-6
    assert abs(oracle.silu(1.0) - 0.7311) < 1e-3
    out = oracle.swiglu([1.0, 0.0, -1.0], [2.0, 3.0, 4.0])
    assert abs(out[0] - oracle.silu(1.0) * 2.0) < 1e-5 and abs(out[1]) < 1e-5
    assert abs(out[2] - oracle.silu(-1.0) * 4.0) < 1e-5
    g = np.linspace(-20, 20, 401).astype(np.float32)
    want = g.astype(np.float64) / (1 + np.exp(-g.astype(np.float64)))
    assert np.max(np.abs(oracle.swiglu(g, np.ones_like(g)) - want)) < 1e-5


# model/src/layers/rope.rs:95-122, tests/layer_correctness_tests.rs:312-337
def test_rope_kats():
    c, s = oracle.rope_table(4, 16, 10000.0)
    v = np.array([1, 2, 3, 4], dtype=np.float32)
    assert np.allclose(oracle.rope_apply(v, c[0], s[0]), v, atol=1e-5)           # pos 0 = identity
    out = oracle.rope_apply(np.array([1, 0, 0, 1], np.float32), c[5], s[5])
    assert abs(np.linalg.norm(out) - np.sqrt(2.0)) < 1e-4                         # norm preserved
    # hd = 4, pos = 1 closed form: pairs (0,2) and (1,3), freq_i = base^(-2i/hd)
    out = oracle.rope_apply(v, c[1], s[1])
    f = [1.0, 10000.0 ** -0.5]
    want = [1 * np.cos(f[0]) - 3 * np.sin(f[0]), 2 * np.cos(f[1]) - 4 * np.sin(f[1]),
            1 * np.sin(f[0]) + 3 * np.cos(f[0]), 2 * np.sin(f[1]) + 4 * np.cos(f[1])]
    assert np.allclose(out, want, atol=1e-5)
    c, s = oracle.rope_table(128, 64, 1e6)
    i = np.arange(64, dtype=np.float64)
    ang = 37 * (1e6 ** (-2 * i / 128))
    assert np.max(np.abs(c[37] - np.cos(ang))) < 2e-5 and np.max(np.abs(s[37] - np.sin(ang))) < 2e-5


def test_softmax():
    p = oracle.softmax([1.0, 2.0, 3.0])
    e = np.exp(np.array([1.0, 2.0, 3.0]) - 3.0)
    assert np.allclose(p, e / e.sum(), atol=1e-6) and abs(p.sum() - 1) < 1e-6
    assert np.allclose(oracle.softmax([1000.0, 1000.0]), 0.5)


# tests/layer_correctness_tests.rs:343-515
def test_attention_kats_and_float64():
    rng = np.random.default_rng(3)
    hd = 32
    q = rng.standard_normal(hd).astype(np.float32)
    k1, v1 = rng.standard_normal((1, hd)).astype(np.float32), rng.standard_normal((1, hd)).astype(np.float32)
    assert np.allclose(oracle.attention_head(q, k1, v1, 1, hd), v1[0], atol=1e-6)   # single token returns V
    T = 77
    K, V = rng.standard_normal((T, hd)).astype(np.float32), rng.standard_normal((T, hd)).astype(np.float32)
    sc = (K.astype(np.float64) @ q) / np.sqrt(hd)
    p = np.exp(sc - sc.max())
    p /= p.sum()
    want = p @ V.astype(np.float64)
    assert np.max(np.abs(oracle.attention_head(q, K, V, T, hd) - want)) < 1e-5
    assert np.all(oracle.attention_head(q, K, V, 0, hd) == 0.0)                      # seq_len 0 -> zeros
    # identical keys -> uniform weights -> mean of V
    Ksame = np.tile(K[:1], (T, 1))
    assert np.allclose(oracle.attention_head(q, Ksame, V, T, hd), V.mean(axis=0), atol=1e-5)


def test_argmax_tie_rules():
    v = np.array([1.0, 5.0, 3.0, 5.0, 2.0], dtype=np.float32)
    assert oracle.argmax_last(v) == 3      # runtime/src/sampling.rs:182-189 (max_by keeps the last)
    assert oracle.argmax_first(v) == 1     # gpu_backend/cuda_kernels.rs:407-436 (strict >)


# ---- whole-model decode against an independent float64 numpy forward -------------------------------
def _f64_forward(cfg, w, hiddens, kv_round=None, visible=None):
    """Textbook Qwen3 decode in float64 from the dequantised matrices (no oracle code involved except dequant,
    which test_oracle.py pins bit for bit).  kv_round(row) -> the row as a cache of limited precision returns it;
    visible(key, query) -> whether the query's attention may look at the key."""
    from helpers import dense_f64
    fmt, h, hd, nq, nkv = cfg["fmt"], cfg["h"], cfg["hd"], cfg["nq"], cfg["nkv"]
    inter, half = cfg["inter"], cfg["hd"] // 2

    def rms(x, wt):
        return wt * x / np.sqrt(np.mean(x * x) + cfg["eps"])

    def rope(v, pos):
        i = np.arange(half, dtype=np.float64)
        ang = pos * cfg["rope_theta"] ** (-2.0 * i / hd)
        c, s = np.cos(ang), np.sin(ang)
        return np.concatenate([v[:half] * c - v[half:] * s, v[:half] * s + v[half:] * c])

    mats = [{k: dense_f64(fmt, lw[k], *shape) for k, shape in
             (("q", (nq * hd, h)), ("k", (nkv * hd, h)), ("v", (nkv * hd, h)), ("o", (h, nq * hd)),
              ("gate", (inter, h)), ("up", (inter, h)), ("down", (h, inter)))} for lw in w["layers"]]
    lm = dense_f64(fmt, w["lm_head"], cfg["vocab"], h)
    K = [[[] for _ in range(nkv)] for _ in w["layers"]]
    V = [[[] for _ in range(nkv)] for _ in w["layers"]]
    outs = []
    for pos, hid in enumerate(hiddens):
        x = hid.astype(np.float64)
        for L, lw in enumerate(w["layers"]):
            n = rms(x, lw["attn_norm"].astype(np.float64))
            q, k, v = mats[L]["q"] @ n, mats[L]["k"] @ n, mats[L]["v"] @ n
            for kh in range(nkv):
                kr, vr = rope(rms(k[kh * hd:(kh + 1) * hd], lw["k_norm"].astype(np.float64)), pos), v[kh * hd:(kh + 1) * hd]
                K[L][kh].append(kv_round(kr) if kv_round else kr)
                V[L][kh].append(kv_round(vr) if kv_round else vr)
            att = np.zeros(nq * hd)
            for qh in range(nq):
                qv = rope(rms(q[qh * hd:(qh + 1) * hd], lw["q_norm"].astype(np.float64)), pos)
                kh = qh // (nq // nkv)
                sc = np.array(K[L][kh]) @ qv / np.sqrt(hd)
                if visible:
                    sc = np.where([visible(t, pos) for t in range(pos + 1)], sc, -np.inf)
                p = np.exp(sc - sc.max())
                att[qh * hd:(qh + 1) * hd] = (p / p.sum()) @ np.array(V[L][kh])
            x = x + mats[L]["o"] @ att
            n = rms(x, lw["ffn_norm"].astype(np.float64))
            g, u = mats[L]["gate"] @ n, mats[L]["up"] @ n
            x = x + mats[L]["down"] @ (g / (1 + np.exp(-g)) * u)
        outs.append(lm @ rms(x, w["final_norm"].astype(np.float64)))
    return outs


def test_model_forward_matches_float64_numpy():
    import pytest
    from oxibonsai_amd import synth
    base = dict(n_layers=2, h=128, inter=256, nq=4, nkv=2, hd=32, vocab=32, max_seq=16, eps=1e-6, rope_theta=1e6)
    for fmt in (0, 1):
        cfg = dict(base, fmt=fmt)
        w = synth.make_model(cfg, 7 + fmt)
        hiddens = [synth.embedding_rows(3, [t], cfg["h"])[0] * 50.0 for t in (5, 9, 2, 30, 11, 4)]
        want = _f64_forward(cfg, w, hiddens)
        m = oracle.OracleModel(cfg, w, kv_f16=False)
        for pos, hid in enumerate(hiddens):
            got = m.forward(hid, pos)
            assert np.max(np.abs(got - want[pos])) < 2e-4 * max(1.0, np.max(np.abs(want[pos]))), (fmt, pos)
        # the double-sum variant of the linear layers (a yardstick, not the reference's arithmetic) sits closer to
        # the float64 forward than the fp32 sums do
        m64 = oracle.OracleModel(cfg, w, kv_f16=False, dot_f64=True)
        e32 = e64 = 0.0
        m = oracle.OracleModel(cfg, w, kv_f16=False)
        for pos, hid in enumerate(hiddens):
            e32 = max(e32, float(np.max(np.abs(m.forward(hid, pos) - want[pos]))))
            e64 = max(e64, float(np.max(np.abs(m64.forward(hid, pos) - want[pos]))))
        assert e64 <= e32 and e64 < 2e-5 * max(1.0, max(float(np.max(np.abs(x))) for x in want))
        # with the f16 KV rounding of the reference's GPU cache the logits move, but only slightly
        m16 = oracle.OracleModel(cfg, w, kv_f16=True)
        d = max(np.max(np.abs(m16.forward(hid, pos) - want[pos])) for pos, hid in enumerate(hiddens))
        assert 0 < d < 2e-2
