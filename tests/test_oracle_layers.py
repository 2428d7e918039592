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
