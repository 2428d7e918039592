"""The committed vectors of tests/golden/vectors.npz (frozen outputs of this repository's oracle, see
tests/golden/make_vectors.py): the oracle must still reproduce them bit for bit, and the HIP path is held to them
through the C ABI with the tolerances of the other parity tests."""
import os
import sys

import numpy as np
import pytest

from helpers import Q1, TQ2, parity_violations
from oracle import oracle
from oxibonsai_amd import synth

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "golden"))
import make_vectors  # noqa: E402

G = np.load(os.path.join(HERE, "golden", "vectors.npz"))


def test_oracle_reproduces_the_committed_vectors_bit_for_bit():
    now = make_vectors.build()
    assert set(now) == set(G.files)
    for k in G.files:
        a, b = np.asarray(now[k]), G[k]
        assert a.dtype == b.dtype and a.shape == b.shape, k
        assert np.array_equal(a.view(np.uint8), b.view(np.uint8)), k   # bit patterns: NaN and -0 included


@pytest.mark.gpu
@pytest.mark.parametrize("fmt,name", [(Q1, "q1"), (TQ2, "tq2")])
def test_gemv_gemm_dequant_against_the_committed_vectors(backend, fmt, name):
    n, k, m = 48, 256, 5
    blocks, x = G[f"{name}_blocks"], G[f"{name}_x"]
    h = backend.upload_weights_raw(blocks, n, k) if fmt == Q1 else backend.upload_weights_ternary(blocks, n, k)
    try:
        assert np.array_equal(backend.dequant(h).reshape(-1).view(np.uint32), G[f"{name}_dequant"].reshape(-1).view(np.uint32))
        y = backend.gemv_q1_g128_cached(h, x[0], n, k) if fmt == Q1 else backend.gemv_tq2_g128_cached(h, x[0], n, k)
        assert parity_violations(y, G[f"{name}_gemv"]) == 0
    finally:
        backend.free_weights(h)
    got = backend.gemm_q1_g128(blocks, x, m, n, k) if fmt == Q1 else backend.gemm_tq2_g128(blocks, x, m, n, k)
    assert parity_violations(np.asarray(got).reshape(m, n), G[f"{name}_gemm"].reshape(m, n), 1e-3) == 0   # m <= 16: the fp32-exact route


@pytest.mark.gpu
def test_kv_row_quantiser_against_the_committed_vectors(backend):
    from oxibonsai_amd.model import KV_FP8_E4M3, KV_I8, kv_quantize_rows
    for mode, name in ((KV_I8, "i8"), (KV_FP8_E4M3, "e4m3")):
        codes, scales = kv_quantize_rows(mode, G["kv_rows"])
        assert np.array_equal(codes, G[f"kv_{name}_codes"]) and np.array_equal(scales, G[f"kv_{name}_scales"])


@pytest.mark.gpu
@pytest.mark.parametrize("fmt,name", [(Q1, "q1"), (TQ2, "tq2")])
@pytest.mark.parametrize("tag", ["f16", "i8", "e4m3", "f16_w4_1"])
def test_model_logits_against_the_committed_vectors(backend, fmt, name, tag):
    from oxibonsai_amd.model import KV_F16, KV_FP8_E4M3, KV_I8, HipModel
    cfg = dict(make_vectors.TINY, fmt=fmt)
    w = synth.make_model(cfg, 60 + fmt)
    opts = {"f16": (KV_F16, 0, 0, 1e-3), "i8": (KV_I8, 0, 0, 2e-3), "e4m3": (KV_FP8_E4M3, 0, 0, 5e-3), "f16_w4_1": (KV_F16, 4, 1, 1e-3)}[tag]
    gpu = HipModel(backend, cfg, w, batch=1)
    try:
        gpu.set_attention(opts[0], opts[1], opts[2])
        want = G[f"model_{name}_{tag}_logits"]
        for p, t in enumerate((3, 17, 5, 29, 11, 2)):
            got, _ = gpu.forward(synth.embedding_rows(61, [t], cfg["h"])[0] * 50.0, p)
            assert parity_violations(got[0], want[p], opts[3]) == 0, (p, float(np.max(np.abs(got[0] - want[p]))))
    finally:
        gpu.close()


@pytest.mark.gpu
@pytest.mark.parametrize("tag", ["k40", "k300", "off_p95", "off_p1"])
def test_sampler_against_the_committed_vectors(backend, tag):
    from oxibonsai_amd.model import sample_logits
    T, k, tp = G[f"sample_{tag}_params"]
    toks, states = sample_logits(G["sample_logits"], float(T), int(k), float(tp), G["sample_seeds"])
    assert np.array_equal(states, G[f"sample_{tag}_states"])
    # the exponentials differ from libm's in rare last places: at most one of the four draws may land on the
    # neighbouring candidate (tests/test_sampler.py checks that such a draw sits on the boundary)
    assert int(np.sum(toks != G[f"sample_{tag}_tokens"])) <= 1
