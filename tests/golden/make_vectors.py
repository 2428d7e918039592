"""Writes tests/golden/vectors.npz: inputs and outputs of this repository's CPU oracle, frozen.

These are NOT outputs of the reference (none could be produced: see README.md); they pin the oracle against
accidental change once its functions have been checked against the reference's known answers, and give the GPU
tests a second, committed yardstick.  Run from the repository root:  python tests/golden/make_vectors.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle import oracle  # noqa: E402
from oxibonsai_amd import synth  # noqa: E402

TINY = dict(n_layers=2, h=128, inter=256, nq=4, nkv=2, hd=32, vocab=32, max_seq=32, eps=1e-6, rope_theta=1e6)


def build() -> dict:
    out = {}
    for fmt, name in ((0, "q1"), (1, "tq2")):
        n, k, m = 48, 256, 5
        blocks = synth.make_blocks(fmt, 40 + fmt, n, k)
        x = synth.normal_f32(50 + fmt, m * k).reshape(m, k)
        out[f"{name}_blocks"] = np.frombuffer(bytes(blocks), dtype=np.uint8).copy()
        out[f"{name}_x"] = x
        out[f"{name}_dequant"] = oracle.dequant(fmt, blocks)
        out[f"{name}_gemv"] = oracle.gemv(fmt, blocks, x[0], n, k)
        out[f"{name}_gemm"] = oracle.gemm(fmt, blocks, x, m, n, k)
    rng = np.random.default_rng(7)
    rows = (rng.standard_normal((6, 64)) * np.array([1.0, 1e-3, 30.0, 1e-6, 1.0, 0.0])[:, None]).astype(np.float32)
    rows[4, :8] = [0.5, 1.5, -2.5, 127.0, -127.0, 63.5, 2.0 ** -9, 0.0]
    out["kv_rows"] = rows
    for mode, name in ((oracle.KV_I8, "i8"), (oracle.KV_FP8_E4M3, "e4m3"), (oracle.KV_FP8_E5M2, "e5m2")):
        cs = [oracle.kv_quantize_row(mode, r) for r in rows]
        out[f"kv_{name}_codes"] = np.stack([c for c, _ in cs])
        out[f"kv_{name}_scales"] = np.array([s for _, s in cs], dtype=np.float32)
    q = rng.standard_normal(32).astype(np.float32)
    K, V = rng.standard_normal((40, 32)).astype(np.float32), rng.standard_normal((40, 32)).astype(np.float32)
    out["attn_q"], out["attn_k"], out["attn_v"] = q, K, V
    out["attn_full"] = oracle.attention_head(q, K, V, 40, 32)
    out["attn_window_12_3"] = oracle.attention_head_windowed(q, K, V, 40, 32, 12, 3)
    for fmt, name in ((0, "q1"), (1, "tq2")):
        cfg = dict(TINY, fmt=fmt)
        w = synth.make_model(cfg, 60 + fmt)
        hid = [synth.embedding_rows(61, [t], cfg["h"])[0] * 50.0 for t in (3, 17, 5, 29, 11, 2)]
        for tag, kw in (("f16", dict(kv_mode=oracle.KV_F16)), ("i8", dict(kv_mode=oracle.KV_I8)),
                        ("e4m3", dict(kv_mode=oracle.KV_FP8_E4M3)), ("f16_w4_1", dict(kv_mode=oracle.KV_F16, window=4, sinks=1))):
            mdl = oracle.OracleModel(cfg, w, **kw)
            out[f"model_{name}_{tag}_logits"] = np.stack([mdl.forward(h, p) for p, h in enumerate(hid)])
    # Sampler::sample: logits, parameters, seeds -> tokens and advanced generator states, for the three routes
    # (top-k by selection, top-k by sorting, filter off)
    lg = (synth.normal_f32(70, 4 * 3000) * 3.0).reshape(4, 3000)
    lg[1, 5] = lg[1, 1234] = lg[1].max() + 0.5
    seeds = np.array([1, 2**63 + 5, 0x9E3779B97F4A7C15, 424242], dtype=np.uint64)
    out["sample_logits"], out["sample_seeds"] = lg, seeds
    for tag, (T, k, tp) in (("k40", (0.7, 40, 0.9)), ("k300", (1.0, 300, 0.95)), ("off_p95", (1.0, 0, 0.95)), ("off_p1", (0.8, 0, 1.0))):
        res = [oracle.sample(lg[b], T, k, tp, int(seeds[b])) for b in range(4)]
        out[f"sample_{tag}_params"] = np.array([T, k, tp], dtype=np.float64)
        out[f"sample_{tag}_tokens"] = np.array([r[0] for r in res], dtype=np.uint32)
        out[f"sample_{tag}_states"] = np.array([r[1] for r in res], dtype=np.uint64)
        out[f"sample_{tag}_draws"] = np.array([r[4] for r in res], dtype=np.float32)
    return out


if __name__ == "__main__":
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "vectors.npz")
    np.savez_compressed(path, **build())
    print(path, os.path.getsize(path), "bytes")
