"""Seeded synthetic inputs in the reference's on-disk block formats.

One generator feeds the GPU path, the CPU oracle and the CPU baseline, so all
three see identical bytes.  Everything derives from a SplitMix64 stream; numpy
only, no libm-dependent step touches the block bytes.

Block formats (bit-exact contract of the reference):
  Q1_0_g128   18 B  [d: f16 LE][qs: 16 B]   weight i = bit (qs[i/8] >> (i%8)) & 1 -> +d / -d
              (crates/oxibonsai-core/src/tensor.rs:25-32, 60-65)
  TQ2_0_g128  34 B  [qs: 32 B][d: f16 LE]   weight j = code (qs[j/4] >> 2*(j%4)) & 3,
              00 -> -1, 01 -> 0, 10 -> +1, 11 -> 0
              (crates/oxibonsai-core/src/quant_ternary.rs:64-71, 191-200)
"""
from __future__ import annotations

import numpy as np

Q1, TQ2 = 0, 1
QK = 128
BLOCK_BYTES = {Q1: 18, TQ2: 34}

_GOLDEN = np.uint64(0x9E3779B97F4A7C15)
_M1 = np.uint64(0xBF58476D1CE4E5B9)
_M2 = np.uint64(0x94D049BB133111EB)


def splitmix64(seed: int, n: int, offset: int = 0) -> np.ndarray:
    """Outputs offset .. offset+n-1 of the SplitMix64 stream started at ``seed``."""
    with np.errstate(over="ignore"):
        idx = np.arange(offset + 1, offset + n + 1, dtype=np.uint64)
        z = np.uint64(seed & 0xFFFFFFFFFFFFFFFF) + idx * _GOLDEN
        z = (z ^ (z >> np.uint64(30))) * _M1
        z = (z ^ (z >> np.uint64(27))) * _M2
        return z ^ (z >> np.uint64(31))


def uniform01(seed: int, n: int) -> np.ndarray:
    """float64 uniforms in [0, 1) from the top 53 bits."""
    return (splitmix64(seed, n) >> np.uint64(11)).astype(np.float64) * (1.0 / (1 << 53))


def normal_f32(seed: int, n: int, std: float = 1.0) -> np.ndarray:
    """N(0, std) float32 via Box-Muller in float64."""
    m = (n + 1) // 2
    u = uniform01(seed, 2 * m)
    r = np.sqrt(-2.0 * np.log(1.0 - u[:m]))
    t = 2.0 * np.pi * u[m:]
    out = np.concatenate([r * np.cos(t), r * np.sin(t)])[:n] * std
    return out.astype(np.float32)


def scales_f16(seed: int, n: int, lo: float, hi: float) -> np.ndarray:
    """U[lo, hi] rounded to nearest-even binary16, returned as uint16 bit patterns."""
    return (lo + (hi - lo) * uniform01(seed, n)).astype(np.float32).astype(np.float16).view(np.uint16)


_TRIT_CODES = np.array([((v % 3) | (((v // 3) % 3) << 2) | (((v // 9) % 3) << 4) | ((v // 27) << 6))
                        for v in range(81)], dtype=np.uint8)


def make_q1_blocks(seed: int, n_blocks: int, lo: float = 0.01, hi: float = 0.1) -> np.ndarray:
    """Q1_0_g128 AoS bytes: sign bits are raw PRNG bits (Bernoulli 0.5), scales U[lo, hi]."""
    out = np.empty((n_blocks, 18), dtype=np.uint8)
    out[:, 0:2] = scales_f16(seed ^ 0x5CA1E5, n_blocks, lo, hi).view(np.uint8).reshape(n_blocks, 2)
    out[:, 2:18] = splitmix64(seed, 2 * n_blocks).view(np.uint8).reshape(n_blocks, 16)
    return out.reshape(-1)


def make_tq2_blocks(seed: int, n_blocks: int, lo: float = 0.005, hi: float = 0.05) -> np.ndarray:
    """TQ2_0_g128 AoS bytes: codes uniform over {00, 01, 10} (never 11), scales U[lo, hi].

    Each 16-bit lane of the stream, reduced mod 81, supplies four base-3 digits = one code byte."""
    out = np.empty((n_blocks, 34), dtype=np.uint8)
    lanes = splitmix64(seed, 8 * n_blocks).view(np.uint16)
    out[:, 0:32] = _TRIT_CODES[lanes % np.uint16(81)].reshape(n_blocks, 32)
    out[:, 32:34] = scales_f16(seed ^ 0x5CA1E5, n_blocks, lo, hi).view(np.uint8).reshape(n_blocks, 2)
    return out.reshape(-1)


def make_blocks(fmt: int, seed: int, n_rows: int, k: int, **kw) -> np.ndarray:
    n = n_rows * (k // QK)
    return make_q1_blocks(seed, n, **kw) if fmt == Q1 else make_tq2_blocks(seed, n, **kw)


def f16_round(a: np.ndarray) -> np.ndarray:
    """Values as they are after f16 storage and widening back to f32 (norms, embeddings)."""
    return a.astype(np.float16).astype(np.float32)


def make_model(cfg: dict, seed: int) -> dict:
    """Random-init Qwen3-shaped weights in reference AoS blocks.

    cfg keys: fmt, n_layers, h, inter, nq, nkv, hd, vocab.  Norm weights are
    1 + N(0, 0.02) and embeddings N(0, 0.02), both stored through f16 as the
    reference loader widens F16 tensors (crates/oxibonsai-model/src/model/weight_loaders.rs:38-46)."""
    fmt, h, inter, hd = cfg["fmt"], cfg["h"], cfg["inter"], cfg["hd"]
    qd, kd = cfg["nq"] * hd, cfg["nkv"] * hd
    layers = []
    s = seed * 1000003
    for _ in range(cfg["n_layers"]):
        lw = {}
        for name, n in (("attn_norm", h), ("q_norm", hd), ("k_norm", hd), ("ffn_norm", h)):
            s += 1
            lw[name] = f16_round(1.0 + normal_f32(s, n, 0.02))
        for name, (nr, k) in (("q", (qd, h)), ("k", (kd, h)), ("v", (kd, h)), ("o", (h, qd)),
                               ("gate", (inter, h)), ("up", (inter, h)), ("down", (h, inter))):
            s += 1
            lw[name] = make_blocks(fmt, s, nr, k)
        layers.append(lw)
    return {"layers": layers,
            "final_norm": f16_round(1.0 + normal_f32(s + 1, h, 0.02)),
            "lm_head": make_blocks(fmt, s + 2, cfg["vocab"], h)}


def embedding_rows(seed: int, token_ids, h: int) -> np.ndarray:
    """Embedding rows N(0, 0.02) through f16, generated per token id so a 151 936-row
    table never has to exist on the host."""
    return np.stack([f16_round(normal_f32((seed << 20) ^ int(t), h, 0.02)) for t in token_ids])


def token_ids(seed: int, n: int, vocab: int) -> np.ndarray:
    """n token ids, uniform over 0 .. vocab - 1 (a seeded random prompt)."""
    return (splitmix64(seed, n) % np.uint64(vocab)).astype(np.uint32)
