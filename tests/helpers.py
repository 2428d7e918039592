"""Shared builders for the tests: reference-style blocks and the reference's own test generators."""
from __future__ import annotations

import numpy as np

Q1, TQ2 = 0, 1


def f16_bits(v: float) -> int:
    return int(np.array([v], dtype=np.float32).astype(np.float16).view(np.uint16)[0])


def q1_block(scale: float, bits) -> np.ndarray:
    """make_block / make_q1_block of the reference tests: [d f16 LE][16 B]
    (crates/oxibonsai-kernels/src/gemv.rs:94-99, tests/gpu_backend_tests.rs:282-290)."""
    b = np.zeros(18, dtype=np.uint8)
    h = f16_bits(scale)
    b[0], b[1] = h & 0xFF, h >> 8
    b[2:] = np.asarray(bits, dtype=np.uint8) if np.ndim(bits) else np.full(16, bits, dtype=np.uint8)
    return b


def tq2_block(scale: float, qs) -> np.ndarray:
    """make_g128_block of the reference tests: [32 B codes][d f16 LE]
    (crates/oxibonsai-kernels/src/gemv_ternary.rs:196-203)."""
    b = np.zeros(34, dtype=np.uint8)
    b[:32] = np.asarray(qs, dtype=np.uint8) if np.ndim(qs) else np.full(32, qs, dtype=np.uint8)
    h = f16_bits(scale)
    b[32], b[33] = h & 0xFF, h >> 8
    return b


def block(fmt: int, scale: float, pattern) -> np.ndarray:
    return q1_block(scale, pattern) if fmt == Q1 else tq2_block(scale, pattern)


def cross_tier_q1(n_rows: int, k: int) -> np.ndarray:
    """Generator of crates/oxibonsai-kernels/tests/cross_tier.rs:18-27:
    block i has scale 0.3 + 0.02 i and bits[j] = (37 i + 13 j + 7) & 0xFF."""
    n = n_rows * (k // 128)
    out = np.zeros((n, 18), dtype=np.uint8)
    for i in range(n):
        out[i] = q1_block(0.3 + 0.02 * i, [(37 * i + 13 * j + 7) & 0xFF for j in range(16)])
    return out.reshape(-1)


def simd_parity_tq2(n_rows: int, k: int):
    """Generator of the reference's SIMD-vs-scalar TQ2 test (crates/oxibonsai-kernels/src/simd_avx2.rs:1147-1160):
    qs = (17 r + 29 b + 11 i) & 0xFF, d = 0.25 + 0.01 r, x = ((7 i % 23) * 0.125) - 1.5."""
    bpr = k // 128
    out = np.zeros((n_rows * bpr, 34), dtype=np.uint8)
    for r in range(n_rows):
        for b in range(bpr):
            out[r * bpr + b] = tq2_block(0.25 + 0.01 * r, [(17 * r + 29 * b + 11 * i) & 0xFF for i in range(32)])
    x = np.array([((7 * i) % 23) * 0.125 - 1.5 for i in range(k)], dtype=np.float32)
    return out.reshape(-1), x


def metal_tq2(n_rows: int, k: int) -> np.ndarray:
    """Codes from the base-3 digits of 31 r + 17 b + byte, as the reference's Metal GEMV test builds them
    (crates/oxibonsai-kernels/src/gpu_backend/metal_graph/tests.rs:481-500); scale 0.01 (1 + (r + b) % 7)."""
    bpr = k // 128
    out = np.zeros((n_rows * bpr, 34), dtype=np.uint8)
    for r in range(n_rows):
        for b in range(bpr):
            qs = []
            for byte in range(32):
                v = 31 * r + 17 * b + byte
                code = 0
                for lane in range(4):
                    code |= (v % 3) << (2 * lane)
                    v //= 3
                qs.append(code)
            out[r * bpr + b] = tq2_block(0.01 * (1 + (r + b) % 7), qs)
    return out.reshape(-1)


def dense_f64(fmt: int, blocks: np.ndarray, n_rows: int, k: int) -> np.ndarray:
    """Independent float64 decode straight from the format definition (not through the oracle)."""
    bpr = k // 128
    if fmt == Q1:
        b = blocks.reshape(n_rows * bpr, 18)
        d = b[:, 0:2].copy().view(np.float16).astype(np.float64).reshape(-1, 1)
        bits = np.unpackbits(b[:, 2:], axis=1, bitorder="little").astype(np.float64)
        w = d * (2.0 * bits - 1.0)
    else:
        b = blocks.reshape(n_rows * bpr, 34)
        d = b[:, 32:34].copy().view(np.float16).astype(np.float64).reshape(-1, 1)
        codes = np.stack([(b[:, :32] >> s) & 3 for s in (0, 2, 4, 6)], axis=-1).reshape(-1, 128)
        w = d * np.array([-1.0, 0.0, 1.0, 0.0])[codes]
    return w.reshape(n_rows, k)


def rel_err(a: np.ndarray, b: np.ndarray) -> np.ndarray:
    """The reference's parity formula |a-b| / max(|a|, |b|, 1e-3)
    (crates/oxibonsai-model/tests/metal_prefill_ternary_parity_tests.rs:297-298)."""
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    return np.abs(a - b) / np.maximum(np.maximum(np.abs(a), np.abs(b)), 1e-3)


def parity_violations(a: np.ndarray, b: np.ndarray, tol: float = 1e-3) -> int:
    """Number of elements failing the reference's gate `abs_err < tol || rel_err < tol`
    (crates/oxibonsai-model/tests/metal_prefill_ternary_parity_tests.rs:294-308)."""
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    abs_err = np.abs(a - b)
    return int(np.count_nonzero(~((abs_err < tol) | (rel_err(a, b) < tol)) | ~np.isfinite(a) | ~np.isfinite(b)))


# ---------------------------------------------------------------------------
# GGUF files for the loader tests.  Layout of GgufWriter::write
# (crates/oxibonsai-core/src/gguf/writer.rs:212-330): magic, version 3, tensor count, metadata count, metadata
# {key string, value type u32, value}, tensor infos {name, n_dims u32, dims u64.., type u32, offset u64}, padding to
# the alignment, tensor data.  Strings are u64 length + bytes; everything little-endian.
# ---------------------------------------------------------------------------
import struct

GGUF_MAGIC = 0x46554747
GGUF_F32, GGUF_F16, GGUF_Q1, GGUF_TQ2 = 0, 1, 41, 42
_VT = {"u8": (0, "<B"), "i8": (1, "<b"), "u16": (2, "<H"), "i16": (3, "<h"), "u32": (4, "<I"), "i32": (5, "<i"),
       "f32": (6, "<f"), "bool": (7, "<B"), "u64": (10, "<Q"), "i64": (11, "<q"), "f64": (12, "<d")}


def _gguf_str(s: str) -> bytes:
    b = s.encode()
    return struct.pack("<Q", len(b)) + b


def _gguf_value(kind: str, v) -> bytes:
    if kind == "str":
        return struct.pack("<I", 8) + _gguf_str(v)
    if kind.startswith("arr_"):
        ek = kind[4:]
        head = struct.pack("<I", 9) + struct.pack("<I", 8 if ek == "str" else _VT[ek][0]) + struct.pack("<Q", len(v))
        return head + b"".join(_gguf_str(x) if ek == "str" else struct.pack(_VT[ek][1], x) for x in v)
    t, f = _VT[kind]
    return struct.pack("<I", t) + struct.pack(f, v)


def gguf_bytes(metadata, tensors, version: int = 3, alignment: int = 32, packed: bool = False,
               magic: int = GGUF_MAGIC) -> bytes:
    """metadata: list of (key, kind, value); tensors: list of (name, shape, type id, data bytes).
    packed=True lays the tensors back to back as the reference's writer does; otherwise every tensor starts at a
    multiple of the alignment, as files written by llama.cpp tools do.  An alignment other than 32 is announced
    with general.alignment."""
    md = list(metadata)
    if alignment != 32 and not any(k == "general.alignment" for k, _, _ in md):
        md.insert(0, ("general.alignment", "u32", alignment))
    out = bytearray(struct.pack("<IIQQ", magic, version, len(tensors), len(md)))
    for k, kind, v in md:
        out += _gguf_str(k) + _gguf_value(kind, v)
    offsets, off = [], 0
    for _, _, _, data in tensors:
        if not packed:
            off = (off + alignment - 1) // alignment * alignment
        offsets.append(off)
        off += len(data)
    for (name, shape, tid, _), o in zip(tensors, offsets):
        out += _gguf_str(name) + struct.pack("<I", len(shape)) + b"".join(struct.pack("<Q", d) for d in shape)
        out += struct.pack("<IQ", tid, o)
    out += b"\0" * ((-len(out)) % alignment)
    base = len(out)
    for (_, _, _, data), o in zip(tensors, offsets):
        out += b"\0" * (base + o - len(out))
        out += bytes(data)
    return bytes(out)


def model_gguf(cfg: dict, w: dict, emb_type: int, emb_table, arch: str = "qwen3", norm_f16: bool = False,
               meta_override: dict | None = None, type_override: dict | None = None, **kw) -> bytes:
    """The synthetic checkpoint of the reference's parity test
    (crates/oxibonsai-model/tests/metal_prefill_ternary_parity_tests.rs:79-224) for any geometry / format:
    cfg and w as for oxibonsai_amd.synth.make_model; emb_table = the stored bytes of token_embd.weight."""
    h, inter, hd = cfg["h"], cfg["inter"], cfg["hd"]
    qd, kd = cfg["nq"] * hd, cfg["nkv"] * hd
    mt = GGUF_Q1 if cfg["fmt"] == Q1 else GGUF_TQ2
    md = [("general.architecture", "str", arch), ("general.name", "str", "SyntheticParityModel"),
          (f"{arch}.embedding_length", "u32", h), (f"{arch}.block_count", "u32", cfg["n_layers"]),
          (f"{arch}.attention.head_count", "u32", cfg["nq"]), (f"{arch}.attention.head_count_kv", "u32", cfg["nkv"]),
          (f"{arch}.feed_forward_length", "u32", inter), (f"{arch}.vocab_size", "u32", cfg["vocab"]),
          (f"{arch}.context_length", "u32", cfg["max_seq"]), (f"{arch}.attention.layer_norm_rms_epsilon", "f32", cfg["eps"]),
          (f"{arch}.rope.freq_base", "f32", cfg["rope_theta"]),
          ("tokenizer.ggml.tokens", "arr_str", [f"<{i}>" for i in range(5)]), ("tokenizer.ggml.eos_token_id", "u32", 2)]

    if meta_override:          # e.g. {"feed_forward_length": 384}: metadata that contradicts the tensor shapes
        md = [(k, kind, meta_override.get(k.split(".", 1)[1], v)) for k, kind, v in md]

    def vec(v):
        a = np.asarray(v, dtype=np.float32)
        return (GGUF_F16, a.astype(np.float16).tobytes()) if norm_f16 else (GGUF_F32, a.tobytes())

    ts = [("token_embd.weight", [h, cfg["vocab"]], emb_type, np.ascontiguousarray(emb_table).tobytes()),
          ("output_norm.weight", [h], *vec(w["final_norm"])),
          ("output.weight", [h, cfg["vocab"]], mt, w["lm_head"].tobytes())]
    for i, lw in enumerate(w["layers"]):
        p = f"blk.{i}."
        ts += [(p + "attn_norm.weight", [h], *vec(lw["attn_norm"])), (p + "ffn_norm.weight", [h], *vec(lw["ffn_norm"])),
               (p + "attn_q_norm.weight", [hd], *vec(lw["q_norm"])), (p + "attn_k_norm.weight", [hd], *vec(lw["k_norm"])),
               (p + "attn_q.weight", [h, qd], mt, lw["q"].tobytes()), (p + "attn_k.weight", [h, kd], mt, lw["k"].tobytes()),
               (p + "attn_v.weight", [h, kd], mt, lw["v"].tobytes()), (p + "attn_output.weight", [qd, h], mt, lw["o"].tobytes()),
               (p + "ffn_gate.weight", [h, inter], mt, lw["gate"].tobytes()), (p + "ffn_up.weight", [h, inter], mt, lw["up"].tobytes()),
               (p + "ffn_down.weight", [inter, h], mt, lw["down"].tobytes())]
    if type_override:          # e.g. {"output.weight": GGUF_Q1}: a tensor stored in another format
        ts = [(n, sh, type_override.get(n, t), d) for n, sh, t, d in ts]
    return gguf_bytes(md, ts, **kw)
