"""GGUF writer for synthetic checkpoints (tests and the loader leg of the bench).

Layout of GgufWriter::write (crates/oxibonsai-core/src/gguf/writer.rs:212-330): magic, version 3, tensor count,
metadata count, metadata {key string, value type u32, value}, tensor infos {name, n_dims u32, dims u64.., type u32,
offset u64}, padding to the alignment, tensor data.  Strings are u64 length + bytes; everything little-endian."""
from __future__ import annotations

import struct

import numpy as np

Q1 = 0

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
               meta_override: dict | None = None, type_override: dict | None = None, emb_rows: int | None = None,
               **kw) -> bytes:
    """The synthetic checkpoint of the reference's parity test
    (crates/oxibonsai-model/tests/metal_prefill_ternary_parity_tests.rs:79-224) for any geometry / format:
    cfg and w as for oxibonsai_amd.synth.make_model; emb_table = the stored bytes of token_embd.weight, which holds
    emb_rows rows (default: as many as the LM head, cfg["vocab"])."""
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

    ts = [("token_embd.weight", [h, emb_rows or cfg["vocab"]], emb_type, np.ascontiguousarray(emb_table).tobytes()),
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
