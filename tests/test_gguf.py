"""GGUF reader of the native-hip tier (host code, no GPU): header, metadata, tensor directory and the model
configuration, against files laid out as the reference's writer and reader define them
(crates/oxibonsai-core/src/gguf/{header,metadata,tensor_info,reader,writer}.rs; config.rs:41-118)."""
import struct

import numpy as np
import pytest

from helpers import GGUF_F16, GGUF_F32, GGUF_Q1, GGUF_TQ2, Q1, TQ2, gguf_bytes, model_gguf
from oxibonsai_amd import GpuError, synth
from oxibonsai_amd.model import gguf_info

TINY = dict(n_layers=2, h=128, inter=256, nq=4, nkv=2, hd=32, vocab=32, max_seq=512, eps=1e-6, rope_theta=1e4)


def _emb_f32(cfg):
    return synth.embedding_rows(3, range(cfg["vocab"]), cfg["h"]).astype(np.float32)


def _write(tmp_path, data, name="m.gguf"):
    p = tmp_path / name
    p.write_bytes(data)
    return str(p)


@pytest.mark.parametrize("fmt", [TQ2, Q1])
@pytest.mark.parametrize("layout", [dict(), dict(packed=True), dict(alignment=64), dict(version=2), dict(alignment=4096)])
def test_info_of_the_reference_parity_checkpoint(tmp_path, fmt, layout):
    cfg = dict(TINY, fmt=fmt)
    w = synth.make_model(cfg, 5)
    info = gguf_info(_write(tmp_path, model_gguf(cfg, w, GGUF_F32, _emb_f32(cfg), **layout)))
    for k in ("n_layers", "h", "inter", "nq", "nkv", "hd", "vocab"):
        assert info[k] == cfg[k], k
    assert info["fmt"] == fmt and info["embedding_type"] == GGUF_F32
    assert info["context_length"] == 512 and info["rope_theta"] == 1e4 and info["eps"] == np.float32(1e-6)
    assert info["architecture"] == "qwen3" and info["name"] == "SyntheticParityModel"
    assert info["version"] == layout.get("version", 3) and info["alignment"] == layout.get("alignment", 32)
    assert info["n_tensors"] == 3 + 11 * cfg["n_layers"]


def test_llm_keys_defaults_and_vocab_from_the_embedding_shape(tmp_path):
    # keys under "<arch>." win, "llm." is the fallback, the Bonsai-8B values the default (config.rs:55-98);
    # head_dim = hidden / heads; the embedding's row count overrides the metadata (model/types/mod.rs:73-86)
    emb = np.zeros((40, 256), dtype=np.float16)
    blk = np.zeros(2 * 256 // 128 * 18, dtype=np.uint8)
    md = [("general.architecture", "str", "bonsai"), ("llm.embedding_length", "u32", 256), ("bonsai.block_count", "u64", 3),
          ("llm.block_count", "u32", 9), ("llm.attention.head_count", "i32", 2), ("bonsai.vocab_size", "u32", 1000),
          ("llm.rope.freq_base", "f64", 5e5), ("some.flag", "bool", True), ("some.bytes", "arr_u8", [1, 2, 3]),
          ("some.i16", "i16", -5), ("some.u16", "u16", 7), ("some.i8", "i8", -1), ("some.u8", "u8", 200), ("some.i64", "i64", -9)]
    ts = [("token_embd.weight", [256, 40], GGUF_F16, emb.tobytes()), ("blk.0.attn_q.weight", [256, 2], GGUF_Q1, blk.tobytes())]
    info = gguf_info(_write(tmp_path, gguf_bytes(md, ts)))
    assert (info["h"], info["n_layers"], info["nq"], info["hd"], info["vocab"]) == (256, 3, 2, 128, 40)
    assert (info["nkv"], info["inter"], info["context_length"]) == (8, 14336, 65536)          # defaults
    assert info["rope_theta"] == 5e5 and info["eps"] == np.float32(1e-6)
    assert info["architecture"] == "bonsai" and info["name"] == "Bonsai-8B"
    assert info["fmt"] == Q1 and info["embedding_type"] == GGUF_F16


def _err(tmp_path, data):
    with pytest.raises(GpuError) as e:
        gguf_info(_write(tmp_path, data))
    assert e.value.kind == "InvalidArgument"
    return str(e.value)


def test_header_errors(tmp_path):
    good = gguf_bytes([], [])
    assert "magic" in _err(tmp_path, gguf_bytes([], [], magic=0xDEADBEEF))            # header.rs reject_invalid_magic
    for v in (1, 4):
        assert "version" in _err(tmp_path, gguf_bytes([], [], version=v))
    for cut in (0, 3, 7, 15, 23):
        assert "end of file" in _err(tmp_path, good[:cut] if cut else b"")
    # the header of the reference's parse_valid_header test: version 3, 291 tensors, 25 metadata entries, 24 bytes
    hdr = struct.pack("<IIQQ", 0x46554747, 3, 291, 25)
    assert "end of file at offset 24" in _err(tmp_path, hdr)
    with pytest.raises(GpuError):
        gguf_info(str(tmp_path / "does_not_exist.gguf"))


def test_truncated_directory_and_bad_entries(tmp_path):
    cfg = dict(TINY, fmt=TQ2)
    data = model_gguf(cfg, synth.make_model(cfg, 5), GGUF_F32, _emb_f32(cfg))
    assert "end of file" in _err(tmp_path, data[:200])                     # inside the metadata
    assert "end of file" in _err(tmp_path, data[:900])                     # inside the tensor directory
    bad_type = struct.pack("<IIQQ", 0x46554747, 3, 0, 1) + struct.pack("<Q", 1) + b"k" + struct.pack("<I", 77)
    assert "value type" in _err(tmp_path, bad_type)
    huge = gguf_bytes([], [])[:16] + struct.pack("<Q", 1) + struct.pack("<Q", 1 << 40)      # a 1 TiB key
    assert "end of file" in _err(tmp_path, huge)


def test_missing_and_unsupported_tensors(tmp_path):
    emb = np.zeros((4, 128), dtype=np.float32)
    ts = [("token_embd.weight", [128, 4], GGUF_F32, emb.tobytes())]
    assert "blk.0.attn_q.weight" in _err(tmp_path, gguf_bytes([], ts))
    assert "token_embd.weight" in _err(tmp_path, gguf_bytes([], []))
    q4 = ("blk.0.attn_q.weight", [128, 32], 2, b"")          # Q4_0: a format of the reference this tier does not run
    assert "tensor type 2" in _err(tmp_path, gguf_bytes([], ts + [q4]))
