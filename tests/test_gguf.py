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


# ---------------------------------------------------------------------------
# The byte strings of the reference's own parser tests (crates/oxibonsai-core/tests/gguf_edge_cases.rs:19-91 build
# them field by field; they are rebuilt here the same way, independently of the package's writer).
# ---------------------------------------------------------------------------
from oxibonsai_amd.model import gguf_metadata, gguf_tensor


def _hdr(magic, version, tensors, metadata):
    return struct.pack("<I", magic) + struct.pack("<I", version) + struct.pack("<Q", tensors) + struct.pack("<Q", metadata)


def _s(x):
    return struct.pack("<Q", len(x)) + x.encode()


def _tinfo(name, shape, type_id, offset):
    return _s(name) + struct.pack("<I", len(shape)) + b"".join(struct.pack("<Q", d) for d in shape) + \
        struct.pack("<I", type_id) + struct.pack("<Q", offset)


def test_reference_edge_case_files(tmp_path):
    # gguf_file_parse_with_one_metadata_entry (:506-520): "test.key" = 42u32
    data = _hdr(0x46554747, 3, 0, 1) + _s("test.key") + struct.pack("<I", 4) + struct.pack("<I", 42)
    data += b"\0" * (64 - len(data))
    p = _write(tmp_path, data)
    assert gguf_metadata(p, "test.key") == "42"
    with pytest.raises(GpuError) as e:
        gguf_metadata(p, "absent.key")
    assert e.value.kind == "WeightNotFound"
    # metadata_value_type_conversions (:274-306) through the configuration reader: a u64 that does not fit u32 and a
    # negative i32 are not usable as u32 (the default stays), f64 narrows to f32
    emb = np.zeros((4, 128), np.float32).tobytes()
    q = np.zeros(4 * 18, np.uint8).tobytes()
    md = [("qwen3.block_count", "u64", 2**64 - 1), ("qwen3.attention.head_count", "i32", -1),
          ("qwen3.embedding_length", "u64", 128), ("qwen3.rope.freq_base", "f64", 2.718281828459045)]
    ts = [("token_embd.weight", [128, 4], GGUF_F32, emb), ("blk.0.attn_q.weight", [128, 4], GGUF_Q1, q)]
    info = gguf_info(_write(tmp_path, gguf_bytes(md, ts), "conv.gguf"))
    assert (info["n_layers"], info["nq"], info["h"]) == (36, 32, 128) and info["rope_theta"] == np.float32(2.718281828459045)
    # metadata_duplicate_keys_last_wins (:329-336), metadata_bool_entry, metadata_array_u32 (:355-371)
    data = _hdr(0x46554747, 3, 0, 4) + _s("k") + struct.pack("<II", 4, 1) + _s("k") + struct.pack("<II", 4, 2)
    data += _s("flag") + struct.pack("<I", 7) + b"\x01"
    data += _s("arr") + struct.pack("<I", 9) + struct.pack("<I", 4) + struct.pack("<Q", 3) + struct.pack("<III", 10, 20, 30)
    p = _write(tmp_path, data + b"\0" * 64, "dup.gguf")
    assert gguf_metadata(p, "k") == "2" and gguf_metadata(p, "flag") == "true" and gguf_metadata(p, "arr") == "[3 x type 4]"


def test_data_section_alignment_and_tensor_offsets(tmp_path):
    # gguf_file_parse_minimal_valid (:491-503): header only -> the data section starts at 32; align_offset table (:465-484)
    for name_len, align, want in ((1, 32, None), (7, 32, None), (8, 32, None), (9, 64, None), (40, 1, None)):
        name = "t" * name_len
        md = [] if align == 32 else [("general.alignment", "u32", align)]
        head = _hdr(0x46554747, 3, 1, len(md))
        for k, _, v in md:
            head += _s(k) + struct.pack("<II", 4, v)
        head += _tinfo(name, [128, 2], 41, 96 if align != 1 else 5)
        start = (len(head) + align - 1) & ~(align - 1)          # the reference's formula
        off = 96 if align != 1 else 5
        payload = bytes(range(36))
        data = head + b"\0" * (start - len(head)) + b"\xEE" * off + payload
        t = gguf_tensor(_write(tmp_path, data, f"a{name_len}.gguf"), name)
        assert t == {"type": 41, "shape": [128, 2], "n_dims": 2, "file_offset": start + off, "bytes": 36}
        assert data[t["file_offset"]:t["file_offset"] + t["bytes"]] == payload
    with pytest.raises(GpuError) as e:                           # tensor_store_missing_tensor (:405-411)
        gguf_tensor(_write(tmp_path, _hdr(0x46554747, 3, 0, 0) + b"\0" * 8, "none.gguf"), "nope")
    assert e.value.kind == "WeightNotFound"
    # tensor_info_zero_dimensions / single_dimension / type sizes (types.rs block_bytes): F32 4, F16 2, 41 18, 42 34 per unit
    head = _hdr(0x46554747, 3, 4, 0) + _tinfo("s", [], 0, 0) + _tinfo("v", [5], 1, 32) + _tinfo("m", [256, 3], 42, 64) + \
        _tinfo("x", [32, 2], 2, 0)
    p = _write(tmp_path, head + b"\0" * 1024, "dims.gguf")
    assert gguf_tensor(p, "s")["bytes"] == 4 and gguf_tensor(p, "s")["n_dims"] == 0
    assert gguf_tensor(p, "v")["bytes"] == 10 and gguf_tensor(p, "m")["bytes"] == 6 * 34
    assert gguf_tensor(p, "x")["bytes"] == 0 and gguf_tensor(p, "x")["type"] == 2          # Q4_0: listed, not read


def test_loader_rejects_an_absurd_block_count_before_allocating(tmp_path):
    # a header that claims 2^32 - 1 layers must be refused by the loader itself (no GPU is touched, nothing is
    # allocated for it), and so must a count the file's tensor directory cannot cover
    import ctypes as C
    from oxibonsai_amd import _lib
    from oxibonsai_amd.model import GgufInfo
    emb = np.zeros((4, 128), np.float32).tobytes()
    q = np.zeros(4 * 18, np.uint8).tobytes()
    ts = [("token_embd.weight", [128, 4], GGUF_F32, emb), ("blk.0.attn_q.weight", [128, 4], GGUF_Q1, q)]
    for count in (0xFFFFFFFF, 4097, 1, 0):
        md = [("qwen3.block_count", "u32", count), ("qwen3.embedding_length", "u32", 128), ("qwen3.attention.head_count", "u32", 1)]
        p = _write(tmp_path, gguf_bytes(md, ts), f"layers{count}.gguf")
        assert gguf_info(p)["n_layers"] == count          # the directory reader reports what the file says
        mid, eid, info = C.c_uint64(0), C.c_uint64(0), GgufInfo()
        rc = _lib.lib().oxb_hip_load_gguf(p.encode(), 0, 1, C.byref(mid), C.byref(eid), C.byref(info))
        assert rc == 5 and "block_count" in _lib.last_error(), (count, _lib.last_error())
        assert info.lm_head_rows == 4                      # no output.weight: falls back to the embedding's rows
