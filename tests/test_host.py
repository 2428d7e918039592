"""Host-side logic of the native-hip library that runs without a GPU: the C ABI surface,
the AoS -> resident repack, argument validation, and the arithmetic model of the device GEMV."""
import ctypes as C
import os
import re

import numpy as np
import pytest

import kernel_model
import oxibonsai_amd as ox
from helpers import Q1, TQ2, block, cross_tier_q1, dense_f64, metal_tq2, simd_parity_tq2
from oracle import oracle
from oxibonsai_amd import _lib, synth

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    declared = set()
    for name in sorted(os.listdir(os.path.join(ROOT, "include"))):          # the boundary and the measurement hooks
        header = open(os.path.join(ROOT, "include", name)).read()
        declared |= set(re.findall(r"\b(oxb_hip_[a-z0-9_]+)\s*\(", header))
    assert len(declared) >= 15
    L = C.CDLL(_lib.LIB_PATH)
    missing = [s for s in sorted(declared) if not hasattr(L, s)]
    assert not missing, missing
    assert declared == set(_lib._SIGNATURES), declared ^ set(_lib._SIGNATURES)


def test_static_library_is_built():
    assert os.path.exists(os.path.join(os.path.dirname(_lib.LIB_PATH), "liboxb_hip.a"))


def test_no_gpu_means_not_available_not_a_fallback():
    L = _lib.lib()
    if L.oxb_hip_device_count() > 0:
        pytest.skip("a GPU is present")
    with pytest.raises(ox.GpuError) as e:
        ox.NativeHipBackend(0)
    assert e.value.kind == "NotAvailable"
    b = block(Q1, 1.0, 0xFF)
    x, y = np.ones(128, np.float32), np.zeros(1, np.float32)
    rc = L.oxb_hip_gemv_q1_g128(b.ctypes.data_as(_lib.u8p), b.size, x.ctypes.data_as(_lib.f32p), 128,
                                y.ctypes.data_as(_lib.f32p), 1, 1, 128)
    assert rc == 1 and "not available" in _lib.last_error().lower()
    assert y[0] == 0.0


@pytest.mark.parametrize("fmt", [Q1, TQ2])
@pytest.mark.parametrize("shape", [(1, 128), (16, 512), (17, 640), (40, 1152), (100, 2048)])
def test_repack_round_trip(fmt, shape):
    n, k = shape
    a = synth.make_blocks(fmt, 100 + n, n, k)
    codes, scales = ox.repack(fmt, a, n, k)
    assert codes.size % 1024 == 0 and scales.size % 128 == 0      # 1 KiB code units, 16-byte aligned sections
    assert np.array_equal(ox.unpack(fmt, codes, scales, n, k), a)


def test_repack_reserved_ternary_code_decodes_to_zero():
    a = block(TQ2, 0.5, 0xFF)  # all 0b11
    codes, scales = ox.repack(TQ2, a, 1, 128)
    back = ox.unpack(TQ2, codes, scales, 1, 128)
    assert np.all(oracle.dequant(TQ2, back) == 0.0) and np.all(oracle.dequant(TQ2, a) == 0.0)
    mixed = block(TQ2, 0.5, 0x9C)
    back = ox.unpack(TQ2, *ox.repack(TQ2, mixed, 1, 128), 1, 128)
    assert np.array_equal(oracle.dequant(TQ2, back), oracle.dequant(TQ2, mixed))


def test_repack_padding_is_zero():
    n, k = 5, 128  # 11 padded rows, 3 padded blocks
    a = synth.make_blocks(Q1, 9, n, k)
    codes, scales = ox.repack(Q1, a, n, k)
    s16 = scales.view(np.uint16).reshape(16, 4)    # [row][q]
    assert np.all(s16[:, 1:] == 0)                 # blocks 1..3 of the superblock do not exist
    assert np.all(s16[5:, :] == 0) and np.all(s16[:5, 0] != 0)
    w = codes.view(np.uint32).reshape(64, 4)
    assert np.all(w[:, 1:] == 0)


def test_repack_argument_validation():
    a = synth.make_blocks(Q1, 1, 4, 256)
    with pytest.raises(ox.GpuError) as e:
        ox.repack(Q1, a, 4, 200)
    assert e.value.kind == "InvalidArgument"
    with pytest.raises(ox.GpuError):
        ox.repack(Q1, a[:-1], 4, 256)
    with pytest.raises(ox.GpuError):
        ox.repack(Q1, a, 0, 256)
    with pytest.raises(ox.GpuError):
        ox.repack(7, a, 4, 256)


# ---- arithmetic model of the device GEMV against the oracle -------------------------------------
@pytest.mark.parametrize("fmt", [Q1, TQ2])
@pytest.mark.parametrize("shape", [(16, 128), (40, 640), (33, 1024)])
def test_device_arithmetic_model_matches_oracle(fmt, shape):
    n, k = shape
    a = synth.make_blocks(fmt, 11 + fmt, n, k)
    x = synth.normal_f32(5, k)
    y = kernel_model.gemv(fmt, *ox.repack(fmt, a, n, k), n, k, x)
    want = dense_f64(fmt, a, n, k) @ x.astype(np.float64)
    yo = oracle.gemv(fmt, a, x, n, k)
    assert np.max(np.abs(y - want)) <= max(np.max(np.abs(yo - want)) * 2, 1e-6)   # no worse than fp32 order effects
    assert np.max(np.abs(y - yo)) < 1e-5


@pytest.mark.parametrize("fmt", [Q1, TQ2])
@pytest.mark.parametrize("shape", [(16, 128), (40, 640), (33, 1024)])
def test_int8_route_model_matches_oracle(fmt, shape):
    """From two activation vectors on the weights take the int8 route; its model stays held to the oracle too."""
    n, k = shape
    a = synth.make_blocks(fmt, 11, n, k)
    x = synth.normal_f32(5, k)
    y = kernel_model.gemv(fmt, *ox.repack(fmt, a, n, k), n, k, x, route="i8")
    want = dense_f64(fmt, a, n, k) @ x.astype(np.float64)
    yo = oracle.gemv(fmt, a, x, n, k)
    assert np.max(np.abs(y - want)) <= max(np.max(np.abs(yo - want)) * 2, 1e-6)
    assert np.max(np.abs(y - yo)) < 1e-5
    y4 = kernel_model.gemv(fmt, *ox.repack(fmt, a, n, k), n, k, x, route="f4")     # the fp4 route of one vector
    assert np.max(np.abs(y - y4)) < 2e-6 * max(1.0, float(np.max(np.abs(y4))))


def test_fp4_route_model_special_inputs():
    """Zero vectors, a NaN, an outlier and exact power-of-two scaling through the model of the fp4 route."""
    a = cross_tier_q1(32, 512)
    rep = ox.repack(Q1, a, 32, 512)
    x = synth.normal_f32(3, 512)
    y = kernel_model.gemv(Q1, *rep, 32, 512, x)
    assert np.all(kernel_model.gemv(Q1, *rep, 32, 512, np.zeros(512, np.float32)) == 0)
    for s in (-100, 66):
        assert np.array_equal(kernel_model.gemv(Q1, *rep, 32, 512, np.ldexp(x, s).astype(np.float32)), np.ldexp(y, s).astype(np.float32))
    xo = x.copy()
    xo[17] = 3000.0
    want = dense_f64(Q1, a, 32, 512) @ xo.astype(np.float64)
    assert np.max(np.abs(kernel_model.gemv(Q1, *rep, 32, 512, xo) - want)) < 1e-6 * np.max(np.abs(want)) + 1e-4
    xo[3] = np.nan
    assert np.all(np.isnan(kernel_model.gemv(Q1, *rep, 32, 512, xo)))


def test_fp4_route_model_tq2_kats_and_special_inputs():
    """The TQ2 variant of the fp4 route (taken by LM-head-sized launches): the reference's closed forms, every field
    position incl. the two's-complement ones, zero and NaN inputs, exact power-of-two scaling."""
    for pat, x, want in [(0xAA, np.ones(128, np.float32), 128.0), (0x00, np.ones(128, np.float32), -128.0),
                         (0x46, np.ones(128, np.float32), 0.0), (0xFF, np.ones(128, np.float32), 0.0),
                         (0x02, np.arange(128, dtype=np.float32), float(sum(range(0, 128, 4)) - sum(k for k in range(128) if k % 4))),
                         (0x80, np.arange(128, dtype=np.float32), float(sum(range(3, 128, 4)) - sum(k for k in range(128) if k % 4 != 3)))]:
        a = block(TQ2, 1.0, pat)
        y = kernel_model.gemv(TQ2, *ox.repack(TQ2, a, 1, 128), 1, 128, x, route="f4")
        assert y[0] == want, (hex(pat), y[0], want)
    a = synth.make_blocks(TQ2, 5, 20, 640)
    rep = ox.repack(TQ2, a, 20, 640)
    x = synth.normal_f32(3, 640)
    y = kernel_model.gemv(TQ2, *rep, 20, 640, x, route="f4")
    want = dense_f64(TQ2, a, 20, 640) @ x.astype(np.float64)
    assert np.max(np.abs(y - want)) < 1e-5
    assert np.all(kernel_model.gemv(TQ2, *rep, 20, 640, np.zeros(640, np.float32), route="f4") == 0)
    for s in (-100, 66):
        assert np.array_equal(kernel_model.gemv(TQ2, *rep, 20, 640, np.ldexp(x, s).astype(np.float32), route="f4"), np.ldexp(y, s).astype(np.float32))
    x[7] = np.nan
    assert np.all(np.isnan(kernel_model.gemv(TQ2, *rep, 20, 640, x, route="f4")))


def test_device_arithmetic_model_reference_kats():
    for fmt, pat, x, want in [
        (Q1, 0xFF, np.arange(128, dtype=np.float32), 8128.0),
        (Q1, 0x00, np.ones(128, np.float32), -128.0),
        (TQ2, 0xAA, np.ones(128, np.float32), 128.0),
        (TQ2, 0x00, np.ones(128, np.float32), -128.0),
        (TQ2, 0x46, np.ones(128, np.float32), 0.0),
        (TQ2, 0xFF, np.ones(128, np.float32), 0.0),
    ]:
        a = block(fmt, 1.0, pat)
        y = kernel_model.gemv(fmt, *ox.repack(fmt, a, 1, 128), 1, 128, x)
        assert abs(y[0] - want) < 1e-3, (fmt, hex(pat), y[0])


def test_device_arithmetic_model_reference_generators_and_outliers():
    a = cross_tier_q1(32, 512)
    x = np.array([(i % 17) * 0.25 - 2.0 for i in range(512)], dtype=np.float32)
    y = kernel_model.gemv(Q1, *ox.repack(Q1, a, 32, 512), 32, 512, x)
    assert np.max(np.abs(y - oracle.gemv(Q1, a, x, 32, 512))) < 1e-2     # outputs are O(1000)
    a, x = simd_parity_tq2(16, 128)
    y = kernel_model.gemv(TQ2, *ox.repack(TQ2, a, 16, 128), 16, 128, x)
    assert np.mean((y - oracle.gemv(TQ2, a, x, 16, 128)) ** 2) < 1e-6
    a = metal_tq2(16, 256)
    # one activation 1000x larger than the rest: the per-vector exponent must not wash out the others
    x = synth.normal_f32(3, 256)
    x[17] = 3000.0
    y = kernel_model.gemv(TQ2, *ox.repack(TQ2, a, 16, 256), 16, 256, x)
    want = dense_f64(TQ2, a, 16, 256) @ x.astype(np.float64)
    assert np.max(np.abs(y - want)) < 1e-3 * 1e-3 * np.max(np.abs(want)) + 1e-4
    assert np.all(kernel_model.gemv(TQ2, *ox.repack(TQ2, a, 16, 256), 16, 256, np.zeros(256, np.float32)) == 0)
    x[3] = np.inf
    assert np.all(np.isnan(kernel_model.gemv(TQ2, *ox.repack(TQ2, a, 16, 256), 16, 256, x)))


def test_ctypes_structs_match_the_header_layout(tmp_path):
    """Size and field offsets of every struct of the C ABI, as a C compiler sees the header, against the ctypes
    mirrors the Python host side passes across the boundary."""
    import shutil
    import subprocess
    from oxibonsai_amd import model as M
    mirrors = {"oxb_layer_ids": M._LayerIds, "oxb_model_desc": M._ModelDesc, "oxb_gguf_info": M.GgufInfo,
               "oxb_sampling": M.Sampling, "oxb_attention_options": M.AttentionOptions, "oxb_kv_pool_info": M.KvPoolInfo}
    cc = shutil.which("gcc") or shutil.which("cc")
    if not cc:
        pytest.skip("no C compiler")
    lines = ['#include <stdio.h>', '#include <stddef.h>', '#include "oxb_hip.h"', 'int main(void) {']
    for cname, cls in mirrors.items():
        lines.append(f'  printf("{cname} %zu\\n", sizeof({cname}));')
        for fname, _ in cls._fields_:
            lines.append(f'  printf("{cname}.{fname} %zu\\n", offsetof({cname}, {fname}));')
    lines += ['  return 0;', '}']
    src = tmp_path / "layout.c"
    src.write_text("\n".join(lines))
    exe = tmp_path / "layout"
    subprocess.run([cc, "-std=c99", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe)], check=True)
    seen = dict(l.split() for l in subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.splitlines())
    for cname, cls in mirrors.items():
        assert int(seen[cname]) == C.sizeof(cls), cname
        for fname, _ in cls._fields_:
            assert int(seen[f"{cname}.{fname}"]) == getattr(cls, fname).offset, (cname, fname)


def _c_decls(text):
    """name -> (parameter count, return type) of every oxb_hip_* prototype in the header."""
    text = re.sub(r"/\*.*?\*/", " ", text, flags=re.S)
    out = {}
    for ret, name, args in re.findall(r"\b(int|void|const char\*)\s+(oxb_hip_[a-z0-9_]+)\s*\(([^)]*)\)\s*;", text):
        args = args.strip()
        out[name] = (0 if args in ("", "void") else args.count(",") + 1, ret)
    return out


def _rust_decls(text):
    text = re.sub(r"//[^\n]*", " ", text)
    out = {}
    for name, args, ret in re.findall(r"pub fn (oxb_hip_[a-z0-9_]+)\s*\(([^)]*)\)\s*(->\s*[^;]+)?;", text):
        args = args.strip().rstrip(",")
        out[name] = (0 if not args else args.count(",") + 1, ret.replace("->", "").strip() if ret else "void")
    return out


def test_rust_overlay_declares_the_header_one_for_one():
    """rust/native_hip/ffi.rs is what a maintainer links against liboxb_hip.a: every prototype of the header must be
    there under the same name with the same number of parameters and the matching return type, and nothing else."""
    c = _c_decls(open(os.path.join(ROOT, "include", "oxb_hip.h")).read())
    r = _rust_decls(open(os.path.join(ROOT, "rust", "native_hip", "ffi.rs")).read())
    assert set(c) == set(r), set(c) ^ set(r)
    ret_map = {"int": "c_int", "void": "void", "const char*": "*const c_char"}
    for name, (n, ret) in c.items():
        assert r[name] == (n, ret_map[ret]), (name, c[name], r[name])


def test_rust_overlay_mirrors_the_reference_signatures():
    """The fused entry points keep the reference's parameter names in the reference's order (read from
    gpu_backend/cuda_full_layer/encode_q1.rs:813-900, encode_ternary.rs:694-774, cuda_prefill/try_apis.rs:42-66,
    cuda_graph/functions.rs:76-145)."""
    src = open(os.path.join(ROOT, "rust", "native_hip", "full_forward.rs")).read() + open(os.path.join(ROOT, "rust", "native_hip", "prefill.rs")).read()

    def params(fn):
        m = re.search(r"pub fn %s\s*\((.*?)\)\s*->" % fn, src, flags=re.S)
        assert m, fn
        return [p.split(":")[0].strip() for p in m.group(1).split(",\n") if p.strip()]

    forward = ["hidden", "layer_params", "rope_cos", "rope_sin", "pos", "nq", "nkv", "head_dim", "heads_per_group", "norm_eps",
               "hidden_size", "intermediate_size", "max_seq_len", "final_norm_bytes", "final_norm_handle"]
    lm = ["lm_head_handle", "lm_head_bytes", "vocab_size"]
    assert params("try_hip_full_forward") == forward
    assert params("try_hip_full_forward_ternary") == forward
    assert params("try_hip_full_forward_with_gpu_lm_head") == forward + lm
    assert params("try_hip_full_forward_ternary_with_gpu_lm_head") == forward + lm
    prefill = ["hidden_batch", "batch_size", "pos_start", "n_layers", "layer_params", "cos_table", "sin_table", "hidden_size",
               "intermediate_size", "nq", "nkv", "head_dim", "heads_per_group", "eps", "max_seq_len", "final_norm_handle",
               "final_norm_bytes", "final_norm_eps", "lm_head_handle", "lm_head_bytes", "lm_head_out_features", "logits_out",
               "greedy_token_id_out"]
    assert params("try_hip_prefill") == prefill
    assert params("try_hip_prefill_ternary") == prefill
    assert params("try_hip_ffn") == ["hidden", "attn_out", "norm_weight", "eps", "attn_proj_handle_id", "attn_proj_bytes",
                                     "gate_up_handle_id", "gate_bytes", "up_bytes", "down_handle_id", "down_bytes", "hidden_size",
                                     "intermediate_size"]
    assert params("try_hip_qkv") == ["input", "output", "weight_handle_id", "q_bytes", "k_bytes", "v_bytes", "n_rows", "k"]


def test_rust_overlay_error_type_fits_the_cuda_call_sites():
    """try_hip_prefill returns HipGraphError where try_cuda_prefill returns CudaGraphError
    (gpu_backend/cuda_prefill/try_apis.rs:318-342): every HIP variant must have its namesake in the reference's enum
    (gpu_backend/cuda_graph/types.rs:25-39, restated here), a conversion must exist for builds with both tiers and
    an alias for builds without the CUDA tier."""
    src = open(os.path.join(ROOT, "rust", "native_hip", "mod.rs")).read()
    body = re.search(r"pub enum HipGraphError \{(.*?)\n\}", src, flags=re.S).group(1)
    variants = set(re.findall(r"^\s{4}([A-Z][A-Za-z]+)", body, flags=re.M))
    cuda = {"DeviceNotFound", "CompilationFailed", "DriverError", "WeightNotFound", "WeightLayoutError", "LockPoisoned"}
    assert variants and variants <= cuda
    conv = re.search(r"impl From<HipGraphError> for super::cuda_graph::CudaGraphError \{(.*?)\n\}", src, flags=re.S).group(1)
    for v in variants:
        assert f"HipGraphError::{v}" in conv and f"C::{v}" in conv, v
    assert "pub type CudaGraphError = HipGraphError;" in src
    assert src.count("impl std::error::Error for HipGraphError") == 1


def test_bench_refuses_more_than_one_gpu():
    """bench.py measures one GPU: --gpus above 1 ends with a message and a non-zero status before anything is loaded."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "one GPU" in r.stderr and r.stdout.strip() == ""
