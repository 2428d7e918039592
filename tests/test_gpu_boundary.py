"""The entry points shaped like the reference's own, through the C ABI on the GPU.

  upload_weights_raw(bytes) / upload_weights_ternary(blocks) carry no shape (gpu_backend/mod.rs:445, 472): the first
  cached call names it (gemv_q1_g128_cached(handle, input, n_rows, k), :457) and the device repacks the bytes;
  try_cuda_full_forward (gpu_backend/cuda_full_layer/encode_q1.rs:813) returns the normed hidden state and receives
  the RoPE rows of its position from the caller (rope_cos / rope_sin)."""
import ctypes as C

import numpy as np
import pytest

from helpers import Q1, TQ2
from kernel_model import gemv as model_gemv
from oracle import oracle
from oxibonsai_amd import GpuError, _lib, repack, synth
from oxibonsai_amd.model import HipModel

pytestmark = pytest.mark.gpu

SHAPES = [(16, 128), (37, 640), (512, 1024), (1000, 4096 + 128), (96, 12800)]


def _upload(backend, fmt, a, shape=(None, None), handle_id=0):
    up = backend.upload_weights_raw if fmt == Q1 else backend.upload_weights_ternary
    return up(a, *shape, handle_id=handle_id)


def _info(h):
    fmt, nr, k, nb = C.c_int(0), C.c_uint32(0), C.c_uint32(0), C.c_size_t(0)
    assert _lib.lib().oxb_hip_weight_info(int(h), C.byref(fmt), C.byref(nr), C.byref(k), C.byref(nb)) == 0
    return fmt.value, nr.value, k.value, nb.value


@pytest.mark.parametrize("fmt", [Q1, TQ2])
@pytest.mark.parametrize("shape", SHAPES)
def test_upload_by_bytes_takes_its_shape_from_the_first_call(backend, fmt, shape):
    """The bytes alone are uploaded; the cached GEMV names (n_rows, k).  What the device then holds decodes to the
    oracle's dequantisation bit for bit (every code and scale went to its place, padding rows and blocks included in
    the odd shapes), and the GEMV equals the numpy model of the kernel run on the HOST repacker's sections bit for bit,
    so the device repack and the host repack agree."""
    n, k = shape
    a = synth.make_blocks(fmt, 0xB17E5 + n + k, n, k)
    x = synth.normal_f32(0xB17E6 + k, k)
    h = _upload(backend, fmt, a)
    try:
        assert _info(h) == (fmt, 0, 0, a.size)
        with pytest.raises(GpuError) as e:
            backend.dequant(h)                      # no shape yet: weight_info says 0 x 0, dequant has nothing to size
        gemv = backend.gemv_q1_g128_cached if fmt == Q1 else backend.gemv_tq2_g128_cached
        with pytest.raises(GpuError) as e:
            gemv(h, x, n + 1, k)                    # block count does not fit: refused, and nothing is bound
        assert e.value.kind == "InvalidArgument"
        assert _info(h)[1:3] == (0, 0)
        y = gemv(h, x, n, k)
        assert _info(h)[:3] == (fmt, n, k)
        with pytest.raises(GpuError):
            gemv(h, np.zeros(k * 2, dtype=np.float32), n // 2 if n % 2 == 0 else n, k * 2)   # the shape stays
        w = backend.dequant(h)
        assert np.array_equal(w.reshape(-1).view(np.uint32), oracle.dequant(fmt, a).view(np.uint32))
        codes, scales = repack(fmt, a, n, k)
        if n * k <= 1 << 20:                        # the numpy model walks every block in Python
            assert np.array_equal(y.view(np.uint32), model_gemv(fmt, codes, scales, n, k, x).view(np.uint32))
        hs = _upload(backend, fmt, a, (n, k))
        try:
            assert np.array_equal(y.view(np.uint32), gemv(hs, x, n, k).view(np.uint32))
        finally:
            backend.free_weights(hs)
    finally:
        backend.free_weights(h)


@pytest.mark.parametrize("fmt", [Q1, TQ2])
def test_upload_by_bytes_rejects_partial_blocks(backend, fmt):
    a = synth.make_blocks(fmt, 5, 16, 128)
    with pytest.raises(GpuError) as e:
        _upload(backend, fmt, a[:-1])
    assert e.value.kind == "InvalidArgument"
    with pytest.raises(GpuError):
        _upload(backend, fmt, a[:0])


def test_first_call_may_be_a_gemm(backend):
    n, k, m = 96, 1024, 24
    a = synth.make_blocks(TQ2, 77, n, k)
    x = synth.normal_f32(78, m * k).reshape(m, k)
    h, hs = _upload(backend, TQ2, a), _upload(backend, TQ2, a, (n, k))
    try:
        assert np.array_equal(backend.gemm_cached(h, x, m, n, k), backend.gemm_cached(hs, x, m, n, k))
    finally:
        backend.free_weights(h)
        backend.free_weights(hs)


CFG = dict(fmt=Q1, n_layers=2, h=256, inter=512, nq=4, nkv=2, hd=64, vocab=160, max_seq=64, eps=1e-6, rope_theta=1e6)


@pytest.mark.parametrize("fmt", [Q1, TQ2])
def test_model_over_weights_uploaded_by_bytes(backend, fmt):
    """Every matrix goes up as bytes alone, as the reference's fused paths hand them over (fused_qkv_bytes, gate_bytes,
    ...: gpu_backend/cuda_full_layer/mod.rs:250-268); the model's dimensions bind the shapes.  Logits equal those of a
    model over shaped uploads bit for bit, decode (graph) and prefill."""
    cfg = dict(CFG, fmt=fmt)
    w = synth.make_model(cfg, 0xB0DE + fmt)
    rows = synth.embedding_rows(3, range(12), cfg["h"]) * 50.0
    a, b = HipModel(backend, cfg, w, shaped_uploads=False), HipModel(backend, cfg, w)
    try:
        la, _ = a.prefill(rows[:8])
        lb, _ = b.prefill(rows[:8])
        assert np.array_equal(la, lb)
        for pos in range(8, 12):
            ga, ta = a.forward(rows[pos], pos)
            gb, tb = b.forward(rows[pos], pos)
            assert np.array_equal(ga, gb) and np.array_equal(ta, tb)
        assert a.uses_graph()
    finally:
        a.close()
        b.close()


def test_replacing_a_weight_by_bytes_under_a_live_model(backend):
    """A weight of a model whose decode step is already a captured graph is replaced by a shape-free upload: the next
    step binds the shape before it captures again (inside the capture nothing may allocate)."""
    cfg = CFG
    w, w2 = synth.make_model(cfg, 91), synth.make_model(cfg, 92)
    rows = synth.embedding_rows(7, range(6), cfg["h"]) * 50.0
    gpu = HipModel(backend, cfg, w)
    mixed = dict(w, layers=[w["layers"][0], dict(w["layers"][1], down=w2["layers"][1]["down"])])
    ref = HipModel(backend, cfg, mixed)
    try:
        for pos in range(3):
            gpu.forward(rows[pos], pos)
            ref.forward(rows[pos], pos)
        assert gpu.uses_graph()
        down_id = int(gpu._ids[1].down)
        backend.upload_weights_raw(w2["layers"][1]["down"], handle_id=down_id)
        assert _info(down_id)[1:3] == (0, 0)
        got, _ = gpu.forward(rows[3], 3)
        want, _ = ref.forward(rows[3], 3)
        assert _info(down_id)[1:3] == (cfg["h"], cfg["inter"])
        assert np.array_equal(got, want)            # the last layer's down projection feeds no cache row
        assert gpu.uses_graph()
    finally:
        gpu.close()
        ref.close()


@pytest.mark.parametrize("fmt", [Q1, TQ2])
@pytest.mark.parametrize("batch", [1, 3])
def test_forward_without_lm_head_returns_the_normed_hidden_state(backend, fmt, batch):
    cfg = dict(CFG, fmt=fmt)
    w = synth.make_model(cfg, 0xF0 + fmt)
    gpu = HipModel(backend, cfg, w, batch=batch, lm_head=False, shaped_uploads=False)
    cpus = [oracle.OracleModel(cfg, w, kv_f16=True) for _ in range(batch)]
    try:
        for pos in range(6):
            rows = np.stack([synth.embedding_rows(11 + s, [pos], cfg["h"])[0] * 50.0 for s in range(batch)])
            got = gpu.forward_hidden(rows, pos)
            for s in range(batch):
                _, want = cpus[s].forward(rows[s], pos, want_normed=True, want_logits=False)
                assert np.max(np.abs(got[s] - want)) < 2e-4 * float(np.max(np.abs(want))), (pos, s)
        with pytest.raises(GpuError) as e:
            gpu.forward(rows, 6)                    # no LM head on the device
        assert e.value.kind == "InvalidArgument"
        gpu.prefill(rows[:1], pos_start=6, want_logits=False)     # cache rows only: allowed
    finally:
        gpu.close()


def test_rope_rows_come_from_the_caller(backend):
    """The model is created with a wrong rope_theta; the caller then hands over the rows of the positions it decodes,
    as the reference's entry points receive them.  The result must be that of a model created with the right theta,
    bit for bit (same table values, same kernels)."""
    cfg = CFG
    w = synth.make_model(cfg, 0xA0)
    good = HipModel(backend, cfg, w)
    late = HipModel(backend, dict(cfg, rope_theta=777.0), w)
    half = cfg["hd"] // 2
    # RopeTable::new (crates/oxibonsai-model/src/layers/rope.rs:27-48), all in f32
    i = np.arange(half, dtype=np.float32)
    freq = (np.float32(1.0) / np.power(np.float32(cfg["rope_theta"]), np.float32(2.0) * i / np.float32(cfg["hd"]))).astype(np.float32)
    rows = synth.embedding_rows(5, range(10), cfg["h"]) * 50.0
    try:
        pre = np.arange(6, dtype=np.float32)[:, None] * freq[None, :]
        late.set_rope_rows(0, np.cos(pre.astype(np.float32)), np.sin(pre.astype(np.float32)))
        la, _ = late.prefill(rows[:6])
        lb, _ = good.prefill(rows[:6])
        tol = 1e-5 * float(np.max(np.abs(lb)))      # numpy's cos/sin and libm's may differ in the last bit
        assert np.max(np.abs(la - lb)) <= tol
        for pos in range(6, 10):
            ang = (np.float32(pos) * freq).astype(np.float32)
            late.set_rope_rows(pos, np.cos(ang), np.sin(ang))
            ga, _ = late.forward(rows[pos], pos)
            gb, _ = good.forward(rows[pos], pos)
            assert np.max(np.abs(ga - gb)) <= tol, pos
        # and without the rows the wrong theta shows
        wrong = HipModel(backend, dict(cfg, rope_theta=777.0), w)
        try:
            lw, _ = wrong.prefill(rows[:6])
            assert np.max(np.abs(lw - lb)) > 100 * tol
        finally:
            wrong.close()
        with pytest.raises(GpuError):
            late.set_rope_rows(cfg["max_seq"] - 1, np.zeros((2, half)), np.zeros((2, half)))
    finally:
        good.close()
        late.close()


@pytest.mark.parametrize("fmt", [Q1, TQ2])
def test_lm_head_joins_a_live_model(backend, fmt):
    """try_cuda_full_forward_with_gpu_lm_head continues on the cache try_cuda_full_forward filled
    (gpu_backend/cuda_full_layer/encode_q1.rs:881-900): positions 0..3 run without an LM head, then the head is
    attached and position 4 must give the logits of a model that had it from the start, bit for bit."""
    cfg = dict(CFG, fmt=fmt)
    w = synth.make_model(cfg, 0x1A0 + fmt)
    rows = synth.embedding_rows(21, range(6), cfg["h"]) * 50.0
    a, b = HipModel(backend, cfg, w, lm_head=False), HipModel(backend, cfg, w)
    try:
        for pos in range(4):
            a.forward_hidden(rows[pos], pos)
            b.forward(rows[pos], pos)
        a.set_lm_head(w["final_norm"], w["lm_head"], cfg["vocab"])
        for pos in range(4, 6):
            ga, ta = a.forward(rows[pos], pos)
            gb, tb = b.forward(rows[pos], pos)
            assert np.array_equal(ga, gb) and np.array_equal(ta, tb)
        assert a.uses_graph()
        a.set_lm_head(None, None, 0)
        with pytest.raises(GpuError):
            a.forward(rows[0], 6)
    finally:
        a.close()
        b.close()


@pytest.mark.parametrize("fmt", [Q1, TQ2])
@pytest.mark.parametrize("h", [1024, 640, 13312, 16384])
def test_batch_attn_phase(backend, fmt, h):
    """RMSNorm + fused QKV product in one launch, against the oracle's RMSNorm and GEMV.  Rows longer than 12288 take
    a second, accumulating launch: each applies 1 / rms of the whole row to its own part of the sum."""
    from oxibonsai_amd.model import batch_attn_phase
    qr, kr = 512, 256
    a = synth.make_blocks(fmt, 0xA77 + fmt, qr + 2 * kr, h)
    x = synth.normal_f32(0xA78, h)
    nw = (1.0 + synth.normal_f32(0xA79, h, 0.02)).astype(np.float32)
    hd = _upload(backend, fmt, a)
    try:
        q, k, v = batch_attn_phase(backend, fmt, x, nw, 1e-6, hd, qr, kr, h)
        normed = oracle.rms_norm(x, nw, 1e-6)
        want = oracle.gemv(fmt, a, normed, qr + 2 * kr, h)
        got = np.concatenate([q, k, v])
        assert np.max(np.abs(got - want)) < 2e-5 * float(np.max(np.abs(want)))
    finally:
        backend.free_weights(hd)
