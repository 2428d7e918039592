"""Runtime behaviour of the native-hip library through the C ABI: calls from several host threads, device memory
given back when handles and models are released (the reference serialises its CUDA graph singleton behind a Mutex,
gpu_backend/cuda_graph/cudagraph_type.rs:18-32; weights live until freed, gpu_backend/mod.rs:445-472)."""
import threading

import numpy as np
import pytest

from helpers import Q1, TQ2
from oracle import oracle
from oxibonsai_amd import synth
from oxibonsai_amd.model import HipModel

pytestmark = pytest.mark.gpu


def test_calls_from_several_threads_are_serialised(backend):
    shapes = [(Q1, 640, 1024), (TQ2, 384, 2048), (Q1, 100, 512), (TQ2, 1000, 256)]
    work = []
    for i, (fmt, n, k) in enumerate(shapes):
        a = synth.make_blocks(fmt, 300 + i, n, k)
        h = backend.upload_weights_raw(a, n, k) if fmt == Q1 else backend.upload_weights_ternary(a, n, k)
        x = synth.normal_f32(400 + i, k)
        call = backend.gemv_q1_g128_cached if fmt == Q1 else backend.gemv_tq2_g128_cached
        work.append((call, h, x, n, k, call(h, x, n, k)))
    errors = []

    def worker(idx):
        call, h, x, n, k, want = work[idx]
        try:
            for _ in range(60):
                got = call(h, x, n, k)
                if not np.array_equal(got, want):
                    errors.append((idx, "result changed"))
                    return
        except Exception as e:   # noqa: BLE001
            errors.append((idx, repr(e)))

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(len(work))]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    for _, h, *_ in work:
        backend.free_weights(h)
    assert not errors, errors


def test_device_memory_returns_when_models_and_weights_go(backend):
    cfg = dict(fmt=TQ2, n_layers=2, h=512, inter=1024, nq=8, nkv=2, hd=64, vocab=1000, max_seq=2048, eps=1e-6, rope_theta=1e6)
    w = synth.make_model(cfg, 5)
    rows = synth.embedding_rows(3, range(40), cfg["h"]) * 50.0

    def cycle():
        m = HipModel(backend, cfg, w, batch=4)
        m.prefill(rows, seq=1, want_logits=False)
        m.forward(np.stack([rows[0]] * 4), [0, 40, 0, 0], want_logits=False)
        m.close()

    cycle()                                  # the library's own grow-only workspaces reach their size here
    backend.synchronize()
    free0, total = backend.memory_info()
    for _ in range(5):
        cycle()
    backend.synchronize()
    free1, _ = backend.memory_info()
    assert total > 0 and abs(free0 - free1) < 8 << 20, (free0, free1)     # within one allocator granule or two


def test_two_models_share_the_device(backend):
    # two resident models with their own caches and graphs, used alternately
    cfgs = [dict(fmt=TQ2, n_layers=2, h=128, inter=256, nq=4, nkv=2, hd=32, vocab=32, max_seq=64, eps=1e-6, rope_theta=1e6),
            dict(fmt=Q1, n_layers=3, h=256, inter=512, nq=4, nkv=4, hd=64, vocab=64, max_seq=64, eps=1e-6, rope_theta=1e4)]
    ws = [synth.make_model(c, 10 + i) for i, c in enumerate(cfgs)]
    gpus = [HipModel(backend, c, w) for c, w in zip(cfgs, ws)]
    cpus = [oracle.OracleModel(c, w, kv_f16=True) for c, w in zip(cfgs, ws)]
    try:
        for pos in range(8):
            for i in ((0, 1) if pos % 2 else (1, 0)):
                r = synth.embedding_rows(20 + i, [pos], cfgs[i]["h"])[0] * 50.0
                got, _ = gpus[i].forward(r, pos)
                want = cpus[i].forward(r, pos)
                assert np.max(np.abs(got[0] - want)) < 1e-3 * max(1.0, float(np.max(np.abs(want)))), (i, pos)
        assert all(g.uses_graph() for g in gpus)
    finally:
        for g in gpus:
            g.close()


def test_replacing_or_freeing_a_weight_of_a_live_model(backend):
    # The captured decode step holds device pointers: after a weight is replaced under its id the next step must
    # compute with the new copy (as a model built from the new weights does), and after it is freed the step must
    # report the missing handle instead of replaying a graph over freed memory.
    import ctypes as C

    from oxibonsai_amd import GpuError, _lib
    cfg = dict(fmt=Q1, n_layers=2, h=128, inter=256, nq=4, nkv=2, hd=32, vocab=32, max_seq=64, eps=1e-6, rope_theta=1e6)
    w = synth.make_model(cfg, 61)
    w2 = synth.make_model(cfg, 62)
    gpu = HipModel(backend, cfg, w)
    rows = synth.embedding_rows(7, range(8), cfg["h"]) * 50.0
    try:
        for pos in range(3):
            gpu.forward(rows[pos], pos)
        assert gpu.uses_graph()
        # replace layer 1's down projection and the final norm vector under their ids
        down_id, norm_id = int(gpu._ids[1].down), int(gpu._vecs[-1])
        backend.upload_weights_raw(w2["layers"][1]["down"], cfg["h"], cfg["inter"], handle_id=down_id)
        nv = np.ascontiguousarray(w2["final_norm"], dtype=np.float32)
        hid = C.c_uint64(norm_id)
        assert _lib.lib().oxb_hip_upload_f32(C.byref(hid), nv.ctypes.data_as(_lib.f32p), nv.size) == 0 and hid.value == norm_id
        mixed = dict(w, final_norm=w2["final_norm"], layers=[w["layers"][0], dict(w["layers"][1], down=w2["layers"][1]["down"])])
        ref = HipModel(backend, cfg, mixed)
        try:
            for pos in range(3):
                ref.forward(rows[pos], pos)
            a, _ = gpu.forward(rows[3], 3)
            b, _ = ref.forward(rows[3], 3)
            # the last layer's down projection and the final norm feed no cache row, so both models hold the same
            # cache for positions 0..2 and must agree bit for bit at position 3
            assert np.array_equal(a, b)
            assert gpu.uses_graph()
        finally:
            ref.close()
        backend.free_weights(down_id)
        gpu._mats.remove(down_id)
        with pytest.raises(GpuError) as e:
            gpu.forward(rows[4], 4)
        assert e.value.kind == "WeightNotFound"
        # the handle comes back: the model works again
        backend.upload_weights_raw(w["layers"][1]["down"], cfg["h"], cfg["inter"], handle_id=down_id)
        gpu._mats.append(down_id)
        got, _ = gpu.forward(rows[4], 4)
        assert np.all(np.isfinite(got))
    finally:
        gpu.close()


def test_graph_replay_on_a_stream_the_caller_set(backend):
    """The token's graph is recorded on the library's own stream and replayed on whichever stream is in use: a caller
    that hands in its own stream gets the replay, and the same logits as on the library's stream."""
    import ctypes as C

    from oxibonsai_amd import _lib
    cfg = dict(fmt=Q1, n_layers=2, h=256, inter=512, nq=4, nkv=2, hd=64, vocab=96, max_seq=32, eps=1e-6, rope_theta=1e6)
    w = synth.make_model(cfg, 910)
    rows = [synth.embedding_rows(911, [i], cfg["h"])[0] * 50.0 for i in range(5)]
    ref = HipModel(backend, cfg, w, batch=1)
    try:
        want = [ref.forward(r, i)[0][0].copy() for i, r in enumerate(rows)]
        assert ref.uses_graph()
    finally:
        ref.close()
    L = _lib.lib()
    hip = C.CDLL("libamdhip64.so.7")      # the runtime the library is linked against, already loaded
    stream = C.c_void_p()
    assert hip.hipStreamCreateWithFlags(C.byref(stream), C.c_uint(1)) == 0 and stream.value    # hipStreamNonBlocking
    assert L.oxb_hip_set_stream(stream) == 0
    try:
        gpu = HipModel(backend, cfg, w, batch=1)
        try:
            for i, r in enumerate(rows):
                got = gpu.forward(r, i)[0][0]
                assert np.array_equal(got, want[i]), i
            assert gpu.uses_graph()
        finally:
            gpu.close()
    finally:
        assert L.oxb_hip_set_stream(None) == 0
        assert hip.hipStreamDestroy(stream) == 0


def test_batched_gemv_captured_cold_into_a_callers_graph(backend):
    """oxb_hip_gemv_dev with eight vectors, captured into the caller's own HIP graph as the first call of its shape
    (no warm-up that could grow a workspace: the pack buffer of the batched route exists from oxb_hip_init on), then
    replayed three times with the inputs changed in between; every replay is held to the eager result."""
    import ctypes as C

    from helpers import DeviceBuffer
    from oxibonsai_amd import _lib
    L, hip = _lib.lib(), DeviceBuffer.hip()
    for f, args in (("hipStreamCreate", [C.POINTER(C.c_void_p)]), ("hipStreamDestroy", [C.c_void_p]),
                    ("hipStreamBeginCapture", [C.c_void_p, C.c_int]), ("hipStreamEndCapture", [C.c_void_p, C.POINTER(C.c_void_p)]),
                    ("hipGraphInstantiate", [C.POINTER(C.c_void_p), C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t]),
                    ("hipGraphLaunch", [C.c_void_p, C.c_void_p]), ("hipStreamSynchronize", [C.c_void_p]),
                    ("hipGraphExecDestroy", [C.c_void_p]), ("hipGraphDestroy", [C.c_void_p])):
        getattr(hip, f).argtypes = args
    n, k, B = 1040, 7168, 8                      # a K no other test uses: nothing of this shape has run before
    a = synth.make_blocks(TQ2, 611, n, k)
    h = backend.upload_weights_ternary(a, n, k)
    xs = [synth.normal_f32(620 + i, B * k).reshape(B, k) for i in range(3)]
    d_x, d_y = DeviceBuffer.from_numpy(xs[0]), DeviceBuffer(B * n * 4)
    stream, graph, gexec = C.c_void_p(0), C.c_void_p(0), C.c_void_p(0)
    assert hip.hipStreamCreate(C.byref(stream)) == 0
    try:
        assert L.oxb_hip_set_stream(stream) == 0
        assert hip.hipStreamBeginCapture(stream, 0) == 0                       # hipStreamCaptureModeGlobal
        rc = L.oxb_hip_gemv_dev(int(h), d_x.ptr, d_y.ptr, n, k, B)
        err = _lib.last_error() if rc else ""
        assert hip.hipStreamEndCapture(stream, C.byref(graph)) == 0
        assert rc == 0, err
        assert hip.hipGraphInstantiate(C.byref(gexec), graph, None, None, 0) == 0
        for x in xs:
            assert hip.hipMemcpy(d_x.ptr, np.ascontiguousarray(x).ctypes.data, x.nbytes, 1) == 0
            d_y.fill(0xFF)
            assert hip.hipGraphLaunch(gexec, stream) == 0
            assert hip.hipStreamSynchronize(stream) == 0
            got = d_y.to_numpy(np.float32, (B, n))
            assert L.oxb_hip_set_stream(None) == 0
            want = backend.gemv_cached_batch(h, x, n, k)                         # eager, on the library's own stream
            assert L.oxb_hip_set_stream(stream) == 0
            assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
            ref = oracle.gemm(TQ2, a, x, B, n, k)
            assert np.max(np.abs(got - ref)) < 1e-5 * np.max(np.abs(ref))
    finally:
        L.oxb_hip_set_stream(None)
        if gexec:
            hip.hipGraphExecDestroy(gexec)
        if graph:
            hip.hipGraphDestroy(graph)
        hip.hipStreamDestroy(stream)
        d_x.free()
        d_y.free()
        backend.free_weights(h)
