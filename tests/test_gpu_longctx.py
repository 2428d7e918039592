"""GPU parity of the long-context options of the attention kernels (sliding window with attention sinks, INT8 and
FP8-E4M3 KV rows) against the CPU oracle with the same options, through the C ABI.

The row quantiser is held bit for bit to the oracle on identical inputs (oxb_hip_kv_quantize_rows).  Inside a model
the device's K and V differ from the oracle's in their last bits before quantisation, so a code may land on the
other side of a rounding boundary: cache contents are compared code for code, a difference being accepted only
where the oracle's own pre-rounding value sits on such a boundary, and logits under the reference's gate form
(abs < tol or rel < tol) with tol 1e-3 for decode and 1e-2 for prefill; with a quantised cache the decode tolerance is
2e-3 (INT8: one code step is 1/127 of the row maximum) or 5e-3 (E4M3: one code step is 1/8 of the value itself, and a
few dozen of the ~3e5 cached values of a run land on the other side of a boundary).

Where the projections run as fp16 GEMMs (prefill, decode batches of nine and more) K and V carry 2^-11 of relative noise
before they are quantised, so a few percent of the codes differ from the free-running oracle's and the logits agree only
to within the quantisation noise itself (held to 2e-2 of the largest logit); batches of three to eight, on the fp32-exact
GEMVs, are held the same way: among several sequences some code always lands on the other side of a boundary.  The tight check there runs the oracle over
the device's own cache rows (OracleModel.load_rows + freeze): same rows, so the attention arithmetic is compared at the
ordinary tolerance."""
import numpy as np
import pytest

from helpers import Q1, TQ2, parity_violations
from oracle import oracle
from oxibonsai_amd import GpuError, synth
from oxibonsai_amd.model import KV_F16, KV_FP8_E4M3, KV_I8, HipModel, kv_quantize_rows

pytestmark = pytest.mark.gpu

ORACLE_MODE = {KV_F16: oracle.KV_F16, KV_I8: oracle.KV_I8, KV_FP8_E4M3: oracle.KV_FP8_E4M3}
TINY = dict(n_layers=2, h=128, inter=256, nq=4, nkv=2, hd=32, vocab=32, max_seq=96, eps=1e-6, rope_theta=1e6)
SMALL = dict(n_layers=2, h=512, inter=1024, nq=8, nkv=2, hd=64, vocab=256, max_seq=420, eps=1e-6, rope_theta=1e6)
MID = dict(n_layers=2, h=512, inter=1024, nq=8, nkv=4, hd=128, vocab=256, max_seq=600, eps=1e-6, rope_theta=1e6)
WIDE = dict(n_layers=1, h=256, inter=512, nq=2, nkv=2, hd=256, vocab=64, max_seq=200, eps=1e-6, rope_theta=1e4)


def _rows(seed, n, h):
    return synth.embedding_rows(seed, [(7 * i + 3) % 211 for i in range(n)], h) * 50.0


# ---- the row quantiser, bit for bit ------------------------------------------------------------------------
@pytest.mark.parametrize("mode", [KV_I8, KV_FP8_E4M3])
@pytest.mark.parametrize("n", [32, 64, 128, 256, 100])
def test_row_quantiser_equals_oracle_bit_for_bit(backend, mode, n):
    rng = np.random.default_rng(n + mode)
    rows = [rng.standard_normal(n) * s for s in (1.0, 1e-3, 40.0, 1e-6, 3e4)]
    rows.append(np.zeros(n))                                      # all-zero row: scale = f32::EPSILON, codes 0
    rows.append(np.full(n, -2.5))                                 # every value the (negative) maximum
    top = 127.0 if mode == KV_I8 else 448.0
    ties = (np.arange(n) % 120 + 0.5) * (1.0 if mode == KV_I8 else 2.0 ** -9)   # half-way points of the code grid ...
    ties[0] = top                                                 # ... under a scale of exactly 1
    rows.append(ties * np.where(np.arange(n) % 2, -1.0, 1.0))
    tiny = np.concatenate([[1.0], rng.uniform(-1, 1, n - 1) * 2.0 ** -rng.integers(6, 14, n - 1)])  # E4M3 subnormals and underflow
    rows.append(tiny)
    rows.append(np.concatenate([[3.0e38, -3.0e38], rng.standard_normal(n - 2)]))  # a huge maximum: everything else rounds to 0
    x = np.array(rows, dtype=np.float32)
    codes, scales = kv_quantize_rows(mode, x)
    for r in range(x.shape[0]):
        wc, ws = oracle.kv_quantize_row(ORACLE_MODE[mode], x[r])
        assert scales[r] == ws, (r, scales[r], ws)
        assert np.array_equal(codes[r], wc), (r, np.nonzero(codes[r] != wc)[0][:5])


@pytest.mark.parametrize("mode", [KV_I8, KV_FP8_E4M3])
def test_every_code_widens_to_the_oracles_value(backend, mode):
    """All 256 code bytes, in each of the four byte positions of a dword and under several row scales, through the
    widening the attention kernels use (oxb_hip_kv_dequantize_rows): code * scale must be the oracle's
    dequantize_row bit for bit (E4M3: subnormal codes, both zeros, +-448; the two NaN codes must come out NaN)."""
    from oxibonsai_amd.model import kv_dequantize_rows
    base = np.arange(256, dtype=np.uint8)
    codes = np.stack([np.roll(base, r) for r in range(4)] + [base[::-1].copy()])          # every byte in every position
    scales = np.array([1.0, 0.37, 2.0 ** -20, 117.5, 1.1920929e-07], dtype=np.float32)
    got = kv_dequantize_rows(mode, codes, scales)
    for r in range(codes.shape[0]):
        want = oracle.kv_dequantize_row(ORACLE_MODE[mode], codes[r], scales[r])
        nan = np.isnan(want)
        assert np.array_equal(np.isnan(got[r]), nan), r
        assert np.array_equal(got[r][~nan].view(np.uint32), want[~nan].view(np.uint32)), (r, np.nonzero(got[r][~nan] != want[~nan])[0][:5])
    assert mode == KV_I8 or np.count_nonzero(np.isnan(got[0])) == 2
    with pytest.raises(GpuError):
        kv_dequantize_rows(mode, np.zeros((1, 30), dtype=np.uint8), np.ones(1, dtype=np.float32))     # rows of whole dwords


def test_row_quantiser_rejects_bad_arguments(backend):
    with pytest.raises(GpuError):
        kv_quantize_rows(KV_F16, np.zeros((2, 32), dtype=np.float32))     # fp16 rows have no codes
    with pytest.raises(GpuError):
        kv_quantize_rows(7, np.zeros((2, 32), dtype=np.float32))
    codes, scales = kv_quantize_rows(KV_I8, np.zeros((0, 32), dtype=np.float32))
    assert codes.shape == (0, 32) and scales.shape == (0,)


# ---- decode --------------------------------------------------------------------------------------------------
def _compare_cache(gpu, cpu, cfg, mode, n_pos):
    """Device cache rows against the oracle's: codes equal unless the oracle's value sits on a rounding boundary."""
    k, v, kc, vc, ks, vs = cpu.cache()
    flips = total = 0
    for L in range(cfg["n_layers"]):
        for hh in range(cfg["nkv"]):
            gk, gv, gks, gvs = gpu.read_kv(L, hh, 0, n_pos)
            if mode == KV_F16:
                # Both sides round an fp32 value to fp16.  In layer 0 the two fp32 values differ only by the summation
                # order of the QKV projection (1e-6 of the row scale): the stored rows are equal or one fp16 step apart.
                # From layer 1 on the inputs themselves differ: every one-step flip in the cache of the layer below moves
                # that layer's attention output, hence this layer's K and V, by up to 1e-3 (rows of O(1) values).
                for got, want in ((gk.astype(np.float32), k[L, hh, :n_pos]), (gv.astype(np.float32), v[L, hh, :n_pos])):
                    step = np.ldexp(1.0, np.floor(np.log2(np.maximum(np.abs(want), 2.0 ** -14))).astype(int) - 10)
                    if L == 0:
                        assert np.all(np.abs(got - want) <= step + 2e-5), float(np.max(np.abs(got - want) - step))
                    else:
                        assert np.allclose(got, want, rtol=2e-3, atol=1e-3)
                assert np.all(gks == 1.0) and np.all(gvs == 1.0)
                continue
            for got_c, got_s, want_c, want_s in ((gk, gks, kc[L, hh, :n_pos], ks[L, hh, :n_pos]),
                                                 (gv, gvs, vc[L, hh, :n_pos], vs[L, hh, :n_pos])):
                assert np.allclose(got_s, want_s, rtol=1e-4)     # the rows differ in their last bits (GEMV summation order)
                diff = got_c != want_c
                total += diff.size
                flips += int(diff.sum())
                if mode == KV_I8:     # a differing code is a neighbour (the value sat within rounding noise of .5)
                    assert np.all(np.abs(got_c.view(np.int8).astype(int) - want_c.view(np.int8).astype(int))[diff] <= 1)
                else:
                    # neighbours on the E4M3 grid; values tiny against the row maximum (V: the GEMV's own 1e-5 of the
                    # output scale is several subnormal steps there) may sit a few steps apart
                    d = np.abs(oracle.fp8_decode(got_c[diff]) - oracle.fp8_decode(want_c[diff]))
                    assert np.all(d <= np.abs(oracle.fp8_decode(want_c[diff])) * 0.13 + 2.0 ** -7)
    assert flips <= max(4, total // 500), (flips, total)


def _dequantised(mode, rows, scales):
    """Device cache rows as attention reads them: fp16 widened, or code * scale in f32 (kv_cache_quant.rs:69-71, 545-556)."""
    if mode == KV_F16:
        return rows.astype(np.float32)
    vals = rows.view(np.int8).astype(np.float32) if mode == KV_I8 else oracle.fp8_decode(rows).reshape(rows.shape)
    return vals * scales[:, None].astype(np.float32)


def _oracle_on_device_cache(gpu, cfg, w, mode, window, sinks, n_pos, seq=0):
    """An oracle whose cache holds the device's own rows 0 .. n_pos - 1, frozen."""
    cpu = oracle.OracleModel(cfg, w, kv_mode=ORACLE_MODE[mode], window=window, sinks=sinks)
    for L in range(cfg["n_layers"]):
        for hh in range(cfg["nkv"]):
            gk, gv, gks, gvs = gpu.read_kv(L, hh, 0, n_pos, seq=seq)
            cpu.load_rows(L, hh, 0, _dequantised(mode, gk, gks), _dequantised(mode, gv, gvs))
    cpu.freeze()
    return cpu


def _decode_parity(backend, cfg, fmt, mode, window, sinks, steps, seed, batch=1, tol=None, check_every=1):
    cfg = dict(cfg, fmt=fmt)
    w = synth.make_model(cfg, seed)
    tol = tol or {KV_F16: 1e-3, KV_I8: 2e-3, KV_FP8_E4M3: 5e-3}[mode]
    gemm_path = batch >= 3          # held like a batch on the fp16 GEMM route (nine sequences and more): with several
                                    # sequences some quantised code always lands on the other side of a rounding boundary
    if gemm_path:
        tol = 1e-2
    cpus = [oracle.OracleModel(cfg, w, kv_mode=ORACLE_MODE[mode], window=window, sinks=sinks) for _ in range(batch)]
    gpu = HipModel(backend, cfg, w, batch=batch)
    try:
        gpu.set_attention(mode, window, sinks)
        o = gpu.attention()
        assert (o.kv_dtype, o.window_size, o.sink_tokens) == (mode, window, sinks)
        for pos in range(steps):
            hidden = np.stack([synth.embedding_rows(seed + b, [(pos * 5 + b) % 97], cfg["h"])[0] * 50.0 for b in range(batch)])
            check = pos % check_every == 0 or pos == steps - 1
            got, _ = gpu.forward(hidden, [pos] * batch, want_logits=check)
            for b in range(batch):
                want = cpus[b].forward(hidden[b], pos, want_logits=check)
                if check and gemm_path and mode != KV_F16:
                    assert np.max(np.abs(got[b] - want)) < 2e-2 * np.max(np.abs(want)), (pos, b)
                elif check:
                    assert parity_violations(got[b], want, tol) == 0, \
                        f"pos {pos} seq {b}: max abs {np.max(np.abs(got[b] - want)):.3e} of {np.max(np.abs(want)):.3e}"
        if gemm_path:               # the last step once more, by an oracle that reads the device's own cache rows
            for b in range(batch):
                want = _oracle_on_device_cache(gpu, cfg, w, mode, window, sinks, steps, seq=b).forward(hidden[b], steps - 1)
                assert parity_violations(got[b], want, tol) == 0, f"seq {b}: max abs {np.max(np.abs(got[b] - want)):.3e}"
        else:
            _compare_cache(gpu, cpus[0], cfg, mode, steps)
        return gpu.uses_graph()
    finally:
        gpu.close()


@pytest.mark.parametrize("mode", [KV_I8, KV_FP8_E4M3])
@pytest.mark.parametrize("cfg,fmt,steps", [(TINY, TQ2, 70), (SMALL, Q1, 300), (MID, Q1, 140), (WIDE, TQ2, 50)])
def test_decode_with_quantised_cache(backend, mode, cfg, fmt, steps):
    assert _decode_parity(backend, cfg, fmt, mode, 0, 0, steps, seed=31 + mode, check_every=7)


@pytest.mark.parametrize("window,sinks", [(16, 4), (5, 0), (3, 7), (1, 0), (130, 2), (400, 4), (128, 128)])
def test_decode_with_sliding_window(backend, window, sinks):
    # 300 positions: the window slides over chunk boundaries (128) and, for the small ones, out of the first chunk
    _decode_parity(backend, SMALL, Q1, KV_F16, window, sinks, 300, seed=41, check_every=11)


@pytest.mark.parametrize("mode", [KV_I8, KV_FP8_E4M3])
def test_decode_with_window_and_quantised_cache(backend, mode):
    _decode_parity(backend, MID, TQ2, mode, 100, 3, 400, seed=51, check_every=13)


@pytest.mark.parametrize("batch", [2, 4])
def test_batched_decode_with_options(backend, batch):
    _decode_parity(backend, SMALL, Q1, KV_I8, 40, 2, 150, seed=61, batch=batch, check_every=9)


# four q heads of 128 per kv head: with five to eight sequences the attention kernel's merging workgroups also quantise
# their output for the O projection (one 512-value superblock each)
PACKS_FOR_O = dict(n_layers=2, h=256, inter=384, nq=8, nkv=2, hd=128, vocab=128, max_seq=256, eps=1e-6, rope_theta=1e6)


@pytest.mark.parametrize("mode,window,sinks", [(KV_I8, 0, 0), (KV_F16, 40, 2), (KV_FP8_E4M3, 100, 3)])
def test_batched_decode_with_options_where_attention_packs_for_o(backend, mode, window, sinks):
    """Six sequences past the first chunk boundary with a quantised cache and / or a window: the option variants of the
    attention kernel share the merge that leaves the O projection its operands."""
    assert _decode_parity(backend, PACKS_FOR_O, Q1, mode, window, sinks, 140, seed=91, batch=6, check_every=9)


def test_sequences_at_different_positions_with_a_window(backend):
    """Two sequences of one batch, one far ahead of the other: every sequence masks by its own position."""
    cfg = dict(SMALL, fmt=Q1)
    w = synth.make_model(cfg, 71)
    window, sinks = 24, 2
    cpus = [oracle.OracleModel(cfg, w, kv_mode=oracle.KV_I8, window=window, sinks=sinks) for _ in range(2)]
    gpu = HipModel(backend, cfg, w, batch=2)
    try:
        gpu.set_attention(KV_I8, window, sinks)
        lead = 170
        filler = _rows(3, 1, cfg["h"])[0]
        for pos in range(lead):                          # sequence 1 runs ahead on its own (sequence 0 idles at 0)
            h1 = synth.embedding_rows(8, [pos % 50], cfg["h"])[0] * 50.0
            cpus[1].forward(h1, pos, want_logits=False)
            gpu.forward(np.stack([filler, h1]), [0, pos], want_logits=False)
        for pos in range(60):
            h0 = synth.embedding_rows(9, [pos % 31], cfg["h"])[0] * 50.0
            h1 = synth.embedding_rows(8, [(pos + 3) % 50], cfg["h"])[0] * 50.0
            got, _ = gpu.forward(np.stack([h0, h1]), [pos, lead + pos])
            assert parity_violations(got[0], cpus[0].forward(h0, pos), 2e-3) == 0, pos
            assert parity_violations(got[1], cpus[1].forward(h1, lead + pos), 2e-3) == 0, pos
    finally:
        gpu.close()


def test_options_can_change_between_runs(backend):
    """fp16 -> INT8 (new cache, start again) -> a window on the same cache -> back to fp16; every run equals its oracle."""
    cfg = dict(TINY, fmt=Q1)
    w = synth.make_model(cfg, 81)
    gpu = HipModel(backend, cfg, w, batch=1)
    try:
        for mode, window, sinks in ((KV_F16, 0, 0), (KV_I8, 0, 0), (KV_I8, 6, 1), (KV_F16, 9, 2), (KV_FP8_E4M3, 0, 0), (KV_F16, 0, 0)):
            gpu.set_attention(mode, window, sinks)
            cpu = oracle.OracleModel(cfg, w, kv_mode=ORACLE_MODE[mode], window=window, sinks=sinks)
            for pos in range(20):
                hidden = synth.embedding_rows(4, [pos], cfg["h"])[0] * 50.0
                got, _ = gpu.forward(hidden, pos)
                assert parity_violations(got[0], cpu.forward(hidden, pos), 5e-3 if mode == KV_FP8_E4M3 else 2e-3) == 0, (mode, window, pos)
        with pytest.raises(GpuError):
            gpu.set_attention(9, 0, 0)
        with pytest.raises(GpuError):
            gpu.read_kv(0, 0, cfg["max_seq"] - 1, 2)
        with pytest.raises(GpuError):
            gpu.read_kv(cfg["n_layers"], 0, 0, 1)
    finally:
        gpu.close()


# ---- prefill ---------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("mode,window,sinks", [(KV_I8, 0, 0), (KV_FP8_E4M3, 0, 0), (KV_F16, 40, 4), (KV_F16, 33, 0),
                                               (KV_I8, 70, 2), (KV_F16, 3, 9)])
@pytest.mark.parametrize("cfg,fmt,n", [(TINY, TQ2, 50), (SMALL, Q1, 200), (MID, Q1, 150), (WIDE, TQ2, 70)])
def test_prefill_with_options_matches_sequential_oracle(backend, mode, window, sinks, cfg, fmt, n):
    cfg = dict(cfg, fmt=fmt)
    w = synth.make_model(cfg, 200 + n)
    cpu = oracle.OracleModel(cfg, w, kv_mode=ORACLE_MODE[mode], window=window, sinks=sinks)
    gpu = HipModel(backend, cfg, w, batch=1)
    dec_tol = {KV_F16: 1e-2, KV_I8: 1e-2, KV_FP8_E4M3: 1e-2}[mode]

    def loose(got, want):           # against the free-running oracle
        if mode == KV_F16:
            assert parity_violations(got, want, 1e-2) == 0, f"max abs {np.max(np.abs(got - want)):.3e}"
        else:
            assert np.max(np.abs(got - want)) < 2e-2 * np.max(np.abs(want)), f"max abs {np.max(np.abs(got - want)):.3e}"
    try:
        gpu.set_attention(mode, window, sinks)
        rows = _rows(5, n, cfg["h"])
        got, tok = gpu.prefill(rows)
        want = None
        for i, r in enumerate(rows):
            want = cpu.forward(r, i, want_logits=i == n - 1)
        loose(got, want)
        assert tok == int(np.argmax(got))
        # the last token once more, by an oracle that reads the rows the prefill stored
        held = _oracle_on_device_cache(gpu, cfg, w, mode, window, sinks, n)
        want = held.forward(rows[-1], n - 1)
        assert parity_violations(got, want, 1e-2) == 0, f"max abs {np.max(np.abs(got - want)):.3e}"
        held.freeze(False)
        for step in range(3):                            # decode continues on the cache the prefill wrote
            r = _rows(6 + step, 1, cfg["h"])[0]
            g, _ = gpu.forward(r, n + step)
            loose(g[0], cpu.forward(r, n + step))
            assert parity_violations(g[0], held.forward(r, n + step), dec_tol) == 0, step
        # a second chunk of the prompt appended by another prefill call
        more = _rows(11, 40, cfg["h"])
        if n + 3 + len(more) <= cfg["max_seq"]:
            got2, _ = gpu.prefill(more, pos_start=n + 3)
            for i, r in enumerate(more):
                want = cpu.forward(r, n + 3 + i, want_logits=i == len(more) - 1)
            loose(got2, want)
            held = _oracle_on_device_cache(gpu, cfg, w, mode, window, sinks, n + 3 + len(more))
            assert parity_violations(got2, held.forward(more[-1], n + 3 + len(more) - 1), 1e-2) == 0
    finally:
        gpu.close()


# ---- paged cache -----------------------------------------------------------------------------------------------
# Paging moves rows, it does not change arithmetic: the kernels read the same keys in the same order, so a paged run
# must reproduce the contiguous run bit for bit (which the tests above hold to the oracle), however the pages of the
# sequences interleave in the pool.
def _interleaved_decode(gpu, cfg, steps, seed):
    """Two sequences advancing at different speeds (sequence 1 moves every step, sequence 0 every third), so that
    their pages alternate irregularly in the pool; returns every step's logits."""
    out = []
    p0 = 0
    for i in range(steps):
        hidden = np.stack([synth.embedding_rows(seed + b, [(i * 5 + b) % 97], cfg["h"])[0] * 50.0 for b in (0, 1)])
        got, tok = gpu.forward(hidden, [p0, i])
        out.append((got.copy(), tok.copy()))
        if i % 3 == 2:
            p0 += 1
    return out


@pytest.mark.parametrize("mode,window,sinks", [(KV_F16, 0, 0), (KV_I8, 0, 0), (KV_FP8_E4M3, 20, 2), (KV_F16, 150, 4)])
@pytest.mark.parametrize("page_size", [16, 32, 64, 128])
def test_paged_decode_equals_contiguous_bit_for_bit(backend, mode, window, sinks, page_size):
    cfg = dict(SMALL, fmt=Q1)
    w = synth.make_model(cfg, 91)
    gpu = HipModel(backend, cfg, w, batch=2)
    try:
        steps = 290
        gpu.set_attention(mode, window, sinks)
        want = _interleaved_decode(gpu, cfg, steps, 7)
        n_pages = -(-steps // page_size) + -(-(steps // 3 + 1) // page_size)     # exactly what the two sequences need
        gpu.set_attention(mode, window, sinks, page_size, n_pages)
        o = gpu.attention()
        assert (o.page_size, o.n_pages) == (page_size, n_pages)
        got = _interleaved_decode(gpu, cfg, steps, 7)
        for i, ((gl, gt), (wl, wt)) in enumerate(zip(got, want)):
            assert np.array_equal(gl, wl) and np.array_equal(gt, wt), i
        assert gpu.kv_pool().free_pages == 0
        assert gpu.kv_capacity(1) == -(-steps // page_size) * page_size
    finally:
        gpu.close()


@pytest.mark.parametrize("mode,window,sinks", [(KV_F16, 0, 0), (KV_I8, 60, 3)])
@pytest.mark.parametrize("page_size", [16, 128])
def test_paged_prefill_equals_contiguous_bit_for_bit(backend, mode, window, sinks, page_size):
    cfg = dict(MID, fmt=TQ2)
    w = synth.make_model(cfg, 93)
    gpu = HipModel(backend, cfg, w, batch=2)
    try:
        def run():
            res = []
            gpu.prefill(_rows(2, 37, cfg["h"]), seq=1)                  # the other slot takes pages first
            res.append(gpu.prefill(_rows(5, 150, cfg["h"]), seq=0))
            res.append(gpu.prefill(_rows(3, 61, cfg["h"]), seq=1, pos_start=37))
            res.append(gpu.prefill(_rows(9, 45, cfg["h"]), seq=0, pos_start=150))
            hidden = np.stack([_rows(12, 1, cfg["h"])[0], _rows(13, 1, cfg["h"])[0]])
            res.append(gpu.forward(hidden, [195, 98]))
            rows = [gpu.read_kv(L, hh, 0, 196, seq=0) for L in range(cfg["n_layers"]) for hh in range(cfg["nkv"])]
            return res, rows
        gpu.set_attention(mode, window, sinks)
        want, want_rows = run()
        gpu.set_attention(mode, window, sinks, page_size, 2 * (-(-200 // page_size)))
        got, got_rows = run()
        for (gl, gt), (wl, wt) in zip(got, want):
            assert np.array_equal(gl, wl) and np.array_equal(np.asarray(gt), np.asarray(wt))
        for g, wnt in zip(got_rows, want_rows):
            assert all(np.array_equal(a, b) for a, b in zip(g, wnt))
    finally:
        gpu.close()


def test_page_pool_accounting(backend):
    """The bookkeeping of crates/oxibonsai-model/tests/paged_kv_cache_tests.rs: lazy allocation, capacity in whole
    pages, exhaustion, pages returning to the pool when a sequence is dropped."""
    cfg = dict(TINY, fmt=Q1)
    w = synth.make_model(cfg, 95)
    gpu = HipModel(backend, cfg, w, batch=3)
    cpu = oracle.OracleModel(cfg, w, kv_mode=oracle.KV_F16)
    try:
        info = gpu.kv_pool()
        assert (info.page_size, info.total_pages, info.free_pages) == (0, 0, 0)      # contiguous: no pool
        assert gpu.kv_capacity(0) == cfg["max_seq"]
        gpu.kv_reserve(0, 5)                                                         # a no-op there
        gpu.set_attention(KV_F16, 0, 0, 16, 5)
        info = gpu.kv_pool()
        assert (info.page_size, info.total_pages, info.free_pages) == (16, 5, 5)
        assert [gpu.kv_capacity(s) for s in range(3)] == [0, 0, 0]                   # sequences start without pages
        gpu.kv_reserve(0, 1)
        assert gpu.kv_capacity(0) == 16 and gpu.kv_pool().free_pages == 4
        gpu.kv_reserve(0, 16)                                                        # still one page
        assert gpu.kv_capacity(0) == 16 and gpu.kv_pool().free_pages == 4
        gpu.kv_reserve(0, 17)
        assert gpu.kv_capacity(0) == 32 and gpu.kv_pool().free_pages == 3
        gpu.kv_reserve(1, 48)
        assert gpu.kv_capacity(1) == 48 and gpu.kv_pool().free_pages == 0
        with pytest.raises(GpuError) as e:                                           # block_pool_oom / paged_cache_oom_error
            gpu.kv_reserve(2, 1)
        assert e.value.kind == "OutOfMemory" and "no free KV blocks" in str(e.value)
        with pytest.raises(GpuError):
            gpu.kv_reserve(0, cfg["max_seq"] + 1)
        with pytest.raises(GpuError):
            gpu.kv_release(3)
        # a decode step that needs a page the pool no longer has fails the same way and leaves the model usable
        hidden = np.stack([synth.embedding_rows(1, [t], cfg["h"])[0] * 50.0 for t in (1, 2, 3)])
        with pytest.raises(GpuError) as e:
            gpu.forward(hidden, [0, 0, 0])
        assert e.value.kind == "OutOfMemory"
        gpu.kv_release(1)                                                            # drop_sequence frees its blocks
        assert gpu.kv_pool().free_pages == 3 and gpu.kv_capacity(1) == 0
        for pos in range(20):                                                        # sequence 2 grows into the freed pages
            got, _ = gpu.forward(hidden, [pos, 0, pos])
            want = cpu.forward(hidden[2], pos)
            assert parity_violations(got[2], want) == 0, pos
        assert gpu.kv_capacity(2) == 32 and gpu.kv_capacity(1) == 16      # slot 1 wrote position 0 again: one page
        gpu.reset()                                                                  # every slot's pages go back
        info = gpu.kv_pool()
        assert info.free_pages == info.total_pages == 5
        for bad in (dict(page_size=24, n_pages=4), dict(page_size=16, n_pages=0), dict(page_size=0, n_pages=3), dict(page_size=256, n_pages=2)):
            with pytest.raises(GpuError):
                gpu.set_attention(KV_F16, 0, 0, **bad)
    finally:
        gpu.close()
