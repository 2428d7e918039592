"""GPU tests of the steps either side of the fused forward, through the C ABI: GGUF checkpoint -> device model,
token embedding lookup on the device, greedy decode and prefill driven by token ids.

The checkpoint is the reference's own synthetic parity model
(crates/oxibonsai-model/tests/metal_prefill_ternary_parity_tests.rs:79-224) written by tests/helpers.py.  A model
loaded from the file must behave bit for bit like one assembled from the same tensors by hand, and both are held
to the CPU oracle."""
import numpy as np
import pytest

from helpers import GGUF_F16, GGUF_F32, GGUF_Q1, GGUF_TQ2, Q1, TQ2, model_gguf, parity_violations
from oracle import oracle
from oxibonsai_amd import GpuError, synth
from oxibonsai_amd.model import Embedding, HipModel

pytestmark = pytest.mark.gpu

TINY = dict(n_layers=2, h=128, inter=256, nq=4, nkv=2, hd=32, vocab=32, max_seq=512, eps=1e-6, rope_theta=1e4)
SMALL = dict(n_layers=2, h=512, inter=1024, nq=8, nkv=2, hd=64, vocab=300, max_seq=256, eps=1e-6, rope_theta=1e6)


def _table(cfg, emb_type, seed=3):
    """(stored bytes, fp32 rows the reference's loader would produce)."""
    v, h = cfg["vocab"], cfg["h"]
    if emb_type in (GGUF_F32, GGUF_F16):
        rows = (synth.embedding_rows(seed, range(v), h) * 50.0).astype(np.float32)
        if emb_type == GGUF_F16:
            st = rows.astype(np.float16)
            return st, st.astype(np.float32)
        return rows, rows
    fmt = Q1 if emb_type == GGUF_Q1 else TQ2
    blocks = synth.make_blocks(fmt, seed, v, h)
    return blocks, oracle.dequant(fmt, blocks).reshape(v, h)


@pytest.mark.parametrize("emb_type", [GGUF_F32, GGUF_F16, GGUF_Q1, GGUF_TQ2])
def test_embedding_rows_match_the_loader_values(backend, emb_type):
    cfg = dict(SMALL)
    stored, rows = _table(cfg, emb_type)
    e = Embedding(stored, emb_type, cfg["vocab"], cfg["h"])
    try:
        ids = [0, 299, 7, 7, 150, 1]
        assert np.array_equal(e.rows(ids), rows[ids])
        with pytest.raises(GpuError) as err:
            e.rows([5, 300])
        assert err.value.kind == "InvalidArgument" and "out of range" in str(err.value)
    finally:
        e.close()


@pytest.mark.parametrize("fmt,emb_type,opts", [(TQ2, GGUF_F32, dict()), (Q1, GGUF_F16, dict(packed=True, norm_f16=True)),
                                               (TQ2, GGUF_TQ2, dict(alignment=256)), (Q1, GGUF_Q1, dict(version=2))])
def test_loaded_model_equals_hand_assembled_model_and_oracle(backend, tmp_path, fmt, emb_type, opts):
    cfg = dict(TINY, fmt=fmt)
    w = synth.make_model(cfg, 40 + fmt)
    stored, rows = _table(cfg, emb_type)
    path = tmp_path / "m.gguf"
    path.write_bytes(model_gguf(cfg, w, emb_type, stored, **opts))
    ref = HipModel(backend, dict(cfg, max_seq=64), w)
    cpu = oracle.OracleModel(cfg, w, kv_f16=True)
    gpu, emb, info = HipModel.from_gguf(backend, str(path), max_seq=64)
    try:
        assert info["fmt"] == fmt and info["embedding_type"] == emb_type and gpu.cfg["vocab"] == cfg["vocab"]
        tok = 3
        for pos in range(6):
            hidden = emb.rows([tok])[0]
            assert np.array_equal(hidden, rows[tok])
            a, ta = gpu.forward(hidden, pos)
            b, tb = ref.forward(hidden, pos)
            assert np.array_equal(a, b) and ta[0] == tb[0]
            assert parity_violations(a[0], cpu.forward(hidden, pos)) == 0
            tok = int(ta[0])
    finally:
        gpu.close()
        emb.close()
        ref.close()


def test_lm_head_with_fewer_rows_than_the_embedding_table(backend, tmp_path):
    # token_embd.weight and output.weight need not have the same row count: the logits have one entry per LM-head
    # row, the embedding lookup accepts every row of the table
    cfg = dict(TINY, fmt=Q1)
    w = synth.make_model(cfg, 77)
    big = dict(cfg, vocab=48)
    stored, rows = _table(big, GGUF_F16)
    path = tmp_path / "m.gguf"
    path.write_bytes(model_gguf(cfg, w, GGUF_F16, stored, emb_rows=48))
    ref = HipModel(backend, dict(cfg, max_seq=64), w)
    gpu, emb, info = HipModel.from_gguf(backend, str(path), max_seq=64)
    try:
        assert (info["vocab"], info["lm_head_rows"], gpu.cfg["vocab"], emb.vocab) == (48, 32, 32, 48)
        hidden = emb.rows([47])[0]
        assert np.array_equal(hidden, rows[47])
        a, ta = gpu.forward(hidden, 0)
        b, tb = ref.forward(hidden, 0)
        assert a.shape == (1, 32) and np.array_equal(a, b) and ta[0] == tb[0]
        logits, tok = gpu.prefill_tokens(emb, [47, 3, 40], pos_start=1)
        assert logits.shape == (32,) and tok == int(np.argmax(logits))
        assert gpu.generate(emb, [47], [4], 3).max() < 32
    finally:
        gpu.close()
        emb.close()
        ref.close()


@pytest.mark.parametrize("batch", [1, 2, 4])
def test_on_device_greedy_loop_equals_host_driven_loop(backend, tmp_path, batch):
    cfg = dict(SMALL, fmt=TQ2)
    w = synth.make_model(cfg, 9)
    stored, rows = _table(cfg, GGUF_F16)
    path = tmp_path / "m.gguf"
    path.write_bytes(model_gguf(cfg, w, GGUF_F16, stored))
    a, emb, _ = HipModel.from_gguf(backend, str(path), batch=batch)
    b = HipModel(backend, cfg, w, batch=batch)
    try:
        start = np.array([5, 17, 200, 31][:batch], dtype=np.uint32)
        pos0 = np.array([0, 3, 1, 2][:batch], dtype=np.uint32)
        # sequences that start above position 0 need a context: give both models the same one
        for sq in range(batch):
            if pos0[sq]:
                ctx = rows[[11 + i for i in range(pos0[sq])]]
                a.prefill(ctx, seq=sq, want_logits=False)
                b.prefill(ctx, seq=sq, want_logits=False)
        n = 24
        got = a.generate(emb, start, pos0, n)
        toks, want = start.copy(), []
        for i in range(n):
            _, toks = b.forward(rows[toks], pos0 + i, want_logits=False)
            want.append(toks.copy())
        assert np.array_equal(got, np.stack(want))
        assert a.uses_graph()
        # the loop can be continued from where it stopped
        more = a.generate(emb, got[-1], pos0 + n, 4)
        for i in range(4):
            _, toks = b.forward(rows[toks], pos0 + n + i, want_logits=False)
            assert np.array_equal(more[i], toks)
    finally:
        a.close()
        b.close()
        emb.close()


def test_prefill_from_token_ids_equals_prefill_from_rows(backend, tmp_path):
    cfg = dict(SMALL, fmt=Q1)
    w = synth.make_model(cfg, 12)
    stored, rows = _table(cfg, GGUF_Q1)
    path = tmp_path / "m.gguf"
    path.write_bytes(model_gguf(cfg, w, GGUF_Q1, stored))
    gpu, emb, _ = HipModel.from_gguf(backend, str(path))
    try:
        ids = [(13 * i + 5) % cfg["vocab"] for i in range(70)]
        la, ta = gpu.prefill_tokens(emb, ids)
        lb, tb = gpu.prefill(rows[ids])
        assert np.array_equal(la, lb) and ta == tb
        cpu = oracle.OracleModel(cfg, w, kv_f16=True)
        want = None
        for i, t in enumerate(ids):
            want = cpu.forward(rows[t], i, want_logits=i == len(ids) - 1)
        assert parity_violations(la, want, 1e-2) == 0
        nxt = gpu.generate(emb, [ta], [len(ids)], 3)          # decode continues on the cache the prefill wrote
        assert nxt.shape == (3, 1)
    finally:
        gpu.close()
        emb.close()


def test_loader_and_token_entry_point_errors(backend, tmp_path):
    cfg = dict(TINY, fmt=TQ2)
    w = synth.make_model(cfg, 2)
    stored, _ = _table(cfg, GGUF_F32)
    data = model_gguf(cfg, w, GGUF_F32, stored)
    (tmp_path / "cut.gguf").write_bytes(data[:len(data) - 1000])          # tensor data past the end of the file
    with pytest.raises(GpuError) as e:
        HipModel.from_gguf(backend, str(tmp_path / "cut.gguf"))
    assert e.value.kind == "InvalidArgument" and "end of file" in str(e.value)
    (tmp_path / "shape.gguf").write_bytes(model_gguf(cfg, w, GGUF_F32, stored, meta_override={"feed_forward_length": 384}))
    with pytest.raises(GpuError) as e:
        HipModel.from_gguf(backend, str(tmp_path / "shape.gguf"))
    assert e.value.kind == "InvalidArgument" and "has shape [128, 256], expected [128, 384]" in str(e.value)
    mixed = model_gguf(cfg, dict(w, lm_head=synth.make_blocks(Q1, 1, cfg["vocab"], cfg["h"])), GGUF_F32, stored,
                       type_override={"output.weight": GGUF_Q1})
    (tmp_path / "mixed.gguf").write_bytes(mixed)
    with pytest.raises(GpuError) as e:                                   # one format for the whole file
        HipModel.from_gguf(backend, str(tmp_path / "mixed.gguf"))
    assert "output.weight has tensor type 41, expected 42" in str(e.value)
    (tmp_path / "ok.gguf").write_bytes(data)
    gpu, emb, _ = HipModel.from_gguf(backend, str(tmp_path / "ok.gguf"), max_seq=16)
    other = Embedding(np.zeros((4, 256), np.float32), GGUF_F32, 4, 256)
    try:
        for bad in (lambda: gpu.generate(emb, [40], [0], 2),              # token id beyond the vocabulary
                    lambda: gpu.generate(emb, [1], [10], 7),              # runs past the context
                    lambda: gpu.generate(other, [1], [0], 1),             # embedding of another hidden size
                    lambda: gpu.prefill_tokens(emb, [1, 2, 99]),
                    lambda: gpu.prefill_tokens(emb, list(range(17)))):
            with pytest.raises(GpuError) as e:
                bad()
            assert e.value.kind == "InvalidArgument"
        assert gpu.generate(emb, [1], [0], 16).shape == (16, 1)           # exactly fills the context
    finally:
        gpu.close()
        emb.close()
        other.close()
