"""A foreign-language caller against the STATIC library: tests/c_abi_replay.c (plain C, built by __graft_entry__.build
and linked against liboxb_hip.a) replays what a Rust `native-hip` tier would call - uploads by bytes, cached GEMV,
model over caller-chosen handle ids, prefill and decode with the caller's RoPE rows, a forward without LM head - and
writes every result to a file.  This test regenerates the program's inputs (the same SplitMix64 byte stream) and holds
the results to the CPU oracle."""
import os
import subprocess
import sys

import numpy as np
import pytest

from helpers import Q1, TQ2
from oracle import oracle
from oxibonsai_amd import synth

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
import __graft_entry__ as entry  # noqa: E402

N_LAYERS, H, INTER, NQ, NKV, HD, VOCAB, MAX_SEQ, N_PREFILL, N_DECODE = 2, 256, 512, 4, 2, 64, 160, 32, 5, 3


def stream_bytes(seed: int, n: int) -> np.ndarray:
    return (synth.splitmix64(seed, n) >> np.uint64(56)).astype(np.uint8)


def blocks(fmt: int, seed: int, rows: int, k: int) -> np.ndarray:
    bb, d_at = (18, 0) if fmt == Q1 else (34, 32)
    a = stream_bytes(seed, rows * (k // 128) * bb).reshape(-1, bb)
    a[:, d_at + 1] = 0x20 | (a[:, d_at + 1] & 0x03)
    return a.reshape(-1)


def f32s(seed: int, n: int, offset: float, div: float) -> np.ndarray:
    return (np.float32(offset) + (stream_bytes(seed, n).astype(np.float32) - np.float32(128.0)) / np.float32(div)).astype(np.float32)


def model_weights(fmt: int, seed: int) -> dict:
    qd, kd = NQ * HD, NKV * HD
    layers = []
    for L in range(N_LAYERS):
        s = seed + 100 * L
        qkv = blocks(fmt, s + 1, qd + 2 * kd, H).reshape(qd + 2 * kd, -1)
        gu = blocks(fmt, s + 6, 2 * INTER, H).reshape(2 * INTER, -1)
        layers.append(dict(attn_norm=f32s(s + 0, H, 1.0, 256.0), q_norm=f32s(s + 2, HD, 1.0, 256.0), k_norm=f32s(s + 3, HD, 1.0, 256.0),
                           ffn_norm=f32s(s + 5, H, 1.0, 256.0), q=qkv[:qd].reshape(-1), k=qkv[qd:qd + kd].reshape(-1),
                           v=qkv[qd + kd:].reshape(-1), o=blocks(fmt, s + 4, H, qd), gate=gu[:INTER].reshape(-1),
                           up=gu[INTER:].reshape(-1), down=blocks(fmt, s + 7, H, INTER)))
    return dict(layers=layers, final_norm=f32s(seed + 900, H, 1.0, 256.0), lm_head=blocks(fmt, seed + 901, VOCAB, H))


def test_replay_program_is_built():
    assert os.path.exists(entry.REPLAY_BIN), "build it with: python __graft_entry__.py"


@pytest.mark.gpu
def test_c_caller_over_the_static_library(tmp_path):
    if not os.path.exists(entry.REPLAY_BIN):
        entry.build_c_abi_replay()
    out = tmp_path / "replay.bin"
    r = subprocess.run([entry.REPLAY_BIN, str(out)], capture_output=True, text=True, timeout=300)
    print(r.stdout, r.stderr)
    assert r.returncode == 0, (r.returncode, r.stderr)
    assert "c_abi_replay: ok" in r.stdout
    raw = np.fromfile(out, dtype=np.uint32)
    at = 0

    def take(n, dtype=np.float32):
        nonlocal at
        v = raw[at:at + n].view(dtype)
        at += n
        return v

    # cached GEMV over weights uploaded by bytes (the north star's bound is 1e-3 relative; fp32-exact products here)
    for fmt, seed, n, k in ((Q1, 11, 96, 640), (TQ2, 21, 80, 1152)):
        y = take(n)
        want = oracle.gemv(fmt, blocks(fmt, seed, n, k), f32s(seed + 1, k, 0.0, 64.0), n, k)
        assert np.max(np.abs(y - want)) < 1e-5 * float(np.max(np.abs(want))), fmt
    cfg = dict(n_layers=N_LAYERS, h=H, inter=INTER, nq=NQ, nkv=NKV, hd=HD, vocab=VOCAB, max_seq=MAX_SEQ, eps=1e-6, rope_theta=10000.0)
    for fmt, seed in ((Q1, 3000), (TQ2, 4000)):
        c = dict(cfg, fmt=fmt)
        w = model_weights(fmt, seed)
        rows = f32s(seed + 950, (N_PREFILL + N_DECODE) * H, 0.0, 32.0).reshape(-1, H)
        cpu = oracle.OracleModel(c, w, kv_f16=True)
        for pos in range(N_PREFILL):
            want = cpu.forward(rows[pos], pos)
        logits, token = take(VOCAB), int(take(1, np.uint32)[0])
        tol = 1e-2 * max(1.0, float(np.max(np.abs(want))))            # batched prefill: fp16 activations
        assert np.max(np.abs(logits - want)) < tol, fmt
        assert token == int(np.argmax(logits))
        for step in range(N_DECODE):
            pos = N_PREFILL + step
            want = cpu.forward(rows[pos], pos)
            logits, token = take(VOCAB), int(take(1, np.uint32)[0])
            assert np.max(np.abs(logits - want)) < tol, (fmt, step)
            top2 = np.sort(want)[-2:]
            if top2[1] - top2[0] > 2 * tol:
                assert token == oracle.argmax_first(want), (fmt, step)
        assert int(take(1, np.uint32)[0]) == 1                         # the decode step ran from a captured graph
        normed = take(H)
        _, want = oracle.OracleModel(c, w, kv_f16=True).forward(rows[0], 0, want_normed=True, want_logits=False)
        assert np.max(np.abs(normed - want)) < 2e-4 * float(np.max(np.abs(want))), fmt
    assert at == raw.size
