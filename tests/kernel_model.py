"""numpy model of the device GEMV arithmetic (quantiser + int8 MFMA + recombination).

It reads the *resident* sections produced by the library's host repacker and
reproduces, step by step, what quant_x_kernel and gemv_mfma_kernel compute:
int8 operands made by AND-masks, eight balanced base-256 activation digits, the
accumulator start values and the fp32 epilogue.  The CPU test suite holds it to
the oracle, which pins the arithmetic design where no GPU is present."""
from __future__ import annotations

import numpy as np

P = 53
ND = 8


def _digits(v: np.ndarray) -> np.ndarray:
    """int64 array -> balanced signed base-256 digits [..., 8]."""
    bias = np.uint64(0x0080808080808080)
    with np.errstate(over="ignore"):
        t = (v.astype(np.int64).view(np.uint64) + bias) ^ bias
    d = np.stack([(t >> np.uint64(8 * i)) & np.uint64(0xFF) for i in range(ND)], axis=-1).astype(np.int64)
    return np.where(d >= 128, d - 256, d)


def quant_x(fmt: int, x: np.ndarray, nblk_pad: int):
    """Returns (B[blk, m, g, jj, bb, digit] int, cneg[blk, digit] int, xexp int or None)."""
    k = x.size
    nblk = k // 128
    if not np.all(np.isfinite(x)):
        return None, None, None
    mx = float(np.max(np.abs(x))) if k else 0.0
    B = np.zeros((nblk_pad, 2, 4, 4, 4, ND), dtype=np.int64)
    cneg = np.zeros((nblk_pad, ND), dtype=np.int64)
    if mx == 0.0:
        return B, cneg, 0
    _, E = np.frexp(np.float32(mx))
    E = int(E)
    blk, m, g, jj, bb = np.meshgrid(np.arange(nblk), np.arange(2), np.arange(4), np.arange(4), np.arange(4),
                                    indexing="ij")
    if fmt == 0:
        j = 4 * m + jj
        kk = blk * 128 + 32 * g + 8 * bb + j
        r = np.rint(np.ldexp(x[kk].astype(np.float64), P - E - j)).astype(np.int64)
        xi = np.where(j == 7, -2 * r, 2 * r)
        cr, cmul = r, (1 << j)
    else:
        kk = blk * 128 + 32 * g + 16 * m + 4 * bb + jj
        xi = np.rint(np.ldexp(x[kk].astype(np.float64), P - E - 2 * jj)).astype(np.int64)
        cr, cmul = xi, np.where(jj < 3, 1 << (2 * jj), 0)
    B[:nblk] = _digits(xi)
    cneg[:nblk] = -(_digits(cr) * cmul[..., None]).sum(axis=(1, 2, 3, 4))
    return B, cneg, E - P


def gemv(fmt: int, codes_u8: np.ndarray, scales_u8: np.ndarray, n_rows: int, k: int, x: np.ndarray) -> np.ndarray:
    n_tiles, n_sb = (n_rows + 15) // 16, (k + 511) // 512
    nblk_pad = n_sb * 4
    B, cneg, xexp = quant_x(fmt, x.astype(np.float32), nblk_pad)
    if B is None:
        return np.full(n_rows, np.nan, dtype=np.float32)
    unit = 256 if fmt == 0 else 512
    codes = codes_u8.view(np.uint32).reshape(n_tiles, n_sb, unit)
    scales = scales_u8.view(np.float16).reshape(n_tiles, n_sb, 4, 4, 4).astype(np.float32)  # [rg][q][v]
    y = np.zeros(n_rows, dtype=np.float32)
    jjs = np.arange(4)
    for tile in range(n_tiles):
        accf = np.zeros((16, ND), dtype=np.float32)  # [row][digit]
        for sb in range(n_sb):
            for q in range(4):
                blk = sb * 4 + q
                I = np.tile(cneg[blk][None, :], (16, 1))  # [row][digit]
                for m in range(2):
                    for g in range(4):
                        lanes = g * 16 + np.arange(16)
                        if fmt == 0:
                            w = codes[tile, sb, lanes * 4 + q].astype(np.int64)
                            a = w[:, None] & (0x01010101 << (4 * m + jjs))[None, :]
                        else:
                            w = codes[tile, sb, (q >> 1) * 256 + lanes * 4 + (q & 1) * 2 + m].astype(np.int64)
                            a = w[:, None] & (0x03030303 << (2 * jjs))[None, :]
                        ab = np.stack([(a >> (8 * b)) & 0xFF for b in range(4)], axis=-1)  # [row][jj][bb]
                        ab = np.where(ab >= 128, ab - 256, ab)
                        I = I + np.einsum("rjb,jbd->rd", ab, B[blk, m, g])
                d = scales[tile, sb, :, q, :].reshape(16)  # row = 4*rg + v
                accf = (accf + I.astype(np.float32) * d[:, None]).astype(np.float32)
        f = accf
        v = np.zeros(16, dtype=np.float32)
        for dgt in range(ND - 1, -1, -1):
            v = (v.astype(np.float64) * 256.0 + f[:, dgt]).astype(np.float32)  # fmaf: one rounding
        rows = tile * 16 + np.arange(16)
        ok = rows < n_rows
        y[rows[ok]] = np.ldexp(v.astype(np.float32), xexp)[ok]
    return y
