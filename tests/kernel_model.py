"""numpy model of the device GEMV arithmetic (quantiser + int8 MFMA + recombination).

It reads the *resident* sections produced by the library's host repacker and
reproduces, step by step, what quant_x_kernel and gemv_mfma_kernel compute:
int8 operands made by AND-masks, eight balanced base-256 activation digits scaled per
exponent group (the K slice of one GEMV wave), the accumulator start values and the fp32 epilogue.  The CPU test suite holds it to
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


def group_sb(n_sb: int) -> int:
    """Superblocks per exponent group = K slice of one GEMV wave (oxb_xq_gsb)."""
    return min(3, max(1, (n_sb + 7) // 8))


def quant_x(fmt: int, x: np.ndarray, nblk_pad: int):
    """Returns (B[blk, m, g, jj, bb, digit] int, cneg[blk, digit] int, xexp[group] int with None for a
    group that holds a NaN or an infinity).  Every exponent group is scaled by its own maximum."""
    k = x.size
    nblk = k // 128
    n_sb = nblk_pad // 4
    gsb = group_sb(n_sb)
    n_groups = (n_sb + gsb - 1) // gsb
    B = np.zeros((nblk_pad, 2, 4, 4, 4, ND), dtype=np.int64)
    cneg = np.zeros((nblk_pad, ND), dtype=np.int64)
    xexp = []
    for gi in range(n_groups):
        b0, b1 = gi * gsb * 4, min((gi + 1) * gsb * 4, nblk)
        xs = x[b0 * 128:b1 * 128]
        if not np.all(np.isfinite(xs)):
            xexp.append(None)
            continue
        mx = float(np.max(np.abs(xs))) if xs.size else 0.0
        if mx == 0.0:
            xexp.append(0)
            continue
        _, E = np.frexp(np.float32(mx))
        E = int(E)
        xexp.append(E - P)
        blk, m, g, jj, bb = np.meshgrid(np.arange(b0, b1), np.arange(2), np.arange(4), np.arange(4), np.arange(4),
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
        B[b0:b1] = _digits(xi)
        cneg[b0:b1] = -(_digits(cr) * cmul[..., None]).sum(axis=(1, 2, 3, 4))
    return B, cneg, xexp


def gemv(fmt: int, codes_u8: np.ndarray, scales_u8: np.ndarray, n_rows: int, k: int, x: np.ndarray) -> np.ndarray:
    n_tiles, n_sb = (n_rows + 15) // 16, (k + 511) // 512
    nblk_pad = n_sb * 4
    gsb = group_sb(n_sb)
    B, cneg, xexp = quant_x(fmt, x.astype(np.float32), nblk_pad)
    if any(e is None for e in xexp):
        return np.full(n_rows, np.nan, dtype=np.float32)
    unit = 256 if fmt == 0 else 512
    codes = codes_u8.view(np.uint32).reshape(n_tiles, n_sb, unit)
    scales = scales_u8.view(np.float16).reshape(n_tiles, n_sb, 4, 4, 4).astype(np.float32)  # [rg][q][v]
    y = np.zeros(n_rows, dtype=np.float32)
    jjs = np.arange(4)
    for tile in range(n_tiles):
        total = np.zeros((16, ND), dtype=np.float32)  # [row][digit], groups added with their exponents
        for gi in range(len(xexp)):
            accf = np.zeros((16, ND), dtype=np.float32)  # one wave's partial sums
            for sb in range(gi * gsb, min((gi + 1) * gsb, n_sb)):
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
            weighted = np.ldexp(accf, xexp[gi] + 8 * np.arange(ND)[None, :]).astype(np.float32)
            total = (total + weighted).astype(np.float32)
        v = np.zeros(16, dtype=np.float32)
        for dgt in range(ND):
            v = (v + total[:, dgt]).astype(np.float32)
        rows = tile * 16 + np.arange(16)
        ok = rows < n_rows
        y[rows[ok]] = v[ok]
    return y
