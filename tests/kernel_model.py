"""numpy model of the device GEMV arithmetic (in-kernel activation quantiser + int8 MFMA + recombination).

It reads the *resident* sections produced by the library's host repacker and reproduces, step by step, what
gemv_kernel computes: int8 weight operands made by AND-masks, four balanced base-256 activation digits scaled per
K slice of a wave, the accumulator start values that cancel the bias of the unsigned code encodings, the joining of
the digit sums, the fp16 block scale, the slice exponent, the waves' partial sums added in wave order.  The CPU test
suite holds it to the oracle, which pins the arithmetic design where no GPU is present; the GPU tests can hold the
kernel to this model bit for bit."""
from __future__ import annotations

import numpy as np

P = {0: 29, 1: 30}          # fixed-point bits below 2^E (Q1 operands hold 2 r)
MAX_SB = 24                  # superblocks of K per launch


def _digits32(v: np.ndarray) -> np.ndarray:
    """int64 values in int32 range -> four balanced signed base-256 digits [..., 4] (the top one takes the rest)."""
    t = ((v.astype(np.int64) + 0x808080) & 0xFFFFFFFF) ^ 0x808080
    d = np.stack([(t >> (8 * i)) & 0xFF for i in range(4)], axis=-1)
    return np.where(d >= 128, d - 256, d)


def _f32(x):
    return np.asarray(x, dtype=np.float32)


def _fma32(a, b, c):
    """fp32 fused multiply-add through float64 (the product of two f32 is exact there)."""
    return _f32(a.astype(np.float64) * b.astype(np.float64) + c.astype(np.float64))


def slice_exponent(xs: np.ndarray):
    """E with 2^E > max |x| over a wave's K slice (None for a slice that holds a NaN or an infinity), and whether
    the slice is all zeros."""
    mxb = int((xs.view(np.uint32) & 0x7FFFFFFF).max())
    if mxb >= 0x7F800000:
        return None, False
    be = mxb >> 23
    return (be if be else 1) - 126, mxb == 0


def quantise_block(fmt: int, xb: np.ndarray, E: int):
    """One 128-activation block at the slice exponent E -> (operand digits [128][4] in k order, start values [4])."""
    k = np.arange(128)
    if fmt == 0:
        js = (k % 8) & 3                            # bit j of its code byte is worth 2^(j & 3): k = 32 g + 8 bb + j
        r = np.rint(np.ldexp(xb.astype(np.float32), (P[0] - E - js).astype(np.int32)).astype(np.float32)).astype(np.int64)
        xi = 2 * r
        csum = int(np.sum(r << js))
    else:
        jj = k % 4                                  # field inside its code byte: k = 32 g + 16 m + 4 bb + jj
        js = 2 * jj
        r = np.rint(np.ldexp(xb.astype(np.float32), (P[1] - E - js).astype(np.int32)).astype(np.float32)).astype(np.int64)
        xi = r
        csum = int(np.sum(np.where(jj < 3, r << js, 0)))
    t = ((-csum + 0x808080) ^ 0x808080)
    c = [((t >> (8 * i)) & 0xFF) for i in range(3)]
    c = [v - 256 if v >= 128 else v for v in c] + [t >> 24]
    return _digits32(xi), np.array(c, dtype=np.int64)


def _weight_bytes(fmt: int, codes, tile: int, sb: int, q: int) -> np.ndarray:
    """Signed int8 operand bytes [16 rows][128 k] of block q of unit (tile, sb), as the AND masks produce them."""
    out = np.zeros((16, 128), dtype=np.int64)
    for g in range(4):
        lanes = g * 16 + np.arange(16)
        if fmt == 0:
            w = codes[tile, sb, lanes * 4 + q].astype(np.int64)
            for i in range(32):                     # bit i of the dword: byte bb = i // 8, position j = i % 8
                out[:, 32 * g + i] = ((w >> i) & 1) << (i % 4)      # high nibbles are masked after a shift by 4
        else:
            for m in range(2):
                w = codes[tile, sb, (q >> 1) * 256 + lanes * 4 + (q & 1) * 2 + m].astype(np.int64)
                for i in range(16):                 # field i: byte bb = i // 4, position jj = i % 4
                    b = ((w >> (2 * i)) & 3) << (2 * (i % 4))
                    out[:, 32 * g + 16 * m + i] = np.where(b >= 128, b - 256, b)
    return out


F4_P = 30                    # fp4 route: x = 2^(E - 30) X with |X| < 2^30
_F4_OPERAND = np.array([0.5, 1.0, 2.0])     # what a set bit reads at position m = 0, 1, 2 of its nibble


def quantise_block_f4(xb: np.ndarray, E: int, fmt: int = 0):
    """fp4 route, one 128-activation block at the slice exponent E -> (digit values [128][16] as the E2M1 numbers
    the A operand holds, sign included; start values [16] of the sixteen digit rows).  Q1: the shift and the sign
    follow the bit position m of the weight in its nibble; TQ2: every weight reads the same."""
    k = np.arange(128)
    m = k & 3                                       # Q1: k = 32 g + 4 i + m: bit m of nibble i of the lane's code dword
    sh = (F4_P - E + (np.array([2, 1, 0, 0])[m] if fmt == 0 else 0 * m)).astype(np.int32)
    mag = np.rint(np.ldexp(np.abs(xb.astype(np.float32)), sh).astype(np.float32)).astype(np.float64)
    mag = np.nan_to_num(mag, nan=0.0).astype(np.uint64)
    neg = np.signbit(xb) ^ ((m == 3) if fmt == 0 else False)    # Q1: the m = 3 operand reads -1 for a set bit
    dig = np.stack([((mag >> np.uint64(2 * j)) & np.uint64(3)).astype(np.float64) * 0.5 for j in range(16)], axis=-1)
    dig = np.where(neg[:, None], -dig, dig)
    if fmt == 0:
        bc = np.where(m < 3, -np.array([0.5, 1.0, 2.0, 0.0])[m], 0.0)
        start = 0.5 * (bc[:, None] * dig).sum(axis=0)
    else:
        start = -dig.sum(axis=0)                    # the digits against a constant -1
    return dig, start


def _weight_operands_f4(codes, tile: int, sb: int, q: int, fmt: int = 0) -> np.ndarray:
    """E2M1 operand values [16 rows][128 k] of block q of unit (tile, sb), as the AND masks produce them (TQ2: times
    the block scale of 2 the instruction applies to that operand: field + 1 -> 0, 1, 2)."""
    out = np.zeros((16, 128), dtype=np.float64)
    for g in range(4):
        lanes = g * 16 + np.arange(16)
        if fmt == 0:
            w = codes[tile, sb, lanes * 4 + q].astype(np.int64)
            for i in range(32):
                b = (w >> i) & 1
                out[:, 32 * g + i] = np.where(b == 1, -1.0, 1.0) if (i & 3) == 3 else b * _F4_OPERAND[i & 3]
        else:
            for m in range(2):
                w = codes[tile, sb, (q >> 1) * 256 + lanes * 4 + (q & 1) * 2 + m].astype(np.int64)
                even = w & 0x33333333
                odd = ((w >> 2) + 0x10101010) & 0x33333333
                for n in range(8):
                    out[:, 32 * g + 16 * m + 2 * n] = (even >> (4 * n)) & 15
                    out[:, 32 * g + 16 * m + 2 * n + 1] = (odd >> (4 * n)) & 15
    return out


def gemv_f4(codes_u8: np.ndarray, scales_u8: np.ndarray, n_rows: int, k: int, x: np.ndarray, fmt: int = 0) -> np.ndarray:
    """gemv_f4_kernel step by step (one activation vector)."""
    n_tiles, n_sb = (n_rows + 15) // 16, (k + 511) // 512
    x = np.asarray(x, dtype=np.float32)
    xp = np.zeros(n_sb * 512, dtype=np.float32)
    xp[:k] = x
    codes = codes_u8.view(np.uint32).reshape(n_tiles, n_sb, 256 if fmt == 0 else 512)
    scales = scales_u8.view(np.float16).reshape(n_tiles, n_sb, 16, 4).astype(np.float32)  # [row][q]
    mq = np.ldexp(np.float32(1.0), 2 * np.arange(16) - 31).astype(np.float32)
    y = np.zeros(n_rows, dtype=np.float32)
    for tile in range(n_tiles):
        total = None
        for sb_begin in range(0, n_sb, MAX_SB):                 # launches
            sb_count = min(MAX_SB, n_sb - sb_begin)
            nsbw = (sb_count + 7) // 8
            S = (sb_count + nsbw - 1) // nsbw
            launch = np.zeros(16, dtype=np.float32)             # waves added in order
            for s in range(S):
                acc = np.zeros((16, 16), dtype=np.float32)      # [row][digit]
                sb_lo, sb_hi = sb_begin + s * nsbw, min(sb_begin + (s + 1) * nsbw, sb_begin + sb_count)
                E, zero = slice_exponent(xp[sb_lo * 512:sb_hi * 512])
                if E is None:
                    return np.full(n_rows, np.nan, dtype=np.float32)
                for sb in range(sb_lo, sb_hi):
                    for q in range(4):
                        dig, start = quantise_block_f4(xp[(sb * 4 + q) * 128:(sb * 4 + q + 1) * 128], E, fmt)
                        r = _f32(start[None, :] + _weight_operands_f4(codes, tile, sb, q, fmt) @ dig)   # exact
                        acc = _fma32(r, np.repeat(scales[tile, sb, :, q][:, None], 16, axis=1), acc)
                vg = []
                for g in range(4):                              # the four digits of a lane group, joined by FMAs
                    v = (acc[:, 4 * g] * mq[4 * g]).astype(np.float32)
                    for jj in range(1, 4):
                        v = _fma32(acc[:, 4 * g + jj], np.full(16, mq[4 * g + jj], np.float32), v)
                    vg.append(v)
                v = ((vg[0] + vg[1]).astype(np.float32) + (vg[2] + vg[3]).astype(np.float32)).astype(np.float32)
                launch = (launch + np.ldexp(v, 0 if zero else E - F4_P + 32).astype(np.float32)).astype(np.float32)
            total = launch if total is None else (total + launch).astype(np.float32)
        rows = tile * 16 + np.arange(16)
        ok = rows < n_rows
        y[rows[ok]] = total[ok]
    return y


def gemv(fmt: int, codes_u8: np.ndarray, scales_u8: np.ndarray, n_rows: int, k: int, x: np.ndarray, route: str | None = None) -> np.ndarray:
    """The route a single activation vector takes on the device: fp4 (`route="i8"` forces the int8 route, which the
    weights take from two vectors on)."""
    if route is None:
        route = "f4"
    if route == "f4":
        return gemv_f4(codes_u8, scales_u8, n_rows, k, x, fmt)
    n_tiles, n_sb = (n_rows + 15) // 16, (k + 511) // 512
    x = np.asarray(x, dtype=np.float32)
    xp = np.zeros(n_sb * 512, dtype=np.float32)
    xp[:k] = x
    unit = 256 if fmt == 0 else 512
    codes = codes_u8.view(np.uint32).reshape(n_tiles, n_sb, unit)
    scales = scales_u8.view(np.float16).reshape(n_tiles, n_sb, 16, 4).astype(np.float32)  # [row][q]
    y = np.zeros(n_rows, dtype=np.float32)
    for tile in range(n_tiles):
        total = None
        for sb_begin in range(0, n_sb, MAX_SB):                 # launches
            sb_count = min(MAX_SB, n_sb - sb_begin)
            nsbw = (sb_count + 7) // 8
            S = (sb_count + nsbw - 1) // nsbw
            launch = np.zeros(16, dtype=np.float32)
            for s in range(S):                                  # waves, added in order
                accf = np.zeros(16, dtype=np.float32)
                sb_lo, sb_hi = sb_begin + s * nsbw, min(sb_begin + (s + 1) * nsbw, sb_begin + sb_count)
                E, zero = slice_exponent(xp[sb_lo * 512:sb_hi * 512])
                if E is None:
                    return np.full(n_rows, np.nan, dtype=np.float32)
                for sb in range(sb_lo, sb_hi):
                    for q in range(4):
                        dig, c4 = quantise_block(fmt, xp[(sb * 4 + q) * 128:(sb * 4 + q + 1) * 128], E)
                        wb = _weight_bytes(fmt, codes, tile, sb, q)
                        acc = c4[None, :] + wb @ dig                                    # [16 rows][4 digits], exact
                        acc = ((acc + 2**31) % 2**32) - 2**31                           # int32 accumulators
                        lo = (acc[:, 0] + (acc[:, 1] << 8) + 2**31) % 2**32 - 2**31
                        hi = (acc[:, 2] + (acc[:, 3] << 8) + 2**31) % 2**32 - 2**31
                        val = _fma32(_f32(hi), _f32(np.full(16, 65536.0)), _f32(lo))
                        accf = _fma32(val, scales[tile, sb, :, q], accf)
                launch = (launch + np.ldexp(accf, 0 if zero else E - P[fmt]).astype(np.float32)).astype(np.float32)
            total = launch if total is None else (total + launch).astype(np.float32)
        rows = tile * 16 + np.arange(16)
        ok = rows < n_rows
        y[rows[ok]] = total[ok]
    return y
