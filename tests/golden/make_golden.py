"""Writes the known-answer vectors in this directory.

Run from the repository root:  python tests/golden/make_golden.py

Every expected output here is computed with exact rational arithmetic
(``fractions.Fraction``) and explicit round-to-nearest-even narrowing, in pure
Python, from the formulas of the path (cited per function).  The script imports
neither the C oracle nor the device package, so the vectors are an independent
third statement that both are checked against.  Sizes are tiny on purpose.

bf16 values are stored as ``uint16`` bit patterns.
"""

from __future__ import annotations

import math
import struct
from fractions import Fraction
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent


# ----------------------------------------------------------- exact narrowing

def round_to_bits(x: Fraction, mant_bits: int, emin: int) -> Fraction:
    """Round ``x`` to a binary float with ``mant_bits`` significand bits (RNE)."""
    if x == 0:
        return Fraction(0)
    sign = -1 if x < 0 else 1
    ax = abs(x)
    e = ax.numerator.bit_length() - ax.denominator.bit_length()
    if Fraction(2) ** e > ax:
        e -= 1
    if Fraction(2) ** (e + 1) <= ax:
        e += 1
    e = max(e, emin)
    ulp = Fraction(2) ** (e - (mant_bits - 1))
    return sign * round(ax / ulp) * ulp  # Fraction round() is half-to-even


def f32(x: Fraction | int | float) -> Fraction:
    return round_to_bits(Fraction(x), 24, -126)


def bf16(x: Fraction) -> Fraction:
    return round_to_bits(Fraction(x), 8, -126)


def f32_bits(x: Fraction) -> int:
    return struct.unpack("<I", struct.pack("<f", float(x)))[0]


def bf16_bits(x: Fraction) -> int:
    return f32_bits(bf16(x)) >> 16


def bf16_bits_of_float(v: float) -> int:
    """bf16 pattern of an fp32 value; keeps the sign of zero, which a Fraction cannot."""
    if v == 0.0:
        return 0x8000 if math.copysign(1.0, v) < 0 else 0
    return bf16_bits(Fraction(v))


def from_bf16_bits(b: int) -> Fraction:
    return Fraction(struct.unpack("<f", struct.pack("<I", int(b) << 16))[0])


def rne_int(x: Fraction) -> int:
    return int(round(x))


def clamp(v: int, lo: int, hi: int) -> int:
    return max(lo, min(hi, v))


# ------------------------------------------------------------ the formulas

def quant_rows(x_bits: np.ndarray, floor: float, qmax: int):
    """s = max(amax|x|, floor)/qmax (fp32); q = clamp(rne(fp32(x/s)), -qmax, qmax).

    Activation form: backends/reference/__init__.py:386-389 (floor 1e-5, 127).
    """
    m, k = x_bits.shape
    q = np.zeros((m, k), dtype=np.int8)
    s = np.zeros(m, dtype=np.float32)
    fl = f32(Fraction(np.float32(floor).item()))
    for i in range(m):
        row = [from_bf16_bits(b) for b in x_bits[i]]
        amax = max(abs(v) for v in row)
        sc = f32(max(amax, fl) / qmax)
        s[i] = float(sc)
        for j, v in enumerate(row):
            q[i, j] = clamp(rne_int(f32(v / sc)), -qmax, qmax)
    return q, s


def qweight_quantize(w: np.ndarray):
    """int8_weights.py:328-332: per-row absmax, floor 1e-8, divisor 127."""
    n, k = w.shape
    wq = np.zeros((n, k), dtype=np.int8)
    scale = np.zeros(n, dtype=np.float32)
    fl = f32(Fraction(np.float32(1e-8).item()))
    for i in range(n):
        row = [Fraction(float(v)) for v in w[i]]
        sc = f32(max(max(abs(v) for v in row), fl) / 127)
        scale[i] = float(sc)
        for j, v in enumerate(row):
            wq[i, j] = clamp(rne_int(f32(v / sc)), -127, 127)
    return wq, scale


def w4_quantize(w: np.ndarray, gs: int):
    """tools/quant_disk_w4a8.py:45-89: group absmax / 7, clamp [-8,7], code = q+8,
    even k low nibble, zero padding (code 8) to whole groups and an even length."""
    n, k = w.shape
    groups = -(-k // gs)
    kp = groups * gs
    ke = kp + (kp & 1)
    packed = np.zeros((ke // 2, n), dtype=np.uint8)
    scale = np.zeros((groups, n), dtype=np.float32)
    fl = f32(Fraction(np.float32(1e-8).item()))
    for i in range(n):
        codes = [8] * ke
        for g in range(groups):
            vals = [Fraction(float(w[i, kk])) if kk < k else Fraction(0)
                    for kk in range(g * gs, (g + 1) * gs)]
            sc = f32(max(max(abs(v) for v in vals), fl) / 7)
            scale[g, i] = float(sc)
            for off, v in enumerate(vals):
                codes[g * gs + off] = clamp(rne_int(f32(v / sc)), -8, 7) + 8
        for j in range(ke // 2):
            packed[j, i] = codes[2 * j] | (codes[2 * j + 1] << 4)
    return packed, scale


def w4_code(packed: np.ndarray, kk: int, n: int) -> int:
    b = int(packed[kk // 2, n])
    return ((b >> 4) if kk & 1 else (b & 15)) - 8


def gemm_w8a8(xq, wq, xs, ws):
    """acc exact; y = bf16(fp32(fp32(fp32(acc) * xs[m]) * ws[n]))
    (backends/corex/kernels/w8a8.cu:208)."""
    m, k = xq.shape
    n = wq.shape[0]
    acc = np.zeros((m, n), dtype=np.int32)
    y = np.zeros((m, n), dtype=np.uint16)
    for i in range(m):
        for j in range(n):
            a = sum(int(xq[i, t]) * int(wq[j, t]) for t in range(k))
            acc[i, j] = a
            t1 = f32(f32(a) * Fraction(float(xs[i])))
            y[i, j] = bf16_bits(f32(t1 * Fraction(float(ws[j]))))
    return acc, y


def linear_w4a8(xq, xs, packed, ws, k: int, gs: int):
    """Per group int32 sum; total = fp32(sum*ws + total) (single rounding), groups
    ascending from 0; y = bf16(fp32(total * xs[m]))
    (backends/corex/kernels/w4a8.cu:168-172,193; w8a8_tcu.cu:484-499,570)."""
    m = xq.shape[0]
    n = packed.shape[1]
    groups = -(-k // gs)
    gacc = np.zeros((m, groups, n), dtype=np.int32)
    y = np.zeros((m, n), dtype=np.uint16)
    for i in range(m):
        for j in range(n):
            total = Fraction(0)
            for g in range(groups):
                s = sum(int(xq[i, t]) * w4_code(packed, t, j)
                        for t in range(g * gs, min(k, (g + 1) * gs)))
                gacc[i, g, j] = s
                total = f32(f32(s) * Fraction(float(ws[g, j])) + total)
            y[i, j] = bf16_bits(f32(total * Fraction(float(xs[i]))))
    return gacc, y


def gemv_w8a16_exact(wq, scale, x_bits):
    """scale[n] * sum_k wq[n,k]*x[m,k], exact, then rounded once to fp32
    (backends/corex/kernels/gemv.cu:784-785: scale applied once after the K-sum)."""
    n, k = wq.shape
    m = x_bits.shape[0]
    out = np.zeros((m, n), dtype=np.float32)
    for i in range(m):
        xv = [from_bf16_bits(b) for b in x_bits[i]]
        for j in range(n):
            acc = sum(int(wq[j, t]) * xv[t] for t in range(k))
            out[i, j] = float(f32(acc * Fraction(float(scale[j]))))
    return out


def linear_qweight_ref(wq, scale, x_bits):
    """backends/reference/__init__.py:93-95 with bf16 operands: the weight is
    rounded to bf16 once (int8_weights.py:359), products summed exactly here,
    result rounded to fp32 (any fp32 summation order lands within rounding of it)."""
    n, k = wq.shape
    m = x_bits.shape[0]
    out = np.zeros((m, n), dtype=np.float32)
    for j in range(n):
        dense = [bf16(f32(int(wq[j, t]) * Fraction(float(scale[j])))) for t in range(k)]
        for i in range(m):
            xv = [from_bf16_bits(b) for b in x_bits[i]]
            out[i, j] = float(f32(sum(d * v for d, v in zip(dense, xv))))
    return out


# ------------------------------------------------------------------ vectors

def to_bf16_bits(a: np.ndarray) -> np.ndarray:
    out = np.zeros(a.shape, dtype=np.uint16)
    for idx in np.ndindex(a.shape):
        out[idx] = bf16_bits_of_float(float(a[idx]))
    return out


def main() -> None:
    rng = np.random.default_rng(1234)

    # --- bf16 narrowing: random, exact halfway cases, signed zero, tiny values
    vals = list(rng.standard_normal(64).astype(np.float32))
    for base in (1.0, 3.0, 127.0, 1e-3, 65280.0):
        b = struct.unpack("<I", struct.pack("<f", base))[0] & 0xFFFF0000
        for low in (0x7FFF, 0x8000, 0x8001, 0x18000 - 0x10000):
            vals.append(struct.unpack("<f", struct.pack("<I", b | low))[0])
            vals.append(struct.unpack("<f", struct.pack("<I", (b + 0x10000) | low))[0])
    vals += [0.0, -0.0, 1e-30, -1e-30, 3.0e38]
    src = np.array(vals, dtype=np.float32)
    np.savez(HERE / "bf16_rne.npz", src=src,
             bits=np.array([bf16_bits_of_float(float(v)) for v in src], dtype=np.uint16))

    # --- activation quantiser: random rows + zero row + spike + constructed ties
    m, k = 6, 48
    x = rng.standard_normal((m, k)).astype(np.float32)
    x[1] = 0.0
    x[2] = 0.0
    x[2, 7] = -3.5
    # row 3: amax 127 -> s = 1 exactly, then half-integers are exact ties
    x[3] = np.array([127.0] + [0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 63.5, -126.5] * 5 + [3.0] * 7,
                    dtype=np.float32)
    # row 4: tiny magnitudes under the 1e-5 floor
    x[4] = (rng.standard_normal(k) * 1e-7).astype(np.float32)
    x[5] = rng.standard_normal(k).astype(np.float32) * 300.0
    xb = to_bf16_bits(x)
    q, s = quant_rows(xb, 1e-5, 127)
    np.savez(HERE / "quant_act_i8.npz", x_bits=xb, q=q, s=s)

    # --- QWeight.quantize
    w = (rng.standard_normal((5, 40)) * 0.02).astype(np.float32)
    w[3] = 0.0
    wq, sc = qweight_quantize(w)
    np.savez(HERE / "qweight_quantize.npz", w=w, wq=wq, scale=sc)

    # --- W4 format: a hand-made 2x2 case plus a ragged seeded case
    hand = np.array([[1.0, -1.0], [7.0, -7.0]], dtype=np.float32)  # gs=2: scales 1/7 and 1
    hp, hs = w4_quantize(hand, 2)
    # row 0: w/s = +-7 -> codes 15, 1 -> byte 0x1F ; row 1: codes 15, 1 -> 0x1F
    assert hp.tolist() == [[0x1F, 0x1F]], hp
    w4w = (rng.standard_normal((6, 200)) * 0.02).astype(np.float32)  # K not a multiple of 128
    p4, s4 = w4_quantize(w4w, 128)
    np.savez(HERE / "w4_quantize.npz", hand_w=hand, hand_packed=hp, hand_scale=hs,
             w=w4w, packed=p4, scale=s4)

    # --- W8A8 GEMM (K = 64 and scales spanning magnitudes)
    m, n, k = 5, 7, 64
    xq = rng.integers(-127, 128, size=(m, k)).astype(np.int8)
    wq8 = rng.integers(-127, 128, size=(n, k)).astype(np.int8)
    xq[0] = 127
    wq8[0] = -127          # extreme accumulator -127*127*64
    xs = (rng.random(m) * 0.05 + 1e-3).astype(np.float32)
    ws8 = (rng.random(n) * 1e-3 + 1e-5).astype(np.float32)
    acc, y = gemm_w8a8(xq, wq8, xs, ws8)
    np.savez(HERE / "gemm_w8a8.npz", xq=xq, wq=wq8, xs=xs, ws=ws8, acc=acc, y=y)

    # --- W4A8 linear: K = 256 (two groups) and a three-group case with a short tail group
    def w4_case(m, n, k, gs):
        wd = (rng.standard_normal((n, k)) * 0.02).astype(np.float32)
        pk, scl = w4_quantize(wd, gs)
        xq_ = rng.integers(-127, 128, size=(m, k)).astype(np.int8)
        xs_ = (rng.random(m) * 0.05 + 1e-3).astype(np.float32)
        ga, yy = linear_w4a8(xq_, xs_, pk, scl, k, gs)
        return dict(packed=pk, scale=scl, xq=xq_, xs=xs_, group_acc=ga, y=yy,
                    k=np.int64(k), gs=np.int64(gs))
    a = w4_case(3, 5, 256, 128)
    b = w4_case(2, 4, 320, 128)
    np.savez(HERE / "linear_w4a8.npz", **{f"a_{kk}": v for kk, v in a.items()},
             **{f"b_{kk}": v for kk, v in b.items()})

    # --- int8 weight-only linear: exact device meaning and the torch-reference meaning
    n, k, m = 6, 64, 3
    wd = (rng.standard_normal((n, k)) * 0.02).astype(np.float32)
    wq1, sc1 = qweight_quantize(wd)
    xb1 = to_bf16_bits(rng.standard_normal((m, k)).astype(np.float32))
    np.savez(HERE / "linear_w8a16.npz", wq=wq1, scale=sc1, x_bits=xb1,
             y_exact=gemv_w8a16_exact(wq1, sc1, xb1), y_ref=linear_qweight_ref(wq1, sc1, xb1))
    print("golden vectors written to", HERE)


if __name__ == "__main__":
    main()
