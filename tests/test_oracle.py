"""Pins the CPU oracle (oracle/coffin_oracle.c) before anything is compared with it.

Three kinds of evidence, none of which retypes the oracle's own formula:
  * the committed known-answer vectors under tests/golden (exact rational
    arithmetic, written by tests/golden/make_golden.py);
  * what the mathematics fixes: invariants, constructed ties, hand-made cases,
    brute force in Python integers / fp64;
  * torch's CPU kernels as an independent engine evaluating the reference's
    expressions (division, round-half-even, bf16 narrowing, ``F.linear``).
"""

from __future__ import annotations

import numpy as np
import pytest
import torch


def _bits(t: torch.Tensor) -> np.ndarray:
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


# ------------------------------------------------------------------ R10 bf16

def test_bf16_matches_golden_and_torch(orc, golden):
    g = golden("bf16_rne")
    assert (orc.bf16_from_f32(g["src"]) == g["bits"]).all()
    rng = np.random.default_rng(7)
    x = (rng.standard_normal(20000) * 10 ** rng.uniform(-6, 6, 20000)).astype(np.float32)
    assert (orc.bf16_from_f32(x) == _bits(torch.from_numpy(x).to(torch.bfloat16))).all()
    assert (orc.bf16_to_f32(orc.bf16_from_f32(x)) ==
            torch.from_numpy(x).to(torch.bfloat16).float().numpy()).all()


def test_bf16_halfway_goes_to_even(orc):
    # 1 + 2^-8 is exactly between bf16(1.0) and the next value: ties to even (1.0);
    # 1 + 3*2^-8 is between 1+2^-7 (odd mantissa) and 1+2^-6 (even): goes up.
    x = np.array([1 + 2.0 ** -8, 1 + 3 * 2.0 ** -8, -(1 + 2.0 ** -8)], dtype=np.float32)
    assert orc.bf16_from_f32(x).tolist() == [0x3F80, 0x3F82, 0xBF80]


# ------------------------------------------------------------ R0 QWeight.quantize

def test_qweight_quantize_golden_invariants_and_torch(orc, golden):
    g = golden("qweight_quantize")
    wq, scale = orc.qweight_quantize(g["w"])
    assert (wq == g["wq"]).all() and (scale == g["scale"]).all()
    # zero row quantises to zeros with the floored scale, never inf/nan
    assert (wq[3] == 0).all() and scale[3] == np.float32(np.float32(1e-8) / np.float32(127.0))

    rng = np.random.default_rng(3)
    w = (rng.standard_normal((64, 300)) * 0.02).astype(np.float32)
    wq, scale = orc.qweight_quantize(w)
    assert np.abs(wq).max() <= 127
    assert (np.abs(wq).max(axis=1) == 127).all()          # every non-zero row reaches +-127
    err = np.abs(w.astype(np.float64) - wq.astype(np.float64) * scale[:, None].astype(np.float64))
    assert (err <= scale[:, None] * (0.5 + 1e-6)).all()    # at most half a step
    wt = torch.from_numpy(w)
    st = wt.abs().amax(-1).clamp_min(1e-8) / 127.0
    qt = (wt / st[:, None]).round().clamp_(-127, 127).to(torch.int8)
    assert (scale == st.numpy()).all() and (wq == qt.numpy()).all()


def test_qweight_dequant_is_one_rounding(orc):
    # tests/test_backends.py:889-903 pins (wq.float()*scale).to(bf16) as a single narrowing.
    rng = np.random.default_rng(5)
    wq = rng.integers(-127, 128, size=(16, 64)).astype(np.int8)
    scale = (rng.random(16) * 1e-3 + 1e-5).astype(np.float32)
    want = (torch.from_numpy(wq).float() * torch.from_numpy(scale)[:, None]).to(torch.bfloat16)
    assert (orc.qweight_dequant_bf16(wq, scale) == _bits(want)).all()


# ------------------------------------------------------- R3 activation quantiser

def test_quant_act_golden(orc, golden):
    g = golden("quant_act_i8")
    q, s = orc.quant_act_i8(g["x_bits"])
    assert (q == g["q"]).all() and (s == g["s"]).all()


def test_quant_act_special_rows(orc):
    k = 32
    x = np.zeros((4, k), dtype=np.float32)
    x[1, 5] = -2.0                                   # single spike -> -127 at the spike
    x[2, :] = 127.0                                  # s = 1 exactly
    x[2, 1:9] = [0.5, 1.5, 2.5, 3.5, -0.5, -1.5, -2.5, -3.5]   # exact ties -> even
    x[3, :] = 1e-7                                   # under the floor: s = 1e-5/127, q = round(1.27)
    q, s = orc.quant_act_i8(orc.bf16_from_f32(x))
    floor_s = np.float32(np.float32(1e-5) / np.float32(127.0))
    assert (q[0] == 0).all() and s[0] == floor_s
    assert q[1, 5] == -127 and np.count_nonzero(q[1]) == 1 and s[1] == np.float32(2.0 / 127.0)
    assert s[2] == 1.0 and q[2, 1:9].tolist() == [0, 2, 2, 4, 0, -2, -2, -4]
    assert s[3] == floor_s and (q[3] == 1).all()


def test_quant_act_uses_division_not_reciprocal(orc):
    # Search for an input where x * (1/s) and x / s round to different integers;
    # the oracle must agree with the division (the torch reference divides).
    rng = np.random.default_rng(11)
    found = 0
    for _ in range(200):
        x = rng.standard_normal((1, 512)).astype(np.float32)
        xb = orc.bf16_from_f32(x)
        xf = orc.bf16_to_f32(xb)
        s = np.float32(max(np.abs(xf).max(), np.float32(1e-5))) / np.float32(127.0)
        by_div = np.rint(xf / s)
        by_rcp = np.rint(xf * (np.float32(1.0) / s))
        q, so = orc.quant_act_i8(xb)
        assert so[0] == s
        assert (q == np.clip(by_div, -127, 127).astype(np.int8)).all()
        found += int((by_div != by_rcp).any())
    assert found > 0, "no discriminating input found; widen the search"


def test_quantiser_rounding_without_per_element_division_is_exhaustively_exact(orc):
    """The GPU kernels divide once per row (rc = 1/s) and round fma(fma(-x*rc, s, x), rc, x*rc)
    instead of x / s.  Every (row absmax, element) pair of finite bf16 values -- about 1e9 --
    gives the same int8 as the division; the quotients themselves are allowed to differ in
    the last bit (they do, in a fraction of a percent of the pairs), the integers are not."""
    assert orc.quant_division_mismatches(0, 0x7F80, check_quotient=False) == 0
    assert orc.quant_division_mismatches(0x3F00, 0x3F10, check_quotient=True) > 0


def test_quant_act_matches_torch_engine(orc):
    g = torch.Generator().manual_seed(1234)
    x = torch.randn(33, 2560, generator=g)
    x = torch.where(torch.rand(33, 2560, generator=g) < 0.01, x * 20, x).bfloat16()
    xf = x.float()
    s = xf.abs().amax(-1).clamp_min(1e-5) / 127.0
    q = (xf / s[:, None]).round().clamp_(-127, 127).to(torch.int8)
    oq, os_ = orc.quant_act_i8(_bits(x))
    assert (oq == q.numpy()).all() and (os_ == s.numpy()).all()
    # unclamped elements are within half a step
    assert (np.abs(xf.numpy() - oq * os_[:, None]) <= os_[:, None] * 0.50002).all()


# ---------------------------------------------------------------- R7 W4 format

def test_w4_pack_golden_and_hand_case(orc, golden):
    g = golden("w4_quantize")
    p, s = orc.w4_quantize(g["hand_w"], 2)
    assert (p == g["hand_packed"]).all() and (s == g["hand_scale"]).all()
    # [[1,-1],[7,-7]] with groups of 2: codes (15, 1) per row -> low nibble 15, high nibble 1
    assert p.tolist() == [[0x1F, 0x1F]]
    assert s.tolist() == [[np.float32(1.0) / np.float32(7.0), 1.0]]
    p, s = orc.w4_quantize(g["w"], 128)
    assert p.shape == (128, 6) and s.shape == (2, 6)       # K=200 padded to 256
    assert (p == g["packed"]).all() and (s == g["scale"]).all()
    assert (p[100:] == 0x88).all()                          # padding is code 8 in both nibbles


def test_w4_nibble_order_and_roundtrip(orc):
    # even k in the low nibble, odd k in the high nibble, K-major rows
    w = np.zeros((1, 128), dtype=np.float32)
    w[0, 0], w[0, 1], w[0, 2] = 7.0, -8.0 * 1.0, 3.0       # amax 8 -> s = 8/7
    p, s = orc.w4_quantize(w, 128)
    step = np.float32(8.0) / np.float32(7.0)
    assert s[0, 0] == step
    assert p[0, 0] == ((6 + 8) | ((-7 + 8) << 4))           # rne(7/s)=6, rne(-8/s)=-7
    assert p[1, 0] == ((3 + 8) | (8 << 4))                  # rne(3/s)=3 (2.625 -> 3)
    rng = np.random.default_rng(9)
    w = (rng.standard_normal((12, 384)) * 0.02).astype(np.float32)
    p, s = orc.w4_quantize(w, 128)
    d = orc.w4_dequant_f32(p, s, 384, 128)
    step = np.repeat(s.T, 128, axis=1)
    assert (np.abs(d - w) <= step * 0.5000001 + 1e-12).all()     # [-7,7] never clamps for absmax/7
    # decoder agrees with a bit-level decode written here
    codes = np.empty((12, 384), dtype=np.int32)
    codes[:, 0::2] = (p & 15).T
    codes[:, 1::2] = (p >> 4).T
    assert (d == (codes - 8).astype(np.float32) * step).all()


def test_w4_quantize_matches_torch_engine(orc):
    g = torch.Generator().manual_seed(1234)
    w = torch.randn(20, 512, generator=g) * 0.02
    grouped = w.view(20, 4, 128)
    s = grouped.abs().amax(-1).clamp_min(1e-8) / 7.0
    q = (grouped / s[..., None]).round().clamp_(-8, 7).to(torch.int32).view(20, 512) + 8
    packed = (q[:, 0::2] | (q[:, 1::2] << 4)).to(torch.uint8).t().contiguous()
    p, so = orc.w4_quantize(w.numpy(), 128)
    assert (p == packed.numpy()).all() and (so == s.t().contiguous().numpy()).all()


# ------------------------------------------------------------------ R4 W8A8

def test_gemm_w8a8_golden(orc, golden):
    g = golden("gemm_w8a8")
    acc, y = orc.gemm_w8a8(g["xq"], g["wq"], g["xs"], g["ws"])
    assert (acc == g["acc"]).all() and (y == g["y"]).all()
    assert acc[0, 0] == -127 * 127 * 64


def test_gemm_w8a8_against_exact_matmul_and_fp32_epilogue(orc):
    rng = np.random.default_rng(21)
    m, n, k = 17, 29, 2560
    xq = rng.integers(-127, 128, size=(m, k)).astype(np.int8)
    wq = rng.integers(-127, 128, size=(n, k)).astype(np.int8)
    xs = (rng.random(m) * 0.05 + 1e-3).astype(np.float32)
    ws = (rng.random(n) * 1e-3 + 1e-5).astype(np.float32)
    acc, y = orc.gemm_w8a8(xq, wq, xs, ws)
    exact = xq.astype(np.int64) @ wq.astype(np.int64).T      # order-free integer arithmetic
    assert (acc == exact).all()
    # epilogue: numpy float32 ops in the stated order, then torch's bf16 narrowing
    t = (acc.astype(np.float32) * xs[:, None]) * ws[None, :]
    assert (y == _bits(torch.from_numpy(t).to(torch.bfloat16))).all()
    # a transposed weight or a swapped scale would not survive this
    assert not (acc == (xq.astype(np.int64)[:, ::-1] @ wq.astype(np.int64).T)).all()


# ------------------------------------------------------------- R5 / R6 W4A8

def test_linear_w4a8_golden(orc, golden):
    g = golden("linear_w4a8")
    for tag in ("a", "b"):
        k, gs = int(g[f"{tag}_k"]), int(g[f"{tag}_gs"])
        gacc, y = orc.linear_w4a8(g[f"{tag}_xq"], g[f"{tag}_xs"], g[f"{tag}_packed"],
                                  g[f"{tag}_scale"], k, gs, want_group_acc=True)
        assert (gacc == g[f"{tag}_group_acc"]).all(), tag
        assert (y == g[f"{tag}_y"]).all(), tag


def test_linear_w4a8_group_sums_and_single_group_closed_form(orc):
    rng = np.random.default_rng(31)
    m, n, k = 4, 9, 512
    w = (rng.standard_normal((n, k)) * 0.02).astype(np.float32)
    packed, ws = orc.w4_quantize(w, 128)
    xq = rng.integers(-127, 128, size=(m, k)).astype(np.int8)
    xs = (rng.random(m) * 0.05 + 1e-3).astype(np.float32)
    gacc, y = orc.linear_w4a8(xq, xs, packed, ws, k, 128, want_group_acc=True)
    codes = np.empty((n, k), dtype=np.int64)
    codes[:, 0::2] = (packed & 15).T
    codes[:, 1::2] = (packed >> 4).T
    codes -= 8
    want = np.einsum("mgk,ngk->mgn", xq.astype(np.int64).reshape(m, 4, 128),
                     codes.reshape(n, 4, 128))
    assert (gacc == want).all()
    # fp64 evaluation of the same sum bounds the fp32 chain: <= G roundings of 2^-24 each
    ref = (want.astype(np.float64) * ws[None].astype(np.float64)).sum(1) * xs[:, None]
    got = orc.bf16_to_f32(y).astype(np.float64)
    assert (np.abs(got - ref) <= np.abs(ref) * 2.0 ** -8 + 1e-9).all()
    # with a single group the chain is one product: closed form in numpy float32
    gacc1, y1 = orc.linear_w4a8(xq[:, :128].copy(), xs, packed[:64].copy(), ws[:1].copy(),
                                128, 128, want_group_acc=True)
    t = (gacc1[:, 0, :].astype(np.float32) * ws[0][None, :]) * xs[:, None]
    assert (y1 == _bits(torch.from_numpy(t).to(torch.bfloat16))).all()


def fused_chain_case():
    """A two-group W4A8 input whose bf16 result tells a fused chain from an unfused
    one and ascending from descending group order.

    Group 0 contributes 127 * 1.0, group 1 contributes -127 * (1 + 2^-23).  The
    single-rounding chain fma(-127, 1+2^-23, 127) keeps the exact residue
    -127 * 2^-23 = -1.984375 * 2^-17 (bf16 0xB77E).  Rounding the second product
    first, or starting from group 1, gives -2^-16 (bf16 0xB780) instead.
    """
    k, gs = 256, 128
    packed = np.full((k // 2, 1), 0x88, dtype=np.uint8)
    packed[0, 0] = 0x89                      # code(k=0)   = 9 -> +1
    packed[64, 0] = 0x87                     # code(k=128) = 7 -> -1
    xq = np.zeros((1, k), dtype=np.int8)
    xq[0, 0], xq[0, 128] = 127, 127
    ws = np.array([[1.0], [1.0 + 2.0 ** -23]], dtype=np.float32)
    xs = np.ones(1, dtype=np.float32)
    return xq, xs, packed, ws, k, gs, 0xB77E


def test_linear_w4a8_chain_is_fused_and_ordered(orc):
    xq, xs, packed, ws, k, gs, want = fused_chain_case()
    gacc, y = orc.linear_w4a8(xq, xs, packed, ws, k, gs, want_group_acc=True)
    assert gacc[0, :, 0].tolist() == [127, -127]
    assert y[0, 0] == want
    # the two plausible mistakes land on the other value
    p1 = np.float32(-127.0) * ws[1, 0]
    assert orc.bf16_from_f32(np.array([np.float32(127.0) + p1]))[0] == 0xB780


# --------------------------------------------------------------- R1 / R2 / R8

def test_linear_w8a16_golden(orc, golden):
    g = golden("linear_w8a16")
    exact = orc.gemv_w8a16_exact(g["wq"], g["scale"], g["x_bits"])
    # double accumulation of exactly representable products: at most one fp32 ulp from exact
    assert np.allclose(exact, g["y_exact"], rtol=2.0 ** -22, atol=1e-12)
    ref = orc.bf16_to_f32(orc.linear_qweight(g["wq"], g["scale"], g["x_bits"]))
    want = orc.bf16_to_f32(orc.bf16_from_f32(g["y_ref"]))
    assert (np.abs(ref - want) <= np.abs(want) * 2.0 ** -7 + 1e-12).all()   # <= 1 bf16 ulp


def test_linear_reference_form_against_torch(orc):
    # The reference's own assertion (tests/test_backends.py:459-469): linear(q, x) equals
    # x @ dequant(q).T.  torch's CPU bf16 F.linear is the engine here.
    g = torch.Generator().manual_seed(1234)
    w = torch.randn(48, 256, generator=g) * 0.02
    x = torch.randn(5, 256, generator=g).bfloat16()
    wq, scale = orc.qweight_quantize(w.numpy())
    dense = (torch.from_numpy(wq).float() * torch.from_numpy(scale)[:, None]).to(torch.bfloat16)
    want = torch.nn.functional.linear(x, dense).float().numpy()
    got = orc.bf16_to_f32(orc.linear_qweight(wq, scale, _bits(x)))
    rel = np.abs(got - want).max() / np.abs(want).max()
    assert rel < 2e-2                                      # BF16_TOL of tests/test_backends.py:54
    # and in wide precision the two agree to fp32 rounding
    want64 = x.double().numpy() @ dense.double().numpy().T
    assert (np.abs(got - want64) <= np.abs(want64) * 2.0 ** -8 + 1e-9).all()


def test_linear_w4weight_is_dequant_then_linear(orc):
    g = torch.Generator().manual_seed(1234)
    w = torch.randn(24, 256, generator=g) * 0.02
    x = torch.randn(3, 256, generator=g).bfloat16()
    packed, scale = orc.w4_quantize(w.numpy(), 128)
    dense = torch.from_numpy(orc.w4_dequant_f32(packed, scale, 256, 128)).to(torch.bfloat16)
    want64 = x.double().numpy() @ dense.double().numpy().T
    got = orc.bf16_to_f32(orc.linear_w4weight(packed, scale, _bits(x), 256, 128))
    assert (np.abs(got - want64) <= np.abs(want64) * 2.0 ** -8 + 1e-9).all()
    # quantization error bound of the format itself: |w - dequant| <= step/2
    assert (np.abs(dense.float().numpy() - w.numpy()) <=
            np.repeat(scale.T, 128, axis=1) * 0.51 + np.abs(w.numpy()) * 2.0 ** -8).all()


# ------------------------------------------- fused producers: silu_mul, rms_norm

def _all_bf16():
    bits = np.arange(65536, dtype=np.uint16)
    return bits, torch.from_numpy(bits.view(np.int16)).view(torch.bfloat16)


def test_silu_table_matches_torch_on_every_finite_bf16_and_the_exact_function(orc):
    """silu of a bf16 value is a function of 16 bits.  All of them against torch's CPU F.silu
    (an independent evaluation of the reference's expression), and against the exact function
    in 50-digit decimal arithmetic wherever the exact value is not within 2^-18 (relative) of a
    bf16 rounding boundary -- the fp32 pipeline's own roundings stay far inside that."""
    from decimal import Decimal, getcontext
    bits, t = _all_bf16()
    got = orc.silu_bf16(bits)
    f = t.float().numpy()
    finite = np.isfinite(f)
    want = _bits(torch.nn.functional.silu(t))
    assert (got[finite] == want[finite]).all()
    # known answers and limits
    as_f = orc.bf16_to_f32(got)
    assert as_f[0x0000] == 0.0 and as_f[0x3F80] == np.float32(0.73046875)      # silu(1) = 0.731058... -> bf16
    assert as_f[0x7F80] == np.inf and np.isnan(as_f[0xFF80])                    # +inf -> +inf, -inf -> nan
    big = f > 20
    assert (got[big & finite] == bits[big & finite]).all()                      # silu(x) -> x
    getcontext().prec = 50
    sample = np.concatenate([np.arange(0x3000, 0x4200, 7), np.arange(0xB000, 0xC200, 7)])   # |x| in [2^-31, 8]
    checked = 0
    for b in sample:
        x = Decimal(float(f[b]))
        exact = x / (1 + (-x).exp())
        lo = float(orc.bf16_to_f32(np.array([got[b]], dtype=np.uint16))[0])
        ulp = 2.0 ** (np.floor(np.log2(abs(lo))) - 7)
        # distance from the returned bf16 value must not exceed half a step, up to the tie margin
        assert abs(exact - Decimal(lo)) <= Decimal(ulp) * (Decimal("0.5") + Decimal(2) ** -10), hex(int(b))
        checked += 1
    assert checked > 1000


def test_silu_mul_quant_is_silu_mul_then_the_quantiser(orc):
    rng = torch.Generator().manual_seed(1234)
    gate = (torch.randn((9, 300), generator=rng) * 3).to(torch.bfloat16)
    up = torch.randn((9, 300), generator=rng).to(torch.bfloat16)
    gate[4].zero_()                                                             # a zero row: q = 0, floor scale
    out, q, s = orc.silu_mul_quant(_bits(gate), _bits(up))
    want = torch.nn.functional.silu(gate) * up                                  # the reference statement, torch CPU
    assert (out == _bits(want)).all()
    q_ref, s_ref = orc.quant_act_i8(out)
    assert (q == q_ref).all() and (s == s_ref).all()
    assert (q[4] == 0).all() and s[4] == np.float32(1e-5) / np.float32(127)
    out2, q2, s2 = orc.silu_mul_quant(_bits(gate), _bits(up), quant=False)
    assert (out2 == out).all() and q2 is None and s2 is None


def test_rms_norm_known_answers_and_the_reference_expression(orc):
    """Closed forms (constant and zero rows), torch's CPU evaluation of the reference's lines
    (backends/reference/__init__.py:195-198) and an fp64 evaluation.  torch sums the squares in
    fp32 in an order of its own, so its scale may sit one fp32 step from the correctly rounded
    one: outputs agree bit for bit except where that step crosses a bf16 boundary."""
    rng = torch.Generator().manual_seed(1234)
    x = (torch.randn((33, 2560), generator=rng) * 2).to(torch.bfloat16)
    w = (1 + 0.1 * torch.randn(2560, generator=rng)).to(torch.bfloat16)
    x[0].zero_()
    x[1] = 0.5
    x[2] = -3.0
    y, x_after = orc.rms_norm(_bits(x), _bits(w))
    assert (x_after == _bits(x)).all()
    yf = orc.bf16_to_f32(y)
    wf = w.float().numpy()
    assert (yf[0] == 0).all()
    assert (yf[1] == wf).all() and (yf[2] == -wf).all()                         # |x| / sqrt(x^2 + 1e-6) -> 1
    xf = x.float()
    scale = torch.rsqrt(xf.pow(2).mean(dim=-1, keepdim=True) + 1e-6)
    ref = (xf * scale).to(torch.bfloat16) * w
    same = (y == _bits(ref))
    assert same.mean() > 0.995
    step = np.abs(yf) * 2.0 ** -7 + 1e-30
    assert (np.abs(yf - ref.float().numpy()) <= step).all()
    x64 = xf.double().numpy()
    s64 = 1.0 / np.sqrt((x64 ** 2).mean(-1, keepdims=True) + 1e-6)
    exact = x64 * s64 * w.double().numpy()
    assert (np.abs(yf - exact) <= np.abs(exact) * 2.0 ** -7 * 1.01 + 1e-30).all()  # two bf16 roundings
    # the residual add: bf16(x + add) written back, then the norm of the sum
    add = torch.randn((33, 2560), generator=rng).to(torch.bfloat16)
    y2, x2 = orc.rms_norm(_bits(x), _bits(w), add=_bits(add))
    summed = x + add                                                            # torch: fp32 add, one narrowing
    assert (x2 == _bits(summed)).all()
    y3, _ = orc.rms_norm(_bits(summed), _bits(w))
    assert (y2 == y3).all()
    # eps matters on small rows: x = 1e-3 -> 1e-3 / sqrt(1e-6 + 1e-6)
    tiny = torch.full((1, 64), 1e-3).to(torch.bfloat16)
    yt, _ = orc.rms_norm(_bits(tiny), _bits(torch.ones(64).to(torch.bfloat16)))
    v = float(tiny[0, 0])
    want = torch.tensor(v / np.sqrt(v * v + 1e-6)).to(torch.bfloat16)
    assert (orc.bf16_to_f32(yt) == float(want)).all()
