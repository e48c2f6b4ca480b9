"""Device parity at every benchmark configuration that the other GPU tests do not reach.

* W8A8 prefill GEMM, K = 2560: every (M, N) of M in {512, 2048, 8192} x N in {9728, 4096}, every
  block-tile kernel forced in turn: a sample of rows bit for bit against the oracle, all rows
  through a checksum of the int32 accumulators, a band of rows against the same rows computed as
  a problem of their own.
* W4A8 on the larger dense shape, K = 5120 -> N = 25600 and K = 25600 -> N = 5120, at M = 1, 64
  and 1024 (GEMV entry up to 16 rows, GEMM entry beyond): a sample of output columns bit for bit
  against the oracle (int32 group sums and bf16 output), every column through a checksum of the
  group sums.
* The W4A8 kernels against the reference's own statement for an int4 weight, which does *not*
  quantise the activations (backends/reference/__init__.py:94, w4a8_weights.py:96-99): the
  distance is the activation-quantisation error and is held to the bound derived at
  ``W4_VS_UNQUANTISED_*``.
"""

from __future__ import annotations

import numpy as np
import pytest
import torch

from coffin_amd import synth
from tests import gpu_util as G

pytestmark = pytest.mark.gpu


@pytest.fixture(params=["auto", "64", "128", "192", "128192", "256", "320", "321", "322"])
def gemm_tile(request):
    if request.param != "auto":
        G.set_option("gemm_tile", int(request.param))
    else:
        G.set_option("gemm_tile", 0)
    return request.param


@pytest.mark.parametrize("m,n", [(512, 9728), (512, 4096), (2048, 9728), (2048, 4096),
                                 (8192, 9728), (8192, 4096)])
def test_gemm_w8a8_every_prefill_configuration(orc, gemm_tile, m, n):
    k = 2560
    g = synth.generator(1234, G.DEV)
    q = synth.int8_weight(n, k, g)
    x = synth.activations(m, k, g, outliers=True)
    xq, xs = G.quant(x)
    # the quantiser itself at this size, on the sampled rows below
    rows = torch.randint(0, m, (22,), generator=torch.Generator().manual_seed(m + n)).tolist()
    rows += [0, 127, 128, 255, 256, m - 129, m - 1]
    ridx = torch.tensor(rows, device=G.DEV)
    xq_ref, xs_ref = orc.quant_act_i8(G.bits(x[ridx]))
    assert (xq[ridx].cpu().numpy() == xq_ref).all() and (xs[ridx].cpu().numpy() == xs_ref).all()
    acc, y = G.gemm_w8a8(xq, q.wq, xs, q.scale)
    acc_ref, y_ref = orc.gemm_w8a8(xq_ref, q.wq.cpu().numpy(), xs_ref, q.scale.cpu().numpy())
    assert (acc[ridx].cpu().numpy() == acc_ref).all()
    assert (G.bits(y[ridx]) == y_ref).all()
    # every element: column and row checksums of the int32 accumulators against exact fp64
    # contractions (|sum| < 2^53)
    col_sum = xq.double().sum(0) @ q.wq.double().t()                      # [N]
    assert (acc.double().sum(0) == col_sum).all()
    row_sum = xq.double() @ q.wq.double().sum(0)                          # [M]
    assert (acc.double().sum(1) == row_sum).all()
    # a band of rows as a smaller problem gives identical bits; and the output without the
    # accumulator dump equals the one with it
    lo = m // 2 - 100
    acc2, y2 = G.gemm_w8a8(xq[lo:lo + 300].contiguous(), q.wq, xs[lo:lo + 300].contiguous(), q.scale)
    assert (acc2 == acc[lo:lo + 300]).all()
    assert (y2.view(torch.int16) == y[lo:lo + 300].view(torch.int16)).all()
    _, y3 = G.gemm_w8a8(xq, q.wq, xs, q.scale, want_acc=False)
    assert (y3.view(torch.int16) == y.view(torch.int16)).all()


def _w4_codes_minus8(w):
    """int8 [N, K] of q = code - 8 from the contract layout (low nibble = even k)."""
    p = w.packed                                                          # [K/2, N]
    out = torch.empty((p.shape[1], p.shape[0] * 2), dtype=torch.float64, device=p.device)
    out[:, 0::2] = ((p & 15).to(torch.float64) - 8).t()
    out[:, 1::2] = ((p >> 4).to(torch.float64) - 8).t()
    return out


@pytest.mark.parametrize("n,k", [(25600, 5120), (5120, 25600)])
@pytest.mark.parametrize("m", [1, 64, 1024])
def test_w4a8_larger_dense_shape_every_batch(orc, m, n, k):
    g = synth.generator(1234, G.DEV)
    w = synth.int4_weight(n, k, g)
    w4, ws = G.w4_repack(w.packed, w.scale, k)
    x = synth.activations(m, k, g)
    xq, xs = G.quant(x)
    xq_h, xs_h = xq.cpu().numpy(), xs.cpu().numpy()
    q_ref, s_ref = orc.quant_act_i8(G.bits(x))
    assert (xq_h == q_ref).all() and (xs_h == s_ref).all()
    gacc, y = G.w4a8(w4, ws, xq, xs, k, gemm=m > 16)
    n_cols = 96 if m <= 64 else 40
    cols = torch.cat([torch.randint(0, n, (n_cols,), generator=torch.Generator().manual_seed(11 + m)),
                      torch.tensor([0, 15, 16, 127, 128, n - 129, n - 17, n - 1])]).to(G.DEV)
    gacc_ref, y_ref = orc.linear_w4a8(xq_h, xs_h, w.packed[:, cols].contiguous().cpu().numpy(),
                                      w.scale[:, cols].contiguous().cpu().numpy(), k, 128,
                                      want_group_acc=True)
    assert (gacc[:, :, cols].cpu().numpy() == gacc_ref).all()
    assert (G.bits(y[:, cols].contiguous()) == y_ref).all()
    # every column: the group sums added over the groups are the plain int8 x int4 products;
    # checksums over rows and over columns against exact fp64 contractions
    codes = _w4_codes_minus8(w)                                           # [N, K] fp64
    total = gacc.double().sum(1)                                          # [M, N]
    assert (total.sum(0) == xq.double().sum(0) @ codes.t()).all()
    assert (total.sum(1) == xq.double() @ codes.sum(0)).all()
    del codes, total
    # the output without the dump of the group sums carries the same bits
    _, y2 = G.w4a8(w4, ws, xq, xs, k, gemm=m > 16, want_acc=False)
    assert (y2.view(torch.int16) == y.view(torch.int16)).all()
    if m == 64:
        # the GEMV entry on 16 of the rows agrees with the GEMM entry on all of them
        _, y16 = G.w4a8(w4, ws, xq[16:32].contiguous(), xs[16:32].contiguous(), k, gemm=False, want_acc=False)
        assert (y16.view(torch.int16) == y[16:32].view(torch.int16)).all()


#: W4A8 kernels against the reference statement on *unquantised* bf16 activations.  With
#: e[k] = x[k] - xq[k]*xs the two differ by sum_k w[n,k]*e[k] plus roundings:
#:   * hard bound: |e[k]| <= xs/2, so |diff| <= (xs/2) * sum_k |w[n,k]|, plus the reference's
#:     weight narrowing to bf16 (relative 2^-9 per weight, against sum_k |w x|) and one bf16
#:     output rounding on each side (2^-8 relative each);
#:   * e is uniform on a step of xs (standard deviation xs/sqrt(12)), so the RMS of the
#:     difference over the outputs is xs/sqrt(12) * sqrt(sum_k w^2) -- about 0.8 % of RMS(y)
#:     for N(0,1) activations of these lengths (xs ~ 3.9/127) -- plus bf16 rounding noise;
#:     asserted below 2 % of RMS(y).
W4_VS_UNQUANTISED_RMS = 2e-2


@pytest.mark.parametrize("m,n,k", [(1, 9728, 2560), (16, 2560, 9728), (64, 2560, 2560), (4, 1024, 5120)])
def test_w4a8_kernels_stay_within_quantisation_error_of_the_unquantised_reference(orc, m, n, k):
    g = synth.generator(1234)
    w = synth.int4_weight(n, k, g)
    x = synth.activations(m, k, g)
    ref = orc.bf16_to_f32(orc.linear_w4weight(w.packed.numpy(), w.scale.numpy(), G.bits(x), k, 128))
    w4, ws = G.w4_repack(w.packed.to(G.DEV), w.scale.to(G.DEV), k)
    xq, xs = G.quant(x.to(G.DEV))
    _, y = G.w4a8(w4, ws, xq, xs, k, gemm=m > 16, want_acc=False)
    got = y.float().cpu().numpy().astype(np.float64)
    dense = orc.w4_dequant_f32(w.packed.numpy(), w.scale.numpy(), k, 128).astype(np.float64)   # [N, K]
    xf = x.float().numpy().astype(np.float64)
    l1 = np.abs(dense).sum(1)                                             # [N]
    absdot = np.abs(xf) @ np.abs(dense).T                                 # [M, N]
    step = xs.cpu().numpy().astype(np.float64)[:, None]
    hard = 0.5 * step * l1[None, :] + absdot * 2.0 ** -9 + (np.abs(ref) + np.abs(got)) * 2.0 ** -8
    assert (np.abs(got - ref) <= hard * 1.001).all()
    rms = np.sqrt((ref.astype(np.float64) ** 2).mean())
    err = np.sqrt(((got - ref) ** 2).mean())
    assert err <= W4_VS_UNQUANTISED_RMS * rms, (err / rms)
    assert err >= 1e-3 * rms            # and they do differ: the reference does not quantise x


# ------------------------------------------------------------- W4A16 (int4 weight-only) GEMV

@pytest.mark.parametrize("n,k", [(9728, 2560), (2560, 9728), (2560, 4096), (6144, 2560), (37, 128), (1001, 384),
                                 (300, 2048), (64, 10240), (5, 6272),
                                 # rows longer than 10240: 6..16 passes (config 5's 25600 -> 5120 among them)
                                 (5120, 25600), (100, 12288), (33, 16384), (17, 20480), (40, 32768), (9, 28672)])
def test_gemv_w4a16_against_the_exact_sum_and_the_unquantised_reference(orc, n, k):
    """The int4 weight-only GEMV is a floating-point path (fp32 sums in the kernel's own order):
    held to the exact value of sum_k (code - 8) * scale * x within its final bf16 rounding plus
    fp32 accumulation noise, and to the reference's torch statement for an int4 weight
    (dequantised to bf16, bf16 product; orc.linear_w4weight) within 1e-2 of the output RMS plus
    one bf16 step -- the bound of the int8 weight-only path."""
    g = synth.generator(1234)
    w = synth.int4_weight(n, k, g)
    x = synth.activations(1, k, g)
    w4, ws = G.w4_repack(w.packed.to(G.DEV), w.scale.to(G.DEV), k)
    y = G.gemv_w4a16(w4, ws, x[0].contiguous().to(G.DEV), k)
    got = y.float().cpu().numpy().astype(np.float64)
    dense = orc.w4_dequant_f32(w.packed.numpy(), w.scale.numpy(), k, 128).astype(np.float64)     # exact: 4-bit x fp16 scale
    exact = dense @ x[0].float().numpy().astype(np.float64)
    rms = np.sqrt((exact ** 2).mean()) + 1e-30
    assert (np.abs(got - exact) <= np.abs(exact) * 2.0 ** -8 * 1.01 + 2e-5 * rms).all()
    ref = orc.bf16_to_f32(orc.linear_w4weight(w.packed.numpy(), w.scale.numpy(), G.bits(x), k, 128))[0]
    assert (np.abs(got - ref) <= 1e-2 * rms + np.abs(ref) * 2.0 ** -7).all()
    assert np.sqrt(((got - exact) ** 2).mean()) / rms < 3e-3
    # zero activations give exact zeros; a power-of-two scaling of the group scales scales exactly
    assert (G.gemv_w4a16(w4, ws, torch.zeros(k, dtype=torch.bfloat16, device=G.DEV), k).float() == 0).all()
    y2 = G.gemv_w4a16(w4, ws * 4.0, x[0].contiguous().to(G.DEV), k)
    assert (y2.float() == y.float() * 4.0).all()


def test_w4a16_switch_in_the_adapter(monkeypatch, orc):
    from coffin_amd import backend
    from coffin_amd.weights import W4A8Weight
    g = synth.generator(3)
    w = synth.int4_weight(512, 2560, g)
    wd = W4A8Weight(w.packed.to(G.DEV), w.scale.to(G.DEV), k=2560)
    x = synth.activations(3, 2560, g).to(G.DEV)
    quantised = backend.linear_m(wd, x)
    monkeypatch.setattr(backend, "W4A16", True)
    unquantised = backend.linear_m(wd, x)
    w4, ws = G.w4_repack(wd.packed, wd.scale, 2560)
    for r in range(3):
        assert (unquantised[r].view(torch.int16) == G.gemv_w4a16(w4, ws, x[r].contiguous(), 2560).view(torch.int16)).all()
    assert (backend.linear(wd, x[1]).view(torch.int16) == unquantised[1].view(torch.int16)).all()
    # the two arithmetics differ by the activation-quantisation error, no more
    diff = (unquantised.float() - quantised.float()).abs()
    rms = unquantised.float().pow(2).mean().sqrt()
    assert 1e-4 * rms < diff.mean() < 2e-2 * rms
    # wider batches keep W4A8
    x8 = synth.activations(8, 2560, g).to(G.DEV)
    monkeypatch.setattr(backend, "W4A16", False)
    want8 = backend.linear_m(wd, x8)
    monkeypatch.setattr(backend, "W4A16", True)
    assert (backend.linear_m(wd, x8).view(torch.int16) == want8.view(torch.int16)).all()
