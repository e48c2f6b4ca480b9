"""Device parity at the projection shapes of the reference's own 4B model.

The benchmark configuration uses intermediate 9728; the reference's model has
intermediate 9216 and the projection table of backends/corex/__init__.py:135-143
(gate_up 2560 -> 18432, full_attn 2560 -> 10240, linear_attn 2560 -> 12352,
o_proj 4096 -> 2560, k5120 5120 -> 2560, mlp_down 9216 -> 2560) and a vocabulary
of 248320 rows (int8_weights.py:312-316).  K = 9216 is nine whole 1024-element
segments (three units of three), 12352 is not a multiple of 128 rows: blockings
the benchmark shapes do not reach.  Same bars as the other parity tests.
"""

from __future__ import annotations

import numpy as np
import pytest
import torch

from coffin_amd import synth
from tests import gpu_util as G
from tests.test_gpu_parity import (_assert_weight_only_tolerance, _w4_case, _w8a16_case, seeded)

pytestmark = pytest.mark.gpu

#: (N, K) of the reference's 4B projections.
LAYER_SHAPES = [(18432, 2560), (10240, 2560), (12352, 2560), (2560, 4096), (2560, 5120), (2560, 9216)]


@pytest.mark.parametrize("n,k", LAYER_SHAPES)
@pytest.mark.parametrize("m", [1, 8])
def test_gemv_w8a16_reference_shapes(orc, m, n, k):
    wq, ws, x, y = _w8a16_case(orc, m, n, k, seeded())
    _assert_weight_only_tolerance(orc, wq, ws, x, y)


@pytest.mark.parametrize("n,k", LAYER_SHAPES)
def test_gemv_w8a16_rows_do_not_depend_on_the_batch(n, k):
    """Row r of a 2..16-row call carries the bits of the single-row call on x[r]."""
    g = synth.generator(1234, G.DEV)
    q = synth.int8_weight(n, k, g)
    x = synth.activations(16, k, g)
    single = torch.cat([G.gemv_w8a16(q.wq, q.scale, x[r:r + 1].contiguous()) for r in (0, 5, 15)])
    for m in (2, 4, 7, 16):
        y = G.gemv_w8a16(q.wq, q.scale, x[:m].contiguous())
        rows = [r for r in (0, 5, 15) if r < m]
        want = single[[(0, 5, 15).index(r) for r in rows]]
        assert (y[rows].view(torch.int16) == want.view(torch.int16)).all(), m


@pytest.mark.parametrize("n,k", [(12352, 2560), (2560, 9216)])
def test_gemv_w8a16_mfma_reference_shapes(orc, n, k):
    wq, ws, x, y = _w8a16_case(orc, 16, n, k, seeded(), mfma=True)
    _assert_weight_only_tolerance(orc, wq, ws, x, y)


def test_gemv_w8a16_vocabulary_rows_sampled(orc):
    """lm_head of the reference's vocabulary (248320 rows): a sample of rows against the
    oracle, and the launch against the same rows computed as a small weight of their own."""
    n, k = 248320, 2560
    g = synth.generator(1234, G.DEV)
    q = synth.int8_weight(n, k, g)
    x = synth.activations(2, k, g)
    y = G.gemv_w8a16(q.wq, q.scale, x)
    ridx = torch.tensor([0, 1, 4095, 131071, 200001, n - 2, n - 1], device=G.DEV)
    sub_w, sub_s = q.wq[ridx].contiguous(), q.scale[ridx].contiguous()
    y_sub = G.gemv_w8a16(sub_w, sub_s, x)
    assert (y[:, ridx].contiguous().view(torch.int16) == y_sub.view(torch.int16)).all()
    ref = orc.bf16_to_f32(orc.linear_qweight(sub_w.cpu().numpy(), sub_s.cpu().numpy(), G.bits(x)))
    rms = float(np.sqrt((ref.astype(np.float64) ** 2).mean()))
    assert (np.abs(y_sub.float().cpu().numpy() - ref) <= 1e-2 * rms + np.abs(ref) * 2.0 ** -7).all()


@pytest.mark.parametrize("m,n,k", [(16, 12352, 2560), (96, 2560, 9216), (16, 2560, 9216), (384, 1544, 9216),
                                   (300, 12352, 512)])
def test_gemm_w8a8_reference_shapes_bit_exact(orc, m, n, k):
    G.set_option("gemm_tile", 0)
    g = seeded()
    q = synth.int8_weight(n, k, g)
    x = synth.activations(m, k, g, outliers=True)
    xq, xs = orc.quant_act_i8(G.bits(x))
    acc_ref, y_ref = orc.gemm_w8a8(xq, q.wq.numpy(), xs, q.scale.numpy())
    acc, y = G.gemm_w8a8(G.dev(xq), q.wq.to(G.DEV), G.dev(xs), q.scale.to(G.DEV))
    assert (acc.cpu().numpy() == acc_ref).all()
    assert (G.bits(y) == y_ref).all()


@pytest.mark.parametrize("m,n,k,gemm", [(1, 18432, 2560, False), (1, 2560, 9216, False), (16, 2560, 9216, False),
                                        (16, 12352, 2560, False), (64, 2560, 9216, True), (320, 1544, 9216, True),
                                        (272, 12352, 256, True)])
def test_w4a8_reference_shapes_bit_exact(orc, m, n, k, gemm):
    w4, ws, xq, xs, gacc_ref, y_ref = _w4_case(orc, m, n, k, seeded())
    gacc, y = G.w4a8(w4, ws, xq, xs, k, gemm=gemm)
    assert (gacc.cpu().numpy() == gacc_ref).all()
    assert (G.bits(y) == y_ref).all()
