"""int4 weights beyond "group 128, K a multiple of 128": group sizes 64 and 256 and rows whose
length is not a whole number of groups (w4a8_weights.py:28-50: any ``group_size``,
``ceil(K / group_size)`` groups, pad code 8; backends/corex/__init__.py:633 takes group sizes
that are multiples of 64 on its matrix path).  Bit for bit against the oracle, through the C ABI and
through the table entries."""

from __future__ import annotations

import numpy as np
import pytest
import torch

from coffin_amd import _native, backend, synth
from coffin_amd.embed import TiedEmbedding
from coffin_amd.weights import W4A8Weight
from tests import gpu_util as G

pytestmark = pytest.mark.gpu


def _weight(n, k, gs, g):
    return W4A8Weight.quantize(synth.dense_weight(n, k, g), group_size=gs)


def _padded(a: np.ndarray, kd: int) -> np.ndarray:
    out = np.zeros((a.shape[0], kd), dtype=a.dtype)
    out[:, :a.shape[1]] = a
    return out


@pytest.mark.parametrize("gs", [64, 256])
@pytest.mark.parametrize("m,n,k", [(1, 9728, 2560), (1, 2560, 9728), (2, 333, 1280), (4, 512, 256), (3, 7, 256),
                                   (8, 1024, 2560), (16, 530, 1536), (16, 2560, 9728), (1, 640, 25600),
                                   (5, 100, 768)])
def test_gemv_w4a8_other_group_sizes_bit_exact(orc, gs, m, n, k):
    g = synth.generator(100 + gs)
    w = _weight(n, k, gs, g)
    x = synth.activations(m, k, g, outliers=True)
    xq, xs = orc.quant_act_i8(G.bits(x))
    gacc_ref, y_ref = orc.linear_w4a8(xq, xs, w.packed.numpy(), w.scale.numpy(), k, gs, want_group_acc=True)
    w4, ws = G.w4_repack(w.packed.to(G.DEV), w.scale.to(G.DEV), k, gs)
    gacc, y = G.w4a8(w4, ws, G.dev(xq), G.dev(xs), k, gemm=False, gs=gs)
    assert (gacc.cpu().numpy() == gacc_ref).all()
    assert (G.bits(y) == y_ref).all()


@pytest.mark.parametrize("gs", [64, 256])
@pytest.mark.parametrize("m,n,k", [(128, 128, 256), (64, 256, 512), (100, 200, 768), (512, 2560, 2560),
                                   (300, 1000, 1280), (17, 64, 256), (1024, 640, 5120), (64, 5120, 25600)])
def test_gemm_w4a8_other_group_sizes_bit_exact(orc, gs, m, n, k):
    g = synth.generator(200 + gs)
    w = _weight(n, k, gs, g)
    x = synth.activations(m, k, g, outliers=True)
    xq, xs = orc.quant_act_i8(G.bits(x))
    want_acc = m * n * (k // gs) <= 1 << 24
    ref = orc.linear_w4a8(xq, xs, w.packed.numpy(), w.scale.numpy(), k, gs, want_group_acc=want_acc)
    w4, ws = G.w4_repack(w.packed.to(G.DEV), w.scale.to(G.DEV), k, gs)
    gacc, y = G.w4a8(w4, ws, G.dev(xq), G.dev(xs), k, gemm=True, want_acc=want_acc, gs=gs)
    if want_acc:
        assert (gacc.cpu().numpy() == ref[0]).all()
        assert (G.bits(y) == ref[1]).all()
        _, y2 = G.w4a8(w4, ws, G.dev(xq), G.dev(xs), k, gemm=True, want_acc=False, gs=gs)
        assert (y2.view(torch.int16) == y.view(torch.int16)).all()
    else:
        assert (G.bits(y) == ref[1]).all()


@pytest.mark.parametrize("gs", [64, 128, 256])
@pytest.mark.parametrize("k", [200, 1000, 2561, 25600 + 72])
@pytest.mark.parametrize("m", [1, 3, 16, 70])
def test_rows_that_are_not_whole_groups_through_the_c_abi(orc, gs, k, m):
    """K = 200 is the reference's own ragged example (tools/quant_disk_w4a8.py pads to 256): the
    device copy is padded to whole groups and steps, the quantised rows with zeros."""
    g = synth.generator(300 + gs + k)
    n = 96 if k > 20000 else 333
    w = _weight(n, k, gs, g)
    x = synth.activations(m, k, g, outliers=True)
    xq, xs = orc.quant_act_i8(G.bits(x))
    y_ref = orc.linear_w4a8(xq, xs, w.packed.numpy(), w.scale.numpy(), k, gs)[1]
    lib = _native.load()
    kd = int(lib.cmi_w4_device_k(k, gs))
    assert kd >= k and kd % gs == 0 and kd % 128 == 0 and kd - k < max(gs, 128)
    w4, ws = G.w4_repack(w.packed.to(G.DEV), w.scale.to(G.DEV), k, gs)
    # quantised rows, padded by the caller
    _, y = G.w4a8(w4, ws, G.dev(_padded(xq, kd)), G.dev(xs), kd, gemm=m > 16, want_acc=False, gs=gs)
    assert (G.bits(y) == y_ref).all()
    # bf16 rows: the entry pads for itself
    nbytes = int(lib.cmi_linear_workspace_bytes(m, kd))
    work = torch.full((nbytes,), 0xA5, dtype=torch.uint8, device=G.DEV)
    xd = x.to(G.DEV)
    y2 = torch.empty((m, n), dtype=torch.bfloat16, device=G.DEV)
    _native.check(lib.cmi_linear_w4a8_bf16(G.ptr(w4), G.ptr(ws), G.ptr(xd), G.ptr(y2), m, n, k, gs, G.ptr(work),
                                           nbytes, G.stream()), "linear_w4a8_bf16")
    assert (G.bits(y2) == y_ref).all()
    y3 = torch.empty((m, n), dtype=torch.bfloat16, device=G.DEV)
    _native.check(lib.cmi_linear_w4a8_bf16_static(G.ptr(w4), G.ptr(ws), G.ptr(xd), G.ptr(y3), m, n, k, gs,
                                                  G.stream()), "linear_w4a8_bf16_static")
    assert (G.bits(y3) == y_ref).all()


@pytest.mark.parametrize("gs,k", [(64, 2560), (256, 2560), (128, 200), (64, 200), (256, 1000), (64, 25600),
                                  (256, 25600)])
def test_table_entries_take_these_weights_natively(orc, monkeypatch, gs, k):
    """No int4 shape of these is left to the torch statement of the op: every entry runs the kernels
    (the dense fallback is made to fail) and carries the oracle's bits; the embedding gather too."""
    g = synth.generator(400 + gs + k)
    n = 320
    w = _weight(n, k, gs, g)
    wd = W4A8Weight(w.packed.to(G.DEV), w.scale.to(G.DEV), k=k, group_size=gs)

    def no_fallback(*_a, **_k):
        raise AssertionError("torch fallback taken")

    monkeypatch.setattr(backend, "_dense", no_fallback)
    for rows, fn in ((1, backend.linear), (4, backend.linear_m), (16, backend.linear_m_verify),
                     (40, backend.linear_prefill), (200, backend.linear_prefill)):
        x = synth.activations(rows, k, g)
        xq, xs = orc.quant_act_i8(G.bits(x))
        y_ref = orc.linear_w4a8(xq, xs, w.packed.numpy(), w.scale.numpy(), k, gs)[1]
        xd = x.to(G.DEV)
        y = fn(wd, xd[0] if rows == 1 else xd)
        assert (G.bits(y).reshape(rows, n) == y_ref).all(), (rows, fn.__name__)
    # producer -> projection in the reference's call order: padded rows are not handed over, same bits
    if k % 8 == 0:
        gain = synth.activations(1, k, g)[0].to(G.DEV).contiguous()
        x = synth.activations(3, k, g).to(G.DEV)
        h = backend.rms_norm(x, gain)
        assert (backend.linear_m(wd, h).view(torch.int16) == backend.linear_m(wd, h.clone()).view(torch.int16)).all()
    emb = TiedEmbedding(wd)
    ids = torch.tensor([0, n - 1, 17, 5], device=G.DEV)
    dense = orc.w4_dequant_f32(w.packed.numpy(), w.scale.numpy(), k, gs)
    assert (G.bits(emb.lookup(ids)) == orc.bf16_from_f32(dense[ids.cpu().numpy()])).all()
