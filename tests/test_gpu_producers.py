"""Device parity of the fused producers of quantised activations (silu_mul_quant, rms_norm_i8,
add_rms_norm_i8), the embedding row gather and the one-call projections, through the C ABI.

Bit for bit against the oracle, and against the unfused sequence on the device (the op writing
bf16, then cmi_quant_act_i8 reading it back), which is the identity the fused entries owe their
callers (backends/protocol.py:274-278, backends/corex/kernels/norm.cu:240-247).
"""

from __future__ import annotations

import ctypes

import numpy as np
import pytest
import torch

from coffin_amd import _native, backend, synth
from coffin_amd.weights import QWeight, W4A8Weight
from tests import gpu_util as G

pytestmark = pytest.mark.gpu


def _silu_mul_quant(gate, up, out=None, want_q=True, want_out=True):
    """gate, up: bf16 device tensors [M,K] (any row pitch).  Returns (out, q, s)."""
    m, k = gate.shape
    if out is None and want_out:
        out = torch.empty((m, k), dtype=torch.bfloat16, device=G.DEV)
    q = torch.empty((m, k), dtype=torch.int8, device=G.DEV) if want_q else None
    s = torch.empty(m, dtype=torch.float32, device=G.DEV) if want_q else None
    ldo = out.stride(0) if out is not None else k
    _native.check(_native.load().cmi_silu_mul_quant(G.ptr(gate), G.ptr(up), G.ptr(out), G.ptr(q), G.ptr(s), m, k,
                                                    gate.stride(0), up.stride(0), ldo, G.stream()), "silu_mul_quant")
    return out, q, s


def test_silu_of_every_bf16_value_matches_the_oracle(orc):
    """silu is a function of 16 bits: all of them, against the oracle's table (which equals
    torch's F.silu on every finite bf16, see the CPU tests), with up = 1 so that the product
    narrowing is the identity, and with a second multiplier."""
    allb = np.arange(65536, dtype=np.uint16).reshape(64, 1024)
    gate = G.bf16_dev(allb)
    for mult in (1.0, -3.0):
        up = torch.full((64, 1024), mult, dtype=torch.bfloat16, device=G.DEV)
        out, _, _ = _silu_mul_quant(gate, up, want_q=False)
        want, _, _ = orc.silu_mul_quant(allb, G.bits(up), quant=False)
        finite = np.isfinite(orc.bf16_to_f32(allb)) & np.isfinite(orc.bf16_to_f32(want))
        assert finite.sum() > 65000
        assert (G.bits(out)[finite] == want[finite]).all()
        # non-finite gates stay non-finite or follow the oracle's limit values
        got_nf = orc.bf16_to_f32(G.bits(out))[~finite]
        want_nf = orc.bf16_to_f32(want)[~finite]
        assert (np.isnan(got_nf) == np.isnan(want_nf)).all()


@pytest.mark.parametrize("m,k", [(1, 9728), (16, 9728), (300, 2560), (5, 1001), (3, 8), (2, 25600),
                                 (7, 33000), (2048, 9728)])
def test_silu_mul_quant_bit_exact_and_equal_to_the_unfused_sequence(orc, m, k):
    g = synth.generator(1234, G.DEV)
    # the two halves of a fused gate_up projection: row pitch 2K
    gu = (torch.randn((m, 2 * k), generator=g, device=G.DEV) * 2.0).to(torch.bfloat16)
    gate, up = gu[:, :k], gu[:, k:]
    out, q, s = _silu_mul_quant(gate, up)
    small = m * k <= 4_000_000
    if small:
        out_ref, q_ref, s_ref = orc.silu_mul_quant(G.bits(gate.contiguous()), G.bits(up.contiguous()))
        assert (G.bits(out) == out_ref).all()
        assert (q.cpu().numpy() == q_ref).all() and (s.cpu().numpy() == s_ref).all()
    else:
        rows = [0, 1, m // 2, m - 1]
        out_ref, q_ref, s_ref = orc.silu_mul_quant(G.bits(gate[rows].contiguous()), G.bits(up[rows].contiguous()))
        assert (G.bits(out[rows]) == out_ref).all()
        assert (q[rows].cpu().numpy() == q_ref).all() and (s[rows].cpu().numpy() == s_ref).all()
    # silu_mul alone (no quantised outputs), then the stand-alone quantiser on what it stored
    out2, _, _ = _silu_mul_quant(gate, up, want_q=False)
    assert (out2.view(torch.int16) == out.view(torch.int16)).all()
    q2, s2 = G.quant(out2)
    assert (q2 == q).all() and (s2 == s).all()
    # quantised outputs only
    _, q3, s3 = _silu_mul_quant(gate, up, want_out=False)
    assert (q3 == q).all() and (s3 == s).all()
    # in place over the up half (the natural call: nothing reads `up` afterwards)
    gu2 = gu.clone()
    _, q4, s4 = _silu_mul_quant(gu2[:, :k], gu2[:, k:], out=gu2[:, k:])
    assert (gu2[:, k:].view(torch.int16) == out.view(torch.int16)).all() and (q4 == q).all() and (s4 == s).all()
    assert (gu2[:, :k].view(torch.int16) == gu[:, :k].view(torch.int16)).all()


def test_silu_mul_table_entries(orc):
    g = synth.generator(7, G.DEV)
    gate = torch.randn((9, 512), generator=g, device=G.DEV).to(torch.bfloat16)
    up = torch.randn((9, 512), generator=g, device=G.DEV).to(torch.bfloat16)
    out = torch.empty_like(gate)
    out_q = torch.empty((9, 512), dtype=torch.int8, device=G.DEV)
    out_s = torch.empty(9, dtype=torch.float32, device=G.DEV)
    assert backend.silu_mul_quant(gate, up, out, out_q, out_s) is out
    out_ref, q_ref, s_ref = orc.silu_mul_quant(G.bits(gate), G.bits(up))
    assert (G.bits(out) == out_ref).all() and (out_q.cpu().numpy() == q_ref).all()
    assert (out_s.cpu().numpy() == s_ref).all()
    plain = torch.empty_like(gate)
    assert backend.silu_mul(gate, up, plain) is plain and (G.bits(plain) == out_ref).all()
    one = torch.empty(512, dtype=torch.bfloat16, device=G.DEV)
    backend.silu_mul(gate[3], up[3], one)                                  # a 1-D row
    assert (G.bits(one) == out_ref[3]).all()
    with pytest.raises(ValueError):
        backend.silu_mul_quant(gate, up[:, :100], out, out_q, out_s)
    # any leading shape (the contract writes [...]): collapsible axes run the kernel, other layouts torch
    g3, u3, o3 = gate.view(3, 3, 512), up.view(3, 3, 512), torch.empty((3, 3, 512), dtype=torch.bfloat16, device=G.DEV)
    assert backend.silu_mul(g3, u3, o3) is o3 and (G.bits(o3).reshape(9, 512) == out_ref).all()
    gt = gate.t().contiguous().t()                                         # innermost stride is not 1
    ot = torch.empty_like(gate)
    backend.silu_mul(gt, up, ot)
    assert torch.allclose(ot.float(), (torch.nn.functional.silu(gt) * up).float())
    gs3 = gate.view(3, 3, 512)[:, :2]                                      # leading axes that do not collapse
    os3 = torch.empty((3, 2, 512), dtype=torch.bfloat16, device=G.DEV)
    backend.silu_mul(gs3, up.view(3, 3, 512)[:, :2], os3)
    assert torch.allclose(os3.float(), out.view(3, 3, 512)[:, :2].float(), rtol=2e-2, atol=1e-3)
    # fp32 inputs are answered by the torch statement of the op
    f = torch.empty((9, 512), device=G.DEV)
    backend.silu_mul(gate.float(), up.float(), f)
    assert torch.allclose(f, torch.nn.functional.silu(gate.float()) * up.float())
    assert "silu_mul_quant" in backend.native_table() and "silu_mul" in backend.native_table()


def _rms_norm_i8(x, w, add=None, eps=1e-6, want_y=True):
    m, n = x.shape
    y = torch.empty((m, n), dtype=torch.bfloat16, device=G.DEV) if want_y else None
    q = torch.empty((m, n), dtype=torch.int8, device=G.DEV)
    s = torch.empty(m, dtype=torch.float32, device=G.DEV)
    lib = _native.load()
    if add is None:
        rc = lib.cmi_rms_norm_i8(G.ptr(x), G.ptr(w), G.ptr(y), G.ptr(q), G.ptr(s), m, n, x.stride(0), n,
                                 ctypes.c_float(eps), G.stream())
    else:
        rc = lib.cmi_add_rms_norm_i8(G.ptr(x), G.ptr(add), G.ptr(w), G.ptr(y), G.ptr(q), G.ptr(s), m, n,
                                     x.stride(0), add.stride(0), n, ctypes.c_float(eps), G.stream())
    _native.check(rc, "rms_norm_i8")
    return y, q, s


@pytest.mark.parametrize("m,n", [(1, 2560), (16, 2560), (513, 2560), (7, 1000), (3, 4096), (2, 8), (4, 33000),
                                 (5, 1001), (2048, 2560)])
@pytest.mark.parametrize("with_add", [False, True])
def test_rms_norm_i8_bit_exact_and_equal_to_norm_then_quantiser(orc, m, n, with_add):
    g = synth.generator(1234, G.DEV)
    wide = (torch.randn((m, n + 64), generator=g, device=G.DEV) * 3.0).to(torch.bfloat16)
    x = wide[:, :n]                                                        # row pitch n + 64
    add = (torch.randn((m, n), generator=g, device=G.DEV)).to(torch.bfloat16) if with_add else None
    w = (1.0 + 0.1 * torch.randn(n, generator=g, device=G.DEV)).to(torch.bfloat16)
    x_before = x.contiguous().clone()
    pad_before = wide[:, n:].clone()
    y, q, s = _rms_norm_i8(x, w, add)
    y_ref, x_ref = orc.rms_norm(G.bits(x_before), G.bits(w), 1e-6, None if add is None else G.bits(add))
    assert (G.bits(x.contiguous()) == x_ref).all()                         # residual stream after the add
    assert (wide[:, n:].view(torch.int16) == pad_before.view(torch.int16)).all()   # beyond N: untouched
    assert (G.bits(y) == y_ref).all()
    q_ref, s_ref = orc.quant_act_i8(y_ref)
    assert (q.cpu().numpy() == q_ref).all() and (s.cpu().numpy() == s_ref).all()
    q2, s2 = G.quant(y)                                                    # the unfused sequence on the device
    assert (q2 == q).all() and (s2 == s).all()
    # quantised outputs only (x already holds the sum: plain norm of it)
    _, q3, s3 = _rms_norm_i8(x, w, None, want_y=False)
    assert (q3 == q).all() and (s3 == s).all()


def test_rms_norm_i8_adapter_and_special_rows(orc):
    g = synth.generator(5, G.DEV)
    x = torch.randn((6, 2560), generator=g, device=G.DEV).to(torch.bfloat16)
    x[1].zero_()                                                           # zero row: scale = 1/sqrt(eps), output 0
    x[2] = 0.5                                                             # constant row
    w = torch.ones(2560, device=G.DEV)                                     # fp32 gain: narrowed once, memoised
    out_q = torch.empty((6, 2560), dtype=torch.int8, device=G.DEV)
    out_s = torch.empty(6, dtype=torch.float32, device=G.DEV)
    y = torch.empty((6, 2560), dtype=torch.bfloat16, device=G.DEV)
    assert backend.rms_norm_i8(x, w, out_q, out_s, out=y) is out_q
    y_ref, _ = orc.rms_norm(G.bits(x), G.bits(w.to(torch.bfloat16)), 1e-6)
    assert (G.bits(y) == y_ref).all()
    assert (y[1].float() == 0).all() and (out_q[1] == 0).all() and float(out_s[1]) == np.float32(1e-5) / np.float32(127)
    assert (y[2].float() == 1.0).all() and (out_q[2] == 127).all()
    add = torch.randn((6, 2560), generator=g, device=G.DEV).to(torch.bfloat16)
    x2 = x.clone()
    backend.rms_norm_i8(x2, w, out_q, out_s, add=add, out=y)
    y_ref2, x_ref2 = orc.rms_norm(G.bits(x), G.bits(w.to(torch.bfloat16)), 1e-6, G.bits(add))
    assert (G.bits(x2) == x_ref2).all() and (G.bits(y) == y_ref2).all()
    with pytest.raises(ValueError):
        backend.rms_norm_i8(x.float(), w, out_q, out_s)


def test_rms_norm_table_entries_share_the_fused_arithmetic(orc):
    """rms_norm / add_rms_norm of the table followed by kv_quant give what rms_norm_i8 gives."""
    g = synth.generator(11, G.DEV)
    x = (torch.randn((7, 2560), generator=g, device=G.DEV) * 2).to(torch.bfloat16)
    add = torch.randn((7, 2560), generator=g, device=G.DEV).to(torch.bfloat16)
    w = (1 + 0.1 * torch.randn(2560, generator=g, device=G.DEV)).to(torch.bfloat16)
    y = backend.rms_norm(x, w)
    y_ref, _ = orc.rms_norm(G.bits(x), G.bits(w))
    assert (G.bits(y) == y_ref).all()
    q = torch.empty((7, 2560), dtype=torch.int8, device=G.DEV)
    s = torch.empty(7, dtype=torch.float32, device=G.DEV)
    backend.kv_quant(y, q, s)
    q2, s2 = torch.empty_like(q), torch.empty_like(s)
    backend.rms_norm_i8(x, w, q2, s2)
    assert (q == q2).all() and (s == s2).all()
    x2, out = x.clone(), torch.empty_like(x)
    assert backend.add_rms_norm(x2, add, w, out) is out
    y_ref2, x_ref2 = orc.rms_norm(G.bits(x), G.bits(w), add=G.bits(add))
    assert (G.bits(out) == y_ref2).all() and (G.bits(x2) == x_ref2).all()
    # fp32 rows take the torch statement of the reference
    xf = x.float()
    want = (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + 1e-6)) * w.float()
    assert torch.allclose(backend.rms_norm(xf, w.float()), want)
    assert "rms_norm" in backend.native_table() and "add_rms_norm" in backend.native_table()


# ------------------------------------------------------------- embedding rows

@pytest.mark.parametrize("n,k", [(3000, 2560), (151936, 2560), (50, 100), (64, 4096)])
def test_embed_rows_i8(orc, n, k):
    g = synth.generator(1234, G.DEV)
    q = synth.int8_weight(n, k, g)
    ids = torch.cat([torch.randint(0, n, (61,), generator=torch.Generator().manual_seed(1)),
                     torch.tensor([0, n - 1, 7, 7])]).to(G.DEV)
    rows = backend.embed_rows(q, ids)
    want = orc.qweight_dequant_bf16(q.wq[ids].cpu().numpy(), q.scale[ids].cpu().numpy())
    assert rows.shape == (65, k) and rows.dtype == torch.bfloat16 and (G.bits(rows) == want).all()
    # ids outside the vocabulary: NaN rows, the others unaffected
    bad = ids.clone()
    bad[3], bad[10] = n, -1
    rows2 = backend.embed_rows(q, bad)
    assert torch.isnan(rows2[3].float()).all() and torch.isnan(rows2[10].float()).all()
    keep = [i for i in range(65) if i not in (3, 10)]
    assert (rows2[keep].view(torch.int16) == rows[keep].view(torch.int16)).all()
    assert backend.embed_rows(q, ids[:0]).shape == (0, k)


@pytest.mark.parametrize("n,k", [(512, 2560), (151936, 2560), (40, 128), (100, 5120)])
def test_embed_rows_w4(orc, n, k):
    g = synth.generator(1234, G.DEV)
    w = synth.int4_weight(n, k, g)
    ids = torch.cat([torch.randint(0, n, (30,), generator=torch.Generator().manual_seed(2)),
                     torch.tensor([0, n - 1])]).to(G.DEV)
    rows = backend.embed_rows(w, ids.to(torch.int32))                      # other integer dtypes are widened
    dense = orc.w4_dequant_f32(w.packed[:, ids].contiguous().cpu().numpy(),
                               w.scale[:, ids].contiguous().cpu().numpy(), k, 128)
    assert (G.bits(rows) == orc.bf16_from_f32(dense)).all()
    bad = ids.clone()
    bad[0] = n + 5
    assert torch.isnan(backend.embed_rows(w, bad)[0].float()).all()


# ---------------------------------------------------- one-call projections

def _workspace(m, k):
    n = int(_native.load().cmi_linear_workspace_bytes(m, k))
    return torch.empty(n, dtype=torch.uint8, device=G.DEV), n


@pytest.mark.parametrize("m,n,k", [(1, 9728, 2560), (2, 9728, 2560), (1, 2560, 9728), (2, 2560, 9728),
                                   (3, 2560, 9728), (1, 9728, 5120), (1, 640, 25600), (16, 1024, 2560),
                                   (17, 300, 2560), (200, 512, 1280)])
def test_linear_w4a8_bf16_equals_quantiser_plus_kernels(orc, m, n, k):
    """Whatever route the entry takes (quantiser folded into the GEMV, or quantiser + GEMV, or
    quantiser + GEMM), output and workspace carry the bits of the separate calls."""
    g = synth.generator(1234)
    w = synth.int4_weight(n, k, g)
    x = synth.activations(m, k, g, outliers=True)
    xq_ref, xs_ref = orc.quant_act_i8(G.bits(x))
    _, y_ref = orc.linear_w4a8(xq_ref, xs_ref, w.packed.numpy(), w.scale.numpy(), k, 128)
    w4, ws = G.w4_repack(w.packed.to(G.DEV), w.scale.to(G.DEV), k)
    work, nbytes = _workspace(m, k)
    y = torch.empty((m, n), dtype=torch.bfloat16, device=G.DEV)
    _native.check(_native.load().cmi_linear_w4a8_bf16(G.ptr(w4), G.ptr(ws), G.ptr(x.to(G.DEV)), G.ptr(y), m, n, k, 128,
                                                      G.ptr(work), nbytes, G.stream()), "linear_w4a8_bf16")
    assert (G.bits(y) == y_ref).all()
    with pytest.raises(ValueError, match="workspace"):
        _native.check(_native.load().cmi_linear_w4a8_bf16(G.ptr(w4), G.ptr(ws), G.ptr(x.to(G.DEV)), G.ptr(y), m, n, k,
                                                          128, G.ptr(work), nbytes - 1, G.stream()), "short")


@pytest.mark.parametrize("m,n,k", [(64, 2560, 9728), (128, 2560, 9728), (33, 4096, 11008), (100, 1500, 10240),
                                   (20, 2560, 11008), (160, 2560, 9728), (250, 2500, 11008), (64, 1024, 2560),
                                   (256, 4096, 2560),
                                   # 257..1024 rows: 128 x 128 tiles in three, two, eight, five and four parts
                                   (300, 2560, 9728), (512, 2560, 9728), (640, 2560, 9728), (400, 1000, 8192),
                                   (700, 1024, 8192), (1024, 1024, 4096)])
def test_linear_w8a8_bf16_split_k_same_bits(orc, m, n, k):
    """With the larger workspace the entry may split K over the idle CUs (few tiles, many K steps:
    the first five shapes on the 64 x 64 tile, the next two on the 128 x 64 tile, the next two stay
    unsplit, the rest take or may take the 128 x 128 tile in parts): the partial sums are integers, so output
    and quantised rows are those of the small workspace and of the oracle, also with a row stride,
    and on a second call (the arrival counters are cleared by every call's quantiser launch)."""
    lib = _native.load()
    g = synth.generator(4321, G.DEV)
    q = synth.int8_weight(n, k, g)
    x = synth.activations(m, k, g, outliers=True)
    small, small_bytes = _workspace(m, k)
    big_bytes = int(lib.cmi_linear_w8a8_workspace_bytes(m, n, k))
    assert big_bytes >= small_bytes + 1024 + 8 * 2**20
    big = torch.full((big_bytes,), 0xA5, dtype=torch.uint8, device=G.DEV)   # counters start as garbage
    y_small = torch.zeros((m, n), dtype=torch.bfloat16, device=G.DEV)
    _native.check(lib.cmi_linear_w8a8_bf16(G.ptr(x), G.ptr(q.wq), G.ptr(q.scale), G.ptr(y_small), m, n, k, n,
                                           G.ptr(small), small_bytes, G.stream()), "linear_w8a8_bf16")
    for ldy in (n, n + 8):
        for _ in range(2):
            y = torch.zeros((m, ldy), dtype=torch.bfloat16, device=G.DEV)
            _native.check(lib.cmi_linear_w8a8_bf16(G.ptr(x), G.ptr(q.wq), G.ptr(q.scale), G.ptr(y), m, n, k, ldy,
                                                   G.ptr(big), big_bytes, G.stream()), "linear_w8a8_bf16")
            assert (y[:, :n].contiguous().view(torch.int16) == y_small.view(torch.int16)).all()
            assert (y[:, n:].float() == 0).all()
    rows = [0, m // 2, m - 1]
    xq_ref, xs_ref = orc.quant_act_i8(G.bits(x[rows]))
    _, y_ref = orc.gemm_w8a8(xq_ref, q.wq.cpu().numpy(), xs_ref, q.scale.cpu().numpy(), want_acc=False)
    assert (G.bits(y_small[rows].contiguous()) == y_ref).all()
    assert (big[:m * k].view(torch.int8).view(m, k) == small[:m * k].view(torch.int8).view(m, k)).all()


@pytest.mark.parametrize("m,n,k", [(64, 1024, 2560), (300, 4096, 2560), (5, 640, 1024), (2048, 4096, 2560)])
def test_linear_w8a8_bf16_equals_quantiser_plus_gemm(orc, m, n, k):
    g = synth.generator(1234, G.DEV)
    q = synth.int8_weight(n, k, g)
    x = synth.activations(m, k, g, outliers=True)
    work, nbytes = _workspace(m, k)
    y = torch.zeros((m, n + 16), dtype=torch.bfloat16, device=G.DEV)
    _native.check(_native.load().cmi_linear_w8a8_bf16(G.ptr(x), G.ptr(q.wq), G.ptr(q.scale), G.ptr(y), m, n, k, n + 16,
                                                      G.ptr(work), nbytes, G.stream()), "linear_w8a8_bf16")
    xq, xs = G.quant(x)
    _, y2 = G.gemm_w8a8(xq, q.wq, xs, q.scale, want_acc=False)
    assert (y[:, :n].contiguous().view(torch.int16) == y2.view(torch.int16)).all() and (y[:, n:].float() == 0).all()
    rows = [0, m // 2, m - 1]
    xq_ref, xs_ref = orc.quant_act_i8(G.bits(x[rows]))
    _, y_ref = orc.gemm_w8a8(xq_ref, q.wq.cpu().numpy(), xs_ref, q.scale.cpu().numpy(), want_acc=False)
    assert (G.bits(y[rows][:, :n].contiguous()) == y_ref).all()
    # the workspace holds the quantised rows and scales the kernel used
    assert (work[:m * k].view(torch.int8).view(m, k) == xq).all()
    off = (m * k + 255) // 256 * 256
    assert (work[off:off + 4 * m].view(torch.float32) == xs).all()
