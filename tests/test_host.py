"""CPU-side checks: the contract mirror, weight containers, caller dispatch, the
vendor declaration and the C-ABI library (load + symbols + argument checks; no
kernel is launched here)."""

from __future__ import annotations

import ctypes
import re
from pathlib import Path

import numpy as np
import pytest
import torch

from coffin_amd import _native, backend, contract, embed, gemv, synth
from coffin_amd.weights import (QWeight, W4A8Weight, dequantize_projection,
                                quantize_projection)

ROOT = Path(__file__).resolve().parent.parent


# ------------------------------------------------------------------ contract

def test_ops_table_names_and_errors():
    assert contract.Ops.NAMES == ("linear", "linear_m", "linear_m_verify", "linear_prefill",
                                  "kv_quant", "silu_mul", "silu_mul_quant", "rms_norm", "add_rms_norm")
    t = contract.Ops.from_mapping({"linear": lambda w, x: x})
    assert t.implemented() == ("linear",) and "kv_quant" in t.missing()
    with pytest.raises(ValueError, match="unknown op"):
        contract.Ops.from_mapping({"linear_fast": lambda: None})
    with pytest.raises(TypeError, match="callable or None"):
        contract.Ops(linear=3)


def test_vendor_spec_validation_and_declaration():
    from coffin_amd.vendors import mi355x
    spec = mi355x.SPEC
    spec.validate()
    assert spec.name == "mi355x" and spec.weight_layout == "nk" and spec.int8_weights
    assert spec.has_kernels and callable(spec.build_ops)
    assert spec.graph is True and spec.autotune is False     # decode is captured; nothing to tune
    assert spec.detection.namespace == "cuda" and spec.detection.hip
    assert all(m == m.lower() for m in spec.detection.name_markers)
    # the generic name every id-table-less AMD host reports must not be claimed
    assert not any(m in "amd radeon graphics" for m in spec.detection.name_markers)
    with pytest.raises(ValueError, match="weight_layout"):
        contract.VendorSpec(name="x", detection=contract.Detection("cuda"),
                            weight_layout="kk").validate()
    with pytest.raises(ValueError, match="has_kernels"):
        contract.VendorSpec(name="x", detection=contract.Detection("cuda"),
                            has_kernels=True).validate()
    if not torch.cuda.is_available():
        # no card: claim is "not mine" and build_ops degrades to an empty table
        assert contract.detect(spec.detection) == contract.CLAIM_NONE
        assert mi355x.build_ops().implemented() == ()


# ------------------------------------------------------------------- weights

def test_qweight_matches_oracle_and_surface(orc):
    g = synth.generator()
    w = synth.dense_weight(70, 300, g)
    q = QWeight.quantize(w, chunk_rows=32)                 # exercises the chunked path
    wq, scale = orc.qweight_quantize(w.numpy())
    assert (q.wq.numpy() == wq).all() and (q.scale.numpy() == scale).all()
    assert (q.n, q.k) == (70, 300) and q.wq.is_contiguous()
    assert q.nbytes() == 70 * 300 + 4 * 70
    d = q.dequant(torch.bfloat16)
    assert (d.view(torch.int16).numpy().view(np.uint16) == orc.qweight_dequant_bf16(wq, scale)).all()
    rows, s = q.rows(torch.tensor([3, 0]))
    assert (rows == q.wq[[3, 0]]).all() and (s == q.scale[[3, 0]]).all()
    z = QWeight.quantize(torch.zeros(2, 8))
    assert (z.wq == 0).all() and torch.isfinite(z.scale).all()


def test_qweight_from_kn_is_a_view_and_validates():
    # int8_weights.py:271-305: a [K, N] buffer wrapped without a copy; wq is the transposed view
    g = synth.generator()
    q = synth.int8_weight(12, 40, g)
    wt = q.wq.t().contiguous()
    v = QWeight.from_kn(wt, q.scale)
    assert (v.n, v.k) == (12, 40) and v.wq.stride() == (1, 12)
    assert v.wq.data_ptr() == wt.data_ptr() and (v.wq == q.wq).all()
    assert (v.dequant(torch.float32) == q.dequant(torch.float32)).all()
    with pytest.raises(ValueError, match="2-D int8"):
        QWeight.from_kn(wt.float(), q.scale)
    with pytest.raises(ValueError, match="1-D fp32"):
        QWeight.from_kn(wt, q.scale.double())
    with pytest.raises(ValueError, match="N = 12"):
        QWeight.from_kn(wt, q.scale[:5])
    with pytest.raises(ValueError, match="contiguous"):
        QWeight.from_kn(q.wq.t(), q.scale)


def test_w4_weight_matches_oracle_and_validates(orc):
    g = synth.generator()
    w = synth.dense_weight(20, 200, g)                     # K not a multiple of the group
    packed, scale = quantize_projection(w, 128)
    p2, s2 = orc.w4_quantize(w.numpy(), 128)
    assert (packed.numpy() == p2).all() and (scale.numpy() == s2).all()
    dense = dequantize_projection(packed, scale, k=200)
    assert (dense.numpy() == orc.w4_dequant_f32(p2, s2, 200, 128)).all()
    W = W4A8Weight(packed, scale, k=200)
    assert W.shape == (20, 200) and (W.to(torch.float32) == dense).all()
    assert (W.rows(torch.tensor([5, 1])) == dense[[5, 1]]).all()
    with pytest.raises(ValueError):
        W4A8Weight(packed.t(), scale, k=200)               # not contiguous [K/2, N]
    with pytest.raises(ValueError):
        W4A8Weight(packed, scale[:1].contiguous(), k=200)  # scale rows do not match groups
    with pytest.raises(ValueError):
        W4A8Weight(packed, scale, k=0)
    with pytest.raises(ValueError):
        quantize_projection(w[0])
    a = W4A8Weight.quantize(synth.dense_weight(6, 256, g))
    b = W4A8Weight.quantize(synth.dense_weight(10, 256, g))
    fused = W4A8Weight.cat_output([a, b])
    assert fused.n == 16 and (fused.to(torch.float32) ==
                              torch.cat([a.to(torch.float32), b.to(torch.float32)])).all()
    with pytest.raises(ValueError, match="share K"):
        W4A8Weight.cat_output([a, W4A8Weight.quantize(synth.dense_weight(4, 128, g))])


def test_synth_scales_are_fp16_representable():
    g = synth.generator()
    q = synth.int8_weight(32, 256, g)
    w4 = synth.int4_weight(16, 256, g)
    assert (q.scale.half().float() == q.scale).all()
    assert (w4.scale.half().float() == w4.scale).all()
    assert q.wq.abs().max() <= 127 and w4.packed.shape == (128, 16)
    x = synth.activations(4, 256, g, outliers=True)
    assert x.dtype == torch.bfloat16 and x.shape == (4, 256)
    assert sum(synth.gemv_bytes(1, n, k) for _, n, k in synth.DECODE_LAYER) == 101_101_568
    assert sum(synth.gemv_bytes(1, n, k) for _, n, k in synth.DECODE_LAYER_FUSED) == 101_086_208
    assert synth.gemv_bytes(1, *synth.LM_HEAD[1:]) == 389_569_024
    assert synth.w4_gemv_bytes(1, 9728, 2560) == 12_865_536
    assert synth.gemm_ops(2048, 9728, 2560) == 2 * 2048 * 9728 * 2560 == 102_005_473_280


# ------------------------------------------------------------ caller dispatch

class Recorder:
    """Fake op table: remembers which entry saw which row count."""

    def __init__(self):
        self.calls = []

    def _make(name):
        def fn(self, w, x):
            self.calls.append((name, tuple(x.shape)))
            n = w.shape[0] if isinstance(w, torch.Tensor) else w.n
            return torch.zeros((n,) if x.dim() == 1 else (x.shape[0], n))
        return fn

    linear = _make("linear")
    linear_m = _make("linear_m")
    linear_m_verify = _make("linear_m_verify")
    linear_prefill = _make("linear_prefill")


def test_gemv_regimes_follow_row_count():
    rec = Recorder()
    op = gemv.GEMV(torch.zeros(6, 4), ops=rec)
    assert (op.N, op.K) == (6, 4)
    assert op(torch.zeros(4)).shape == (6,)
    assert op.linear_m(torch.zeros(1, 4)).shape == (1, 6)      # one row -> linear on x[0]
    assert op.linear_m(torch.zeros(5, 4)).shape == (5, 6)
    assert op.linear_m_verify(torch.zeros(1, 4)).shape == (1, 6)
    op.linear_m_verify(torch.zeros(3, 4))
    assert op.prefill(torch.zeros(1, 4)).shape == (1, 6)
    op.prefill(torch.zeros(2, 4)); op.prefill(torch.zeros(8, 4)); op.prefill(torch.zeros(9, 4))
    assert rec.calls == [
        ("linear", (4,)), ("linear", (4,)), ("linear_m", (5, 4)), ("linear", (4,)),
        ("linear_m_verify", (3, 4)), ("linear", (4,)), ("linear_m", (2, 4)),
        ("linear_m", (8, 4)), ("linear_prefill", (9, 4))]


def test_gemv_group_fuses_and_splits():
    g = synth.generator()
    qa, qb = synth.int8_weight(6, 32, g), synth.int8_weight(10, 32, g)
    rec = Recorder()
    grp = gemv.GEMVGroup([qa, qb], ops=rec)
    assert grp.sizes == [6, 10] and grp.g.N == 16 and grp.g.q is not None
    assert (grp.g.w.wq[:6] == qa.wq).all() and (grp.g.w.scale[6:] == qb.scale).all()
    a, b = grp(torch.zeros(32))
    assert a.shape == (6,) and b.shape == (10,)
    a, b = grp.linear_m(torch.zeros(1, 32))
    assert a.shape == (1, 6) and b.shape == (1, 10)
    a, b = grp.prefill(torch.zeros(12, 32))
    assert a.shape == (12, 6) and b.shape == (12, 10)
    wa, wb = synth.int4_weight(4, 128, g), synth.int4_weight(8, 128, g)
    g4 = gemv.GEMVGroup([wa, wb], ops=rec)
    assert g4.g.q4 is not None and g4.g.N == 12
    with pytest.raises(ValueError, match="same weight format"):
        gemv.GEMVGroup([qa, wa], ops=rec)
    dense = gemv.GEMVGroup([torch.ones(2, 4), torch.zeros(3, 4)], ops=rec)
    assert dense.g.w.shape == (5, 4)


def test_tied_embedding_routes_lookup_and_projection():
    """Quantized storage is gathered by the native row gather (handed the weight object and the
    ids), plain storage by index_select; both projection entries go to the table; the
    reference's attribute surface (ops/embed.py:29-104) is kept."""
    g = synth.generator()
    ids = torch.tensor([5, 0, 39, 5, 17])
    seen = []

    def gather(w, i):
        seen.append((w, i))
        return torch.zeros((i.numel(), w.k), dtype=torch.bfloat16)

    q = synth.int8_weight(40, 96, g)
    emb = embed.TiedEmbedding(q, ops=Recorder(), gather=gather)
    assert emb.shape == (40, 96) and emb.q is q and emb.q4 is None and emb.w is None and emb.gemv.q is q
    assert emb.lookup(ids).shape == (5, 96) and seen[-1][0] is q and seen[-1][1] is ids
    w4 = synth.int4_weight(40, 256, g)
    emb4 = embed.TiedEmbedding(w4, ops=Recorder(), gather=gather)
    assert emb4.shape == (40, 256) and emb4.q4 is w4 and emb4.q is None and emb4.gemv.q4 is w4
    assert emb4.lookup(ids).shape == (5, 256) and seen[-1][0] is w4
    # no CPU path for quantized storage: the default gather refuses a CPU weight
    with pytest.raises(ValueError, match="GPU"):
        embed.TiedEmbedding(q, ops=Recorder()).lookup(ids)
    plain = torch.randn(12, 8, generator=g)
    embp = embed.TiedEmbedding(plain, ops=Recorder(), gather=gather)
    assert embp.shape == (12, 8) and embp.w is plain and len(seen) == 2
    assert (embp.lookup(torch.tensor([3, 3, 11])) == plain[[3, 3, 11]].to(torch.bfloat16)).all()
    rec = Recorder()
    proj = embed.TiedEmbedding(q, ops=rec, gather=gather)
    assert proj(torch.zeros(96)).shape == (40,) and proj.prefill(torch.zeros(9, 96)).shape == (9, 40)
    assert [c[0] for c in rec.calls] == ["linear", "linear_prefill"]


# --------------------------------------------------------------- adapters, CPU

def test_adapter_answers_dense_and_refuses_cpu_quantized():
    torch.manual_seed(1234)
    w, x = torch.randn(8, 6), torch.randn(6)
    # the reference's own dense assertion, tests/test_backends.py:451-457
    assert torch.allclose(backend.linear(w, x), x @ w.t(), rtol=1e-5, atol=1e-6)
    X = torch.randn(5, 6)
    for fn in (backend.linear_m, backend.linear_m_verify, backend.linear_prefill):
        assert torch.allclose(fn(w, X), X @ w.t(), rtol=1e-5, atol=1e-6)
    q = QWeight.quantize(w)
    with pytest.raises(ValueError, match="GPU"):
        backend.linear(q, x.bfloat16())
    assert set(backend.native_table()) == set(contract.Ops.NAMES)


def test_w4_operands_are_checked_before_any_address_reaches_a_kernel():
    """A duck-typed int4 weight hands raw addresses to the re-layout kernel; dtype, contiguity
    and shape must be refused on the host (the device check comes last and fails here too)."""
    from types import SimpleNamespace as NS
    k, n, gs = 256, 8, 128
    good = dict(packed=torch.zeros((k // 2, n), dtype=torch.uint8), scale=torch.ones((k // gs, n)),
                k=k, n=n, group_size=gs)
    for patch, match in (
            (dict(packed=torch.zeros((k // 2, n), dtype=torch.int8)), "uint8"),
            (dict(packed=torch.zeros((n, k // 2), dtype=torch.uint8).t()), "contiguous"),
            (dict(packed=torch.zeros((k // 2 - 1, n), dtype=torch.uint8)), "does not hold"),
            (dict(packed=torch.zeros((k // 2, n + 1), dtype=torch.uint8)), "does not hold"),
            (dict(scale=torch.ones((k // gs, n), dtype=torch.float16)), "fp32"),
            (dict(scale=torch.ones((n, k // gs)).t()), "contiguous"),
            (dict(scale=torch.ones((k // gs + 1, n))), "does not match"),
            (dict(), "GPU")):
        with pytest.raises(ValueError, match=match):
            backend._w4_check(NS(**{**good, **patch}))
    # shapes the kernels are not built for are answered by the torch statement of the op
    assert backend._kernels_take(NS(**good))
    assert backend._kernels_take(NS(**{**good, "group_size": 64})) and backend._kernels_take(NS(**{**good, "k": 192}))
    assert not backend._kernels_take(NS(**{**good, "group_size": 96}))
    assert not backend._kernels_take(NS(**{**good, "group_size": 32}))
    assert backend._kernels_take(NS(wq=torch.zeros((4, 32), dtype=torch.int8), scale=torch.ones(4)))
    assert not backend._kernels_take(NS(wq=torch.zeros((4, 24), dtype=torch.int8), scale=torch.ones(4)))


def test_scratch_never_moves_under_a_caller_and_the_record_pool_evicts_the_oldest(monkeypatch):
    """Scratch addresses may sit inside captured graphs: a block is outgrown, never freed or moved."""
    arena = backend._Arena("test")
    monkeypatch.setattr(backend, "_WORKSPACE", arena)
    backend._WORKSPACE_BYTES.clear()
    cpu = torch.device("cpu")
    a, nbytes = backend._scratch(1, 16, cpu)
    assert nbytes == 512                                   # 16 B of rows + 4 B of scale, 256 each
    first = arena.blocks[None]
    assert a == first.data_ptr() and first.numel() >= nbytes
    for rows in range(2, 40):                              # forty other shapes: same block, same address
        assert backend._scratch(rows, 16, cpu)[0] == a
    assert not arena.retired
    big, big_bytes = backend._scratch(4096, 4096, cpu)     # outgrows the block
    assert arena.retired == [first] and arena.blocks[None].numel() >= big_bytes
    assert first.data_ptr() == a                           # the outgrown block is still allocated
    assert backend._scratch(1, 16, cpu)[0] == big          # one block serves every shape
    backend._WORKSPACE_BYTES.clear()
    monkeypatch.setattr(backend, "_RECORDS_MAX", 2)
    backend._RECORDS.clear()
    g = synth.generator()
    ws = [synth.int8_weight(4, 32, g) for _ in range(3)]
    backend._make_record(ws[0])
    backend._make_record(ws[1])
    assert backend._lookup(ws[0]) is not None              # refreshed
    backend._make_record(ws[2])                            # evicts ws[1]
    assert backend._lookup(ws[1]) is None and backend._lookup(ws[0]) is not None
    backend._RECORDS.clear()


def test_weight_records_are_cached_weakly_and_revalidated():
    """The adapters resolve a weight's operand addresses once; the cached record must stop
    being trusted when the weight object swaps a tensor, and must not keep weights alive."""
    import gc
    import weakref
    g = synth.generator()
    q = synth.int8_weight(6, 32, g)
    rec = backend._make_record(q)
    assert backend._lookup(q) is rec and (rec.kind, rec.n, rec.k) == (8, 6, 32)
    assert rec.a == q.wq.data_ptr() and rec.b == q.scale.data_ptr()
    q.wq = q.wq.clone()                      # same object, new tensor: record is stale
    assert backend._lookup(q) is None
    rec2 = backend._make_record(q)
    assert backend._lookup(q) is rec2 and rec2.a == q.wq.data_ptr()
    alive = weakref.ref(q.wq)
    del q, rec, rec2
    gc.collect()
    assert alive() is None                   # the cache holds weak references only
    assert backend._lookup(torch.zeros(2, 2)) is None


def test_kv_quant_torch_branch_matches_oracle(orc):
    g = synth.generator()
    x = synth.activations(5, 96, g)
    out_q = torch.empty(5, 96, dtype=torch.int8)
    out_s = torch.empty(5, dtype=torch.float32)
    assert backend.kv_quant(x, out_q, out_s) is out_q
    q, s = orc.quant_act_i8(x.view(torch.int16).numpy().view(np.uint16))
    assert (out_q.numpy() == q).all() and (out_s.numpy() == s).all()
    with pytest.raises(ValueError):
        backend.kv_quant(x, out_q[:4], out_s)


# --------------------------------------------------------------------- C ABI

def _declared_symbols() -> list[str]:
    text = (ROOT / "include" / "coffin_mi355.h").read_text()
    return sorted(set(re.findall(r"\b(cmi_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _native.load()
    names = _declared_symbols()
    for name in names:
        assert getattr(lib, name) is not None
    assert (set(_native.SIGNATURES) | set(_native.OTHER_RESTYPES) | {"cmi_abi_version", "cmi_last_error"}
            == set(names))
    assert lib.cmi_abi_version() == _native.ABI_VERSION


def test_set_option_validates_names_and_values():
    lib = _native.load()
    for name, good, bad in ((b"gemm_tile", (64, 128, 192, 256, 320, 6464, 128192, 0), (1, 100, -1)),
                            (b"gemv_wholerow", (0, 1, -1), (2, -2)),
                            (b"w4_decode_waves", (4, 16, 0), (1, 8, -1)),
                            (b"w4_decode_chain", (1, 40108, 40116, 80216, 160416, 0), (2, 8, 16, 40132, 40316, 20116, -1))):
        for v in bad:
            assert lib.cmi_set_option(name, v) == _native.E_ARG
            assert "expected" in _native.last_error()
        for v in good:
            assert lib.cmi_set_option(name, v) == _native.OK
    assert lib.cmi_set_option(b"no_such_option", 0) == _native.E_ARG
    assert "unknown option" in _native.last_error()
    assert lib.cmi_set_option(None, 0) == _native.E_ARG


def test_entry_points_reject_bad_arguments_before_touching_the_device():
    lib = _native.load()
    null, one = ctypes.c_void_p(0), ctypes.c_void_p(256)
    assert lib.cmi_quant_act_i8(null, one, one, 1, 8, null) == _native.E_ARG
    assert "null pointer" in _native.last_error()
    assert lib.cmi_gemv_w8a16_mfma(one, one, one, one, 65, 8, 128, null) == _native.E_UNSUPPORTED
    assert lib.cmi_gemv_w8a16_mfma(one, one, one, one, 4, 8, 64, null) == _native.E_UNSUPPORTED
    assert "multiple of 128" in _native.last_error()
    assert lib.cmi_gemv_w8a16_mfma(null, one, one, one, 4, 8, 128, null) == _native.E_ARG
    assert lib.cmi_gemv_w8a16(one, one, one, one, 17, 8, 16, null) == _native.E_UNSUPPORTED
    assert "outside 1..16" in _native.last_error()
    assert lib.cmi_gemv_w8a16(one, one, one, one, 1, 8, 24, null) == _native.E_UNSUPPORTED
    assert lib.cmi_gemv_w8a16(ctypes.c_void_p(8), one, one, one, 1, 8, 16, null) == _native.E_ARG
    assert lib.cmi_gemv_w4a8(one, one, one, one, one, null, 1, 8, 256, 96, null) == _native.E_UNSUPPORTED
    assert "64, 128 and 256" in _native.last_error()
    assert lib.cmi_gemv_w4a8(one, one, one, one, one, null, 1, 8, 192, 128, null) == _native.E_UNSUPPORTED
    assert lib.cmi_gemv_w4a8(one, one, one, one, one, null, 1, 8, 320, 256, null) == _native.E_UNSUPPORTED
    assert lib.cmi_gemm_w8a8(one, one, one, one, one, null, 4, 8, 64, 4, null) == _native.E_ARG
    assert "ldy" in _native.last_error()
    assert lib.cmi_gemm_w4a8(one, one, one, one, one, null, 4, 8, 200, 128, null) == _native.E_UNSUPPORTED
    assert lib.cmi_gemm_w4a8(one, one, one, one, one, null, 4, 8, 256, 32, null) == _native.E_UNSUPPORTED
    assert lib.cmi_w4_repack(one, one, one, one, 8, 100, 96, null) == _native.E_UNSUPPORTED
    assert [lib.cmi_w4_device_k(k, gs) for k, gs in ((200, 128), (200, 64), (200, 256), (2560, 128), (2561, 64),
                                                      (300, 256), (128, 32), (0, 128))] == [256, 256, 256, 2560, 2688, 512, 0, 0]
    with pytest.raises(ValueError, match="cmi_gemv_w8a16"):
        _native.check(lib.cmi_gemv_w8a16(one, one, one, one, 0, 8, 16, null), "gemv")
