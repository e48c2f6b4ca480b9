"""The table entries as coffin's callers use them, on the device.

Mirrors the reference's own assertions for this path (tests/test_backends.py:451-469:
``linear``, ``linear_m`` and ``linear_prefill`` agree with a matmul against the
dequantised weight, and dispatch happens on the storage type) and the contract
rules of backends/protocol.py:143-159,252-258.
"""

from __future__ import annotations

import numpy as np
import pytest
import torch

from coffin_amd import backend, gemv, synth
from coffin_amd.vendors import mi355x
from coffin_amd.weights import QWeight, W4A8Weight
from tests import gpu_util as G

pytestmark = pytest.mark.gpu

BF16_TOL = 2e-2      # tests/test_backends.py:54
FP32_TOL = 1e-5      # tests/test_backends.py:57


def _rel(got: torch.Tensor, ref: torch.Tensor) -> float:
    """max |got-ref| / max |ref| -- the reference's metric (tests/test_backends.py:74-80)."""
    return float((got.float() - ref.float()).abs().max() / ref.float().abs().max().clamp_min(1e-12))


def _q8(n, k, g):
    q = synth.int8_weight(n, k, g)
    return QWeight(q.wq.to(G.DEV), q.scale.to(G.DEV))


def _w4(n, k, g):
    w = synth.int4_weight(n, k, g)
    return W4A8Weight(w.packed.to(G.DEV), w.scale.to(G.DEV), k=k)


def test_vendor_builds_the_native_table():
    ops = mi355x.build_ops()
    assert set(ops.implemented()) == {"linear", "linear_m", "linear_m_verify", "linear_prefill",
                                      "kv_quant", "silu_mul", "silu_mul_quant", "rms_norm", "add_rms_norm"}
    from coffin_amd import contract
    # a board that reports its name is claimed by name; a host without the amdgpu id table
    # reports the generic "AMD Radeon Graphics", which is left to explicit selection
    name = torch.cuda.get_device_name(0).lower()
    named = any(m in name for m in mi355x.SPEC.detection.name_markers)
    assert contract.detect(mi355x.SPEC.detection) == (contract.CLAIM_NAME if named else contract.CLAIM_NONE)


def test_reference_linear_assertions_on_device():
    torch.manual_seed(1234)
    w, x = torch.randn(8, 6, device=G.DEV), torch.randn(6, device=G.DEV)
    assert _rel(backend.linear(w, x), x @ w.t()) < FP32_TOL
    X = torch.randn(5, 6, device=G.DEV)
    assert _rel(backend.linear_m(w, X), X @ w.t()) < FP32_TOL
    assert _rel(backend.linear_prefill(w, X), X @ w.t()) < FP32_TOL
    # int8 storage with fp32 activations: the torch statement, dispatch on storage type
    q = QWeight.quantize(w)
    dense = q.dequant(torch.float32)
    assert _rel(backend.linear(q, x), x @ dense.t()) < FP32_TOL
    assert _rel(backend.linear_m(q, X[:3]), X[:3] @ dense.t()) < FP32_TOL
    assert _rel(backend.linear_prefill(q, X[:3]), X[:3] @ dense.t()) < FP32_TOL


def test_kn_stored_weight_gives_the_bits_of_the_row_major_one():
    # QWeight.from_kn hands the adapter a transposed view; it answers from one private row-major copy
    g = synth.generator()
    q = _q8(1536, 2560, g)
    kn = QWeight.from_kn(q.wq.t().contiguous(), q.scale)
    for rows in (1, 4, 16, 96):
        x = synth.activations(rows, 2560, g).to(G.DEV)
        for fn in (backend.linear_m, backend.linear_m_verify, backend.linear_prefill):
            a, b = fn(q, x), fn(kn, x)
            assert (a.view(torch.int16) == b.view(torch.int16)).all(), (fn.__name__, rows)
    assert (backend.linear(q, x[0]).view(torch.int16) == backend.linear(kn, x[0]).view(torch.int16)).all()


@pytest.mark.parametrize("rows", [64, 100, 192, 300, 512])
def test_prefill_chunk_on_a_long_narrow_projection_splits_k_with_the_same_bits(rows):
    """64..512 rows of a down-projection shape (few tiles, many K steps): the adapter's workspace
    lets the fused entry split K; output is that of quantiser + cmi_gemm_w8a8 (which never splits)."""
    g = synth.generator()
    q = _q8(2560, 9728, g)
    x = synth.activations(rows, 9728, g).to(G.DEV)
    y = backend.linear_prefill(q, x)
    xq, xs = G.quant(x)
    _, want = G.gemm_w8a8(xq, q.wq.to(G.DEV), xs, q.scale.to(G.DEV), want_acc=False)
    assert (y.view(torch.int16) == want.view(torch.int16)).all()
    again = backend.linear_prefill(q, x)            # the arrival counters are cleared by every call
    assert (again.view(torch.int16) == want.view(torch.int16)).all()


@pytest.mark.parametrize("rows", [None, 1, 2, 8, 16, 17, 40])
def test_int8_entries_agree_with_dequant_matmul(rows):
    g = synth.generator()
    q = _q8(1536, 2560, g)
    x = synth.activations(rows or 1, 2560, g).to(G.DEV)
    x = x[0] if rows is None else x
    dense = q.dequant(torch.float32)
    ref = x.float() @ dense.t()
    for fn in (backend.linear, backend.linear_m, backend.linear_m_verify, backend.linear_prefill):
        y = fn(q, x)
        assert y.dtype == x.dtype and y.shape == ref.shape and y.is_contiguous()
        assert _rel(y, ref) < BF16_TOL
    # decode entries are bit-identical to each other whatever the batch (the static-batch contract)
    a, b = backend.linear(q, x), backend.linear_m(q, x)
    assert (a.view(torch.int16) == b.view(torch.int16)).all()
    if rows is not None and rows > 1:
        one = backend.linear(q, x[rows - 1])
        assert (one.view(torch.int16) == a[rows - 1].view(torch.int16)).all()
        # verify and short prefill chunks take the matrix-pipe GEMV from three rows up: the same
        # bits from both entries, independent of the rows that travel along (chunks of 16 included)
        v, p = backend.linear_m_verify(q, x), backend.linear_prefill(q, x)
        assert (v.view(torch.int16) == p.view(torch.int16)).all()
        if rows >= 3:
            first = backend.linear_m_verify(q, x[:3].contiguous())
            assert (first.view(torch.int16) == v[:3].view(torch.int16)).all()
        else:
            assert (v.view(torch.int16) == a.view(torch.int16)).all()


def test_batch_switch_moves_every_weight_only_call_to_the_matrix_pipe(monkeypatch):
    """COFFIN_AMD_BATCH_MFMA: one kernel family for linear, linear_m, verify and short prefill,
    so the static-batch contract (row r == single-row call) holds in that setting too."""
    g = synth.generator()
    q = _q8(512, 2560, g)
    x = synth.activations(8, 2560, g).to(G.DEV)
    exact = backend.linear_m(q, x)
    monkeypatch.setattr(backend, "BATCH_MFMA", True)
    fast = backend.linear_m(q, x)
    assert _rel(fast, exact.float()) < 1e-2
    for fn in (backend.linear, backend.linear_m_verify, backend.linear_prefill):
        assert (fn(q, x).view(torch.int16) == fast.view(torch.int16)).all()
    for r in (0, 3, 7):
        assert (backend.linear(q, x[r]).view(torch.int16) == fast[r].view(torch.int16)).all()
    two = backend.linear_m(q, x[:2].contiguous())
    assert (two.view(torch.int16) == fast[:2].view(torch.int16)).all()


def test_prefill_switches_to_w8a8_and_matches_the_oracle(orc):
    g = synth.generator()
    q = _q8(1024, 2560, g)
    x = synth.activations(200, 2560, g, outliers=True).to(G.DEV)
    y = backend.linear_prefill(q, x)
    xq, xs = orc.quant_act_i8(G.bits(x))
    _, y_ref = orc.gemm_w8a8(xq, q.wq.cpu().numpy(), xs, q.scale.cpu().numpy(), want_acc=False)
    assert (G.bits(y) == y_ref).all()
    # below the threshold prefill keeps weight-only numerics (matrix-pipe GEMV, as verify does)
    small = backend.linear_prefill(q, x[:63].contiguous())
    assert (small.view(torch.int16) == backend.linear_m_verify(q, x[:63].contiguous()).view(torch.int16)).all()
    assert _rel(small, backend.linear_m(q, x[:63].contiguous()).float()) < 1e-2
    # and the W8A8 answer is the unquantised product up to int8 activation noise (rows
    # with a x20 outlier have a 20x coarser step, hence the loose bound)
    assert _rel(y, x.float() @ q.dequant(torch.float32).t()) < 1e-1


@pytest.mark.parametrize("rows", [1, 2, 8, 16, 17, 40])
def test_verify_switch_takes_w8a8_and_matches_the_oracle(orc, monkeypatch, rows):
    """The opt-in W8A8 verify route (the counterpart of corex's COFFIN_COREX_W8A8_DP4A_VERIFY):
    from two rows up the answer is the W8A8 oracle's, bit for bit; one row and the switch
    being off keep the weight-only numerics."""
    g = synth.generator()
    q = _q8(1536, 2560, g)
    x = synth.activations(rows, 2560, g, outliers=True).to(G.DEV)
    off = backend.linear_m_verify(q, x)
    if rows < 3:
        assert (off.view(torch.int16) == backend.linear_m(q, x).view(torch.int16)).all()
    else:                                    # weight-only either way, summation order differs
        assert _rel(off, backend.linear_m(q, x).float()) < 1e-2
    monkeypatch.setattr(backend, "W8A8_VERIFY", True)
    on = backend.linear_m_verify(q, x)
    assert on.shape == off.shape and on.dtype == off.dtype and on.is_contiguous()
    if rows < 2:
        assert (on.view(torch.int16) == off.view(torch.int16)).all()
        return
    xq, xs = orc.quant_act_i8(G.bits(x))
    _, y_ref = orc.gemm_w8a8(xq, q.wq.cpu().numpy(), xs, q.scale.cpu().numpy(), want_acc=False)
    assert (G.bits(on) == y_ref).all()
    # int4 weights and plain tensors are not affected by the switch
    w = _w4(256, 2560, g)
    assert (backend.linear_m_verify(w, x).view(torch.int16) == backend.linear_m(w, x).view(torch.int16)).all()


@pytest.mark.parametrize("rows", [None, 1, 4, 16, 17, 64, 300])
def test_w4_entries_match_the_oracle_bit_for_bit(orc, rows):
    g = synth.generator()
    w = _w4(768, 2560, g)
    x = synth.activations(rows or 1, 2560, g).to(G.DEV)
    xq, xs = orc.quant_act_i8(G.bits(x))
    _, y_ref = orc.linear_w4a8(xq, xs, w.packed.cpu().numpy(), w.scale.cpu().numpy(), 2560, 128)
    arg = x[0] if rows is None else x
    for fn in (backend.linear, backend.linear_m, backend.linear_m_verify, backend.linear_prefill):
        y = fn(w, arg)
        assert y.dtype == torch.bfloat16
        assert y.shape == ((768,) if rows is None else (x.shape[0], 768))
        assert (G.bits(y).reshape(y_ref.shape) == y_ref).all()
    # unquantised-activation reference (what the torch backend computes) is close
    ref = x.float() @ w.to(torch.float32).t()
    assert _rel(y.reshape(ref.shape), ref) < 5e-2


@pytest.mark.parametrize("n,k", [(8192, 5120), (1024, 5120), (512, 9728)])
def test_w4_long_rows_take_the_same_bits_on_every_route(orc, n, k):
    # rows beyond 4096 leave the dot-product kernel: matrix-pipe GEMV, one launch or two
    # (quantiser + GEMV) depending on the number of workgroups; the bits are the oracle's either way
    g = synth.generator()
    w = _w4(n, k, g)
    for rows in (1, 2, 3):
        x = synth.activations(rows, k, g).to(G.DEV)
        xq, xs = orc.quant_act_i8(G.bits(x))
        _, y_ref = orc.linear_w4a8(xq, xs, w.packed.cpu().numpy(), w.scale.cpu().numpy(), k, 128)
        for fn in (backend.linear_m, backend.linear_m_verify):
            assert (G.bits(fn(w, x)) == y_ref).all(), (fn.__name__, rows)
        assert (G.bits(backend.linear(w, x[0])) == y_ref[0]).all()


def test_tied_embedding_on_the_gpu(orc):
    """Row gather on the device gives the oracle's dequantised rows; the projection is the
    native GEMV on the same weight (ops/embed.py:64-104)."""
    from coffin_amd import embed
    g = synth.generator()
    q = _q8(3000, 2560, g)
    emb = embed.TiedEmbedding(q)
    ids = torch.tensor([7, 2999, 0, 7, 1234], device=G.DEV)
    rows = emb.lookup(ids)
    want = orc.qweight_dequant_bf16(q.wq.cpu().numpy(), q.scale.cpu().numpy())[ids.cpu().numpy()]
    assert rows.dtype == torch.bfloat16 and (G.bits(rows) == want).all()
    x = synth.activations(1, 2560, g).to(G.DEV)[0]
    assert (emb(x).view(torch.int16) == backend.linear(q, x).view(torch.int16)).all()
    w = _w4(512, 2560, g)
    emb4 = embed.TiedEmbedding(w)
    dense = orc.w4_dequant_f32(w.packed.cpu().numpy(), w.scale.cpu().numpy(), 2560)
    ids4 = torch.tensor([0, 511, 100], device=G.DEV)
    assert (G.bits(emb4.lookup(ids4)) == orc.bf16_from_f32(dense[ids4.cpu().numpy()])).all()
    assert (emb4(x).view(torch.int16) == backend.linear(w, x).view(torch.int16)).all()


def test_adapters_replay_inside_a_captured_graph():
    """A decode step is captured once and replayed (the callers' engines do that): every
    replay, with fresh activation contents in the same buffers, must equal the eager answer."""
    g = synth.generator()
    q, w = _q8(1024, 2560, g), _w4(768, 2560, g)
    x1 = synth.activations(1, 2560, g).to(G.DEV)[0].contiguous()
    x16 = synth.activations(16, 2560, g).to(G.DEV)
    x100 = synth.activations(100, 2560, g).to(G.DEV)

    def step():
        return (backend.linear(q, x1), backend.linear(w, x1), backend.linear_m(q, x16),
                backend.linear_m(w, x16), backend.linear_prefill(q, x100), backend.linear_prefill(w, x100))

    step()                                   # warm-up: lazy library state, scratch buffers
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
        with torch.cuda.graph(graph, stream=side):
            outs = step()
    torch.cuda.current_stream().wait_stream(side)
    for seed in (1, 2, 3):
        gg = synth.generator(seed)
        x1.copy_(synth.activations(1, 2560, gg)[0])
        x16.copy_(synth.activations(16, 2560, gg))
        x100.copy_(synth.activations(100, 2560, gg))
        graph.replay()
        torch.cuda.synchronize()
        for got, want in zip(outs, step()):
            assert (got.view(torch.int16) == want.view(torch.int16)).all()


def test_first_use_of_a_weight_inside_capture_is_refused():
    """The SPEC declares decode capturable; what capture cannot hold is a weight's first use (its
    private re-laid-out copy would be allocated and rebuilt inside the graph).  The adapter says
    so before anything is launched, and the same weight works once it has been touched eagerly."""
    from coffin_amd.vendors import mi355x
    assert mi355x.SPEC.graph is True
    g = synth.generator()
    w = _w4(256, 512, g)
    x = synth.activations(1, 512, g).to(G.DEV)[0].contiguous()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with pytest.raises(RuntimeError, match="inside graph capture"):
            with torch.cuda.graph(graph, stream=side):
                _kept = x * 1                # so the abandoned graph is not an empty one
                backend.linear(w, x)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    want = backend.linear(w, x)
    graph2 = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph2, stream=side):
            got = backend.linear(w, x)
    torch.cuda.current_stream().wait_stream(side)
    graph2.replay()
    torch.cuda.synchronize()
    assert (got.view(torch.int16) == want.view(torch.int16)).all()


def test_outputs_are_fresh_and_inputs_untouched():
    g = synth.generator()
    q, w = _q8(256, 512, g), _w4(256, 512, g)
    x = synth.activations(3, 512, g).to(G.DEV)
    keep = x.clone()
    wq_keep, packed_keep = q.wq.clone(), w.packed.clone()
    a, b = backend.linear(q, x), backend.linear(q, x)
    c, d = backend.linear(w, x), backend.linear(w, x)
    assert a.data_ptr() != b.data_ptr() and c.data_ptr() != d.data_ptr()
    assert (x == keep).all() and (q.wq == wq_keep).all() and (w.packed == packed_keep).all()
    # the re-laid-out int4 copy is made once per weight
    from coffin_amd.backend import _w4_operands
    assert _w4_operands(w)[0].data_ptr() == _w4_operands(w)[0].data_ptr()


def test_shape_and_device_errors():
    g = synth.generator()
    q, w = _q8(64, 128, g), _w4(64, 128, g)
    bad = torch.zeros(3, 64, dtype=torch.bfloat16, device=G.DEV)
    for weight in (q, w):
        with pytest.raises(ValueError):
            backend.linear(weight, bad)
        with pytest.raises(ValueError):
            backend.linear(weight, torch.zeros(2, 3, 128, dtype=torch.bfloat16, device=G.DEV))
        with pytest.raises(ValueError, match="GPU"):
            backend.linear(weight, torch.zeros(128, dtype=torch.bfloat16))
    odd = W4A8Weight(torch.full((128, 8), 0x88, dtype=torch.uint8, device=G.DEV),
                     torch.ones((4, 8), device=G.DEV), k=256, group_size=64)
    # a group size the kernels are not built for is answered by the torch statement of the op
    # (backends/reference/__init__.py:93-95), as the reference's adapter falls back for shapes its
    # kernels refuse
    xo = synth.activations(3, 256, g).to(G.DEV)
    want = torch.nn.functional.linear(xo, odd.to(torch.bfloat16))
    assert (backend.linear_m(odd, xo).view(torch.int16) == want.view(torch.int16)).all()
    empty = backend.linear_m(q, torch.zeros(0, 128, dtype=torch.bfloat16, device=G.DEV))
    assert empty.shape == (0, 64)


def test_kv_quant_writes_through_caller_buffers(orc):
    g = synth.generator()
    x = synth.activations(9, 256, g).to(G.DEV)
    out_q = torch.zeros(9, 256, dtype=torch.int8, device=G.DEV)
    out_s = torch.zeros(9, dtype=torch.float32, device=G.DEV)
    qp, sp = out_q.data_ptr(), out_s.data_ptr()
    assert backend.kv_quant(x, out_q, out_s) is out_q
    assert (out_q.data_ptr(), out_s.data_ptr()) == (qp, sp)
    q, s = orc.quant_act_i8(G.bits(x))
    assert (out_q.cpu().numpy() == q).all() and (out_s.cpu().numpy() == s).all()
    # fp32 rows take the torch statement of the same formula
    xf = x.float()
    backend.kv_quant(xf, out_q, out_s)
    assert (out_q.cpu().numpy() == q).all()


@pytest.mark.parametrize("rows", [1, 3, 16, 70, 200])
def test_quantised_rows_feed_the_projection_behind_a_fused_producer(rows):
    """rms_norm_i8 / silu_mul_quant write int8 rows + scales; linear_quantized consumes them.  The
    result carries the bits of the bf16 route (norm written as bf16, then the projection that
    quantises for itself): W4A8 at every row count, W8A8 through linear_prefill from 64 rows."""
    g = synth.generator(11)
    k, n = 2560, 1024
    x = synth.activations(rows, k, g).to(G.DEV)
    gain = synth.activations(1, k, g)[0].to(G.DEV).contiguous()
    xq = torch.empty((rows, k), dtype=torch.int8, device=G.DEV)
    xs = torch.empty(rows, dtype=torch.float32, device=G.DEV)
    y_bf16 = torch.empty_like(x)
    backend.rms_norm_i8(x, gain, xq, xs, out=y_bf16)
    w4, q8 = _w4(n, k, g), _q8(n, k, g)
    got4 = backend.linear_quantized(w4, xq, xs)
    want4 = backend.linear(w4, y_bf16)
    assert (got4.view(torch.int16) == want4.view(torch.int16)).all()
    got8 = backend.linear_quantized(q8, xq, xs)
    if rows >= 64:
        want8 = backend.linear_prefill(q8, y_bf16)
        assert (got8.view(torch.int16) == want8.view(torch.int16)).all()
    else:
        # below 64 rows linear_prefill stays weight-only: compare with quantiser + W8A8 run separately
        q2, s2 = torch.empty_like(xq), torch.empty_like(xs)
        backend.kv_quant(y_bf16, q2, s2)
        assert (q2 == xq).all() and (s2.view(torch.int32) == xs.view(torch.int32)).all()
        assert (backend.linear_quantized(q8, q2, s2).view(torch.int16) == got8.view(torch.int16)).all()
    # the SwiGLU product in front of a down projection
    gu = synth.activations(rows, 2 * k, g).to(G.DEV)
    prod = torch.empty((rows, k), dtype=torch.bfloat16, device=G.DEV)
    backend.silu_mul_quant(gu[:, :k], gu[:, k:], prod, xq, xs)
    assert (backend.linear_quantized(w4, xq, xs).view(torch.int16) == backend.linear(w4, prod).view(torch.int16)).all()
    with pytest.raises(ValueError):
        backend.linear_quantized(w4, xq[:, :128], xs)
    with pytest.raises(ValueError):
        backend.linear_quantized(w4, xq.to(torch.int16), xs)


def test_gemv_objects_on_device():
    g = synth.generator()
    qa, qb = _q8(512, 2560, g), _q8(256, 2560, g)
    x = synth.activations(4, 2560, g).to(G.DEV)
    single_a, single_b = gemv.GEMV(qa), gemv.GEMV(qb)
    group = gemv.GEMVGroup([qa, qb])
    fa, fb = group(x[0])
    assert (fa.view(torch.int16) == single_a(x[0]).view(torch.int16)).all()
    assert (fb.view(torch.int16) == single_b(x[0]).view(torch.int16)).all()
    ma, mb = group.linear_m(x)
    assert ma.shape == (4, 512) and mb.shape == (4, 256)
    assert (ma.view(torch.int16) == single_a.linear_m(x).view(torch.int16)).all()
    pa, _ = group.prefill(x[:1])
    assert pa.shape == (1, 512)
    wa, wb = _w4(256, 2560, g), _w4(128, 2560, g)
    g4 = gemv.GEMVGroup([wa, wb])
    ya, yb = g4(x[0])
    assert (ya.view(torch.int16) == gemv.GEMV(wa)(x[0]).view(torch.int16)).all()
    assert (yb.view(torch.int16) == gemv.GEMV(wb)(x[0]).view(torch.int16)).all()


def test_launches_follow_the_current_stream():
    g = synth.generator()
    q = _q8(512, 2560, g)
    x = synth.activations(1, 2560, g).to(G.DEV)
    want = backend.linear(q, x)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        got = backend.linear(q, x)
    side.synchronize()
    assert (got.view(torch.int16) == want.view(torch.int16)).all()


def test_pre_quantised_directory_feeds_the_kernels(tmp_path, orc):
    """A coffin-int8-kn-v1 / coffin-w4a8-kn-v1 directory read straight to the GPU gives weights the
    adapters take as they are: same bits as the weights the directory was written from."""
    import json
    from safetensors.torch import save_file
    from coffin_amd import quantized_load as ql
    g = synth.generator()
    q = synth.int8_weight(640, 2560, g)
    key = "model.language_model.layers.0.mlp.down_proj.weight"
    save_file({key: q.wq.t().contiguous(), key + "#scale": q.scale}, str(tmp_path / "quant-00001-of-00001.safetensors"))
    (tmp_path / ql.INDEX_NAME).write_text(json.dumps({"format": ql.FORMAT_INT8, "weight_dtype": "bfloat16", "tensors": {
        key: {"kind": "q8", "shape": [2560, 640], "scale_key": key + "#scale", "shard": "quant-00001-of-00001.safetensors"}}}))
    w = ql.load(tmp_path, device=G.DEV)[key]
    assert w.wq.device.type == "cuda" and w.wq.is_contiguous() and tuple(w.wq.shape) == (640, 2560)
    x = synth.activations(3, 2560, g).to(G.DEV)
    ref = QWeight(q.wq.to(G.DEV), q.scale.to(G.DEV))
    assert (backend.linear_m(w, x).view(torch.int16) == backend.linear_m(ref, x).view(torch.int16)).all()
    assert (backend.linear(w, x[0]).view(torch.int16) == backend.linear(ref, x[0]).view(torch.int16)).all()


# ------------------------------------------------ quantised rows handed forward by the producers

def _count_quantised_routes(monkeypatch):
    calls = []
    real = backend._rows_quantised

    def spy(rec, xq, xs, rows, out, stream):
        calls.append((rec.kind, rows))
        return real(rec, xq, xs, rows, out, stream)

    monkeypatch.setattr(backend, "_rows_quantised", spy)
    return calls


@pytest.mark.parametrize("rows", [1, 2, 16, 70, 300, 1100])
def test_table_entry_sequence_hands_quantised_rows_to_the_projection(monkeypatch, rows):
    """The reference's own call sequence -- ``rms_norm`` then ``linear``, ``add_rms_norm`` then
    ``linear``, ``silu_mul`` then ``linear`` (ops/norm.py:87,135, models/qwen35/blocks.py:69) -- runs
    the integer kernels on the rows the producer quantised, with the bits of the route that
    quantises the bf16 rows again."""
    g = synth.generator(5)
    k, n = 2560, 1536
    w4, q8 = _w4(n, k, g), _q8(n, k, g)
    wd = _w4(k, 2 * k, g)                      # a "down" projection for the SwiGLU product
    x = synth.activations(rows, k, g).to(G.DEV)
    gain = synth.activations(1, k, g)[0].to(G.DEV).contiguous()
    add = synth.activations(rows, k, g).to(G.DEV)
    gu = synth.activations(rows, 4 * k, g).to(G.DEV)

    def sequence():
        outs = []
        h = backend.rms_norm(x, gain)
        hv = h.view(-1) if rows == 1 else h.view(rows, k)          # ops/norm.py:87 hands out a view
        outs.append(backend.linear(w4, hv))
        outs.append(backend.linear_prefill(w4, h))                 # a second consumer of the same rows
        outs.append(backend.linear_prefill(q8, h))                 # W8A8 from 64 rows, weight-only below
        res = x.clone()
        nxt = torch.empty_like(res)
        backend.add_rms_norm(res, add, gain, nxt)
        outs.append(backend.linear_m(w4, nxt) if rows > 1 else backend.linear(w4, nxt[0]))
        gate, up = gu[:, :2 * k], gu[:, 2 * k:]                    # halves of a fused gate_up output
        prod = backend.silu_mul(gate, up, up)
        outs.append(backend.linear_prefill(wd, prod))
        return outs

    gu0 = gu.clone()                           # silu_mul overwrites the `up` half in place
    monkeypatch.setattr(backend, "HANDOVER_MIN_ROWS", 1)   # the mechanism at every row count (default: from 2 rows)
    monkeypatch.setattr(backend, "HANDOVER", False)
    want = sequence()
    monkeypatch.setattr(backend, "HANDOVER", True)
    calls = _count_quantised_routes(monkeypatch)
    gu.copy_(gu0)
    got = sequence()
    for i, (a, b) in enumerate(zip(got, want)):
        assert (a.view(torch.int16) == b.view(torch.int16)).all(), i
    kinds = [c[0] for c in calls]
    assert kinds.count(4) == 4                                     # every int4 projection took the handed rows
    assert kinds.count(8) == (1 if rows >= 64 and not backend._splits_k(rows, n, k, x.device) else 0)


def test_handed_rows_are_not_trusted_after_the_tensor_changed(monkeypatch):
    g = synth.generator(6)
    k, n = 2560, 1024
    w4 = _w4(n, k, g)
    x = synth.activations(4, k, g).to(G.DEV)
    gain = synth.activations(1, k, g)[0].to(G.DEV).contiguous()
    backend.linear(w4, x)                                          # a quantising consumer has been seen
    calls = _count_quantised_routes(monkeypatch)

    def fresh(t):                                                  # the same values in memory of their own
        return backend.linear_m(w4, t.clone())

    h = backend.rms_norm(x, gain)
    assert (backend.linear_m(w4, h).view(torch.int16) == fresh(h).view(torch.int16)).all()
    assert len(calls) == 1
    h.mul_(2)                                                      # torch writes announce themselves
    assert (backend.linear_m(w4, h).view(torch.int16) == fresh(h).view(torch.int16)).all()
    assert len(calls) == 1
    h = backend.rms_norm(x, gain)
    other = h.clone()                                              # same values, other memory: not the handed tensor
    backend.linear_m(w4, other)
    assert len(calls) == 1
    backend.linear_m(w4, h[:2])                                    # fewer rows than were handed
    assert len(calls) == 1
    backend.linear_m(w4, h)
    assert len(calls) == 2
    # one of this backend's own kernels writes into the tensor: the entry goes
    gate = synth.activations(4, k, g).to(G.DEV)
    q = torch.empty((4, k), dtype=torch.int8, device=G.DEV)
    s = torch.empty(4, dtype=torch.float32, device=G.DEV)
    h = backend.rms_norm(x, gain)
    backend.silu_mul_quant(gate, x, h, q, s)
    assert (backend.linear_m(w4, h).view(torch.int16) == fresh(h).view(torch.int16)).all()
    assert len(calls) == 2
    # a single row is not handed by default (quantising costs the producer what it saves the projection)
    one = backend.rms_norm(x[:1], gain)
    backend.linear(w4, one[0])
    assert len(calls) == 2 and backend._HANDED is None
    # switched off, nothing is handed
    backend.configure(handover=False)
    try:
        h = backend.rms_norm(x, gain)
        backend.linear_m(w4, h)
        assert len(calls) == 2 and backend._HANDED is None
    finally:
        backend.configure(handover=True)


def test_handed_rows_inside_a_captured_graph_and_not_across_its_edge(monkeypatch):
    """Producer and consumer recorded into one capture replay together (fresh inputs, same bits as
    eager); a consumer recorded into a capture does not read rows an eager producer left."""
    g = synth.generator(8)
    k, n = 2560, 1024
    w4 = _w4(n, k, g)
    gain = synth.activations(1, k, g)[0].to(G.DEV).contiguous()
    x = synth.activations(2, k, g).to(G.DEV)
    gu = synth.activations(2, 2 * k, g).to(G.DEV)

    def step():
        a = backend.linear_m(w4, backend.rms_norm(x, gain))
        up = gu[:, k:].clone()
        b = backend.linear_m(w4, backend.silu_mul(gu[:, :k], up, up))
        return a, b

    step()
    torch.cuda.synchronize()
    calls = _count_quantised_routes(monkeypatch)
    eager_h = backend.rms_norm(x, gain)                            # handed eagerly, consumed under capture: refused
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            crossing = backend.linear_m(w4, eager_h)
            assert len(calls) == 0
            outs = step()
            assert len(calls) == 2
    torch.cuda.current_stream().wait_stream(side)
    for seed in (1, 2, 3):
        gg = synth.generator(seed)
        x.copy_(synth.activations(2, k, gg))
        gu.copy_(synth.activations(2, 2 * k, gg))
        junk = torch.randn(1 << 20, device=G.DEV)                  # eager work between the replays
        del junk
        graph.replay()
        torch.cuda.synchronize()
        backend.configure(handover=False)
        try:
            want = step()
        finally:
            backend.configure(handover=True)
        for a, b in zip(outs, want):
            assert (a.view(torch.int16) == b.view(torch.int16)).all()
    assert crossing.shape == (2, n)


def test_scratch_captured_by_a_graph_survives_forty_other_shapes():
    """A captured step holds raw addresses of the adapter's scratch; calls with many other shapes
    (which once evicted and freed it) must leave the replay's bits alone."""
    g = synth.generator(9)
    k, n = 2560, 1024
    w4, q8 = _w4(n, k, g), _q8(n, k, g)
    x4 = synth.activations(4, k, g).to(G.DEV)
    x80 = synth.activations(80, k, g).to(G.DEV)

    def step():
        return backend.linear_m(w4, x4), backend.linear_prefill(q8, x80), backend.linear_prefill(w4, x80)

    step()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            outs = step()
    torch.cuda.current_stream().wait_stream(side)
    hold = []
    for rows in range(65, 65 + 44):                                 # other prefill lengths, growing scratch
        xs = synth.activations(rows * 8, k, synth.generator(rows)).to(G.DEV)
        backend.linear_prefill(q8, xs)
        backend.linear_prefill(w4, xs)
        hold.append(torch.full((1 << 18,), float(rows), device=G.DEV))   # memory a freed block would be reused for
    torch.cuda.synchronize()
    gg = synth.generator(77)
    x4.copy_(synth.activations(4, k, gg))
    x80.copy_(synth.activations(80, k, gg))
    graph.replay()
    torch.cuda.synchronize()
    for a, b in zip(outs, step()):
        assert (a.view(torch.int16) == b.view(torch.int16)).all()
    for rows, t in zip(range(65, 65 + 44), hold):
        assert bool((t == float(rows)).all())


def test_family_is_a_property_of_the_weight_or_the_process():
    """Static-batch decode is owed "row r == single-row call" (models/qwen35/batch.py:19-22).  It
    holds in the dot-product family (default) and in the matrix-pipe family, chosen per weight
    (attribute ``batch_family``) or per process (``configure``) -- every entry switches together."""
    g = synth.generator(10)
    k, n = 2560, 1536
    x = synth.activations(16, k, g).to(G.DEV)
    plain = _q8(n, k, g)
    fast = QWeight(plain.wq, plain.scale, batch_family="mfma")
    y_dot, y_mfma = backend.linear_m(plain, x), backend.linear_m(fast, x)
    assert _rel(y_mfma, y_dot.float()) < 1e-2
    assert not (y_mfma.view(torch.int16) == y_dot.view(torch.int16)).all()      # two summation orders
    for w, y in ((plain, y_dot), (fast, y_mfma)):
        for r in (0, 5, 15):
            assert (backend.linear(w, x[r]).view(torch.int16) == y[r].view(torch.int16)).all()
        for m in (2, 4, 8):
            assert (backend.linear_m(w, x[:m].contiguous()).view(torch.int16) == y[:m].view(torch.int16)).all()
    # mfma family: verify and short prefill chunks are the same kernel, so the same bits
    assert (backend.linear_m_verify(fast, x).view(torch.int16) == y_mfma.view(torch.int16)).all()
    assert (backend.linear_prefill(fast, x).view(torch.int16) == y_mfma.view(torch.int16)).all()
    # the process-wide switch does the same for weights that do not say
    try:
        assert backend.configure(batch_family="mfma")["batch_family"] == "mfma"
        assert (backend.linear_m(plain, x).view(torch.int16) == y_mfma.view(torch.int16)).all()
        assert (backend.linear(plain, x[3]).view(torch.int16) == y_mfma[3].view(torch.int16)).all()
    finally:
        backend.configure(batch_family="dot")
    assert (backend.linear_m(plain, x).view(torch.int16) == y_dot.view(torch.int16)).all()
    with pytest.raises(ValueError):
        backend.configure(batch_family="tensor")
    # the C entry that takes the family as an argument: any number of rows in one call
    lib = backend._native.load()
    x100 = synth.activations(100, k, g).to(G.DEV)
    for family, mfma in ((0, False), (1, True)):
        y = torch.empty((100, n), dtype=torch.bfloat16, device=G.DEV)
        backend._native.check(lib.cmi_linear_w8a16(G.ptr(plain.wq), G.ptr(plain.scale), G.ptr(x100), G.ptr(y),
                                                   100, n, k, family, G.stream()), "linear_w8a16")
        step = 64 if mfma else 16
        for lo in range(0, 100, step):
            piece = G.gemv_w8a16(plain.wq, plain.scale, x100[lo:lo + step].contiguous(), mfma=mfma)
            assert (y[lo:lo + step].view(torch.int16) == piece.view(torch.int16)).all()
    assert lib.cmi_linear_w8a16(G.ptr(plain.wq), G.ptr(plain.scale), G.ptr(x100), G.ptr(y), 100, n, k, 2,
                                G.stream()) == backend._native.E_ARG
