"""The projection entry that allocates nothing (cmi_linear_w4a8_bf16_static) against the entry it
is a variant of (cmi_linear_w4a8_bf16 with a caller's workspace): same bits, on two calls in a
row, the second with a smaller input (the fixed array keeps the first call's contents)."""

from __future__ import annotations

import ctypes

import pytest
import torch

from coffin_amd import _native, synth
from tests import gpu_util as G

pytestmark = pytest.mark.gpu


def _with_workspace(w4, ws, x, n, k):
    m = x.shape[0]
    lib = _native.load()
    nbytes = int(lib.cmi_linear_workspace_bytes(m, k))
    work = torch.empty(nbytes, dtype=torch.uint8, device=G.DEV)
    y = torch.empty((m, n), dtype=torch.bfloat16, device=G.DEV)
    _native.check(lib.cmi_linear_w4a8_bf16(G.ptr(w4), G.ptr(ws), G.ptr(x), G.ptr(y), m, n, k, 128, G.ptr(work),
                                           nbytes, G.stream()), "linear_w4a8_bf16")
    return y


def _static(w4, ws, x, n, k):
    m = x.shape[0]
    y = torch.empty((m, n), dtype=torch.bfloat16, device=G.DEV)
    _native.check(_native.load().cmi_linear_w4a8_bf16_static(G.ptr(w4), G.ptr(ws), G.ptr(x), G.ptr(y), m, n, k, 128,
                                                             G.stream()), "linear_w4a8_bf16_static")
    return y


def test_static_workspace_entry_matches_the_workspace_entry_on_consecutive_calls():
    g = synth.generator(1234, G.DEV)
    n, k = 2560, 9728
    w = synth.int4_weight(n, k, g)
    w4, ws = G.w4_repack(w.packed, w.scale, k)
    big = synth.activations(48, k, g, outliers=True)        # quantiser + GEMM route, 467 KB of staging
    small = synth.activations(5, k, g, outliers=True)       # quantiser + GEMV route, fewer rows than before
    one = synth.activations(1, k, g)                        # the GEMV that quantises by itself: no staging
    got = [_static(w4, ws, x, n, k) for x in (big, small, one, small)]
    torch.cuda.synchronize()
    want = [_with_workspace(w4, ws, x, n, k) for x in (big, small, one, small)]
    for a, b in zip(got, want):
        assert (a.view(torch.int16) == b.view(torch.int16)).all()
    # a second shape on the same array
    n2, k2 = 1024, 2560
    w2 = synth.int4_weight(n2, k2, g)
    w42, ws2 = G.w4_repack(w2.packed, w2.scale, k2)
    x2 = synth.activations(300, k2, g)
    assert (_static(w42, ws2, x2, n2, k2).view(torch.int16) == _with_workspace(w42, ws2, x2, n2, k2).view(torch.int16)).all()
    x3 = synth.activations(2, k2, g)
    assert (_static(w42, ws2, x3, n2, k2).view(torch.int16) == _with_workspace(w42, ws2, x3, n2, k2).view(torch.int16)).all()


def test_static_workspace_entry_replays_inside_a_captured_graph():
    """What the entry exists for: after one eager call per shape (the first call on a device takes
    the array's address and raises the kernels' LDS limits, which a capture cannot record), the call
    is recorded into a graph -- a hipMalloc or an attribute change inside it would fail the capture --
    and replayed on new activations in the same buffer, bit for bit the eager result."""
    g = synth.generator(4321, G.DEV)
    n, k = 1536, 2560
    w = synth.int4_weight(n, k, g)
    w4, ws = G.w4_repack(w.packed, w.scale, k)
    xs = {m: synth.activations(m, k, g) for m in (1, 6, 40)}
    for x in xs.values():
        _static(w4, ws, x, n, k)                             # warm-up, eager
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            outs = {m: _static(w4, ws, x, n, k) for m, x in xs.items()}
    torch.cuda.current_stream().wait_stream(side)
    for seed in (1, 2, 3):
        gg = synth.generator(seed, G.DEV)
        for m, x in xs.items():
            x.copy_(synth.activations(m, k, gg))
        graph.replay()
        torch.cuda.synchronize()
        for m, x in xs.items():
            want = _with_workspace(w4, ws, x, n, k)
            assert (outs[m].view(torch.int16) == want.view(torch.int16)).all(), (seed, m)


def test_static_workspace_entry_refuses_what_does_not_fit():
    lib = _native.load()
    one = ctypes.c_void_p(256)
    # 8 MiB of quantised rows and 16384 rows are the limits; nothing is launched for these
    assert lib.cmi_linear_w4a8_bf16_static(one, one, one, one, 1024, 8, 8320, 128, None) == _native.E_UNSUPPORTED
    assert "exceeds the fixed workspace" in _native.last_error()
    assert lib.cmi_linear_w4a8_bf16_static(one, one, one, one, 16385, 8, 128, 128, None) == _native.E_UNSUPPORTED
    assert lib.cmi_linear_w4a8_bf16_static(None, one, one, one, 4, 8, 128, 128, None) == _native.E_ARG
