"""Helpers for the GPU parity tests: call the C ABI with torch device tensors."""

from __future__ import annotations

import ctypes

import numpy as np
import torch

from coffin_amd import _native

DEV = "cuda"


def ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else ctypes.c_void_p(0)


def stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def set_option(name: str, value: int) -> None:
    """Kernel-selection override of the library (cmi_set_option): gemm_tile, gemv_wholerow."""
    _native.check(_native.load().cmi_set_option(name.encode(), int(value)), "set_option")


def dev(a: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def bits(t: torch.Tensor) -> np.ndarray:
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def bf16_dev(bits_: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(bits_).view(np.int16)).view(torch.bfloat16).to(DEV)


def quant(x: torch.Tensor):
    m, k = x.shape
    q = torch.empty((m, k), dtype=torch.int8, device=DEV)
    s = torch.empty(m, dtype=torch.float32, device=DEV)
    _native.check(_native.load().cmi_quant_act_i8(ptr(x), ptr(q), ptr(s), m, k, stream()), "quant")
    return q, s


def gemv_w8a16(wq, ws, x, mfma: bool = False):
    """The dot-product GEMV, or (mfma) the matrix-pipe one for batches."""
    m, k = x.shape
    n = wq.shape[0]
    y = torch.empty((m, n), dtype=torch.bfloat16, device=DEV)
    fn = _native.load().cmi_gemv_w8a16_mfma if mfma else _native.load().cmi_gemv_w8a16
    _native.check(fn(ptr(wq), ptr(ws), ptr(x), ptr(y), m, n, k, stream()), "gemv_w8a16")
    return y


def gemm_w8a8(xq, wq, xs, ws, want_acc=True, ldy=None):
    m, k = xq.shape
    n = wq.shape[0]
    ldy = ldy or n
    y = torch.zeros((m, ldy), dtype=torch.bfloat16, device=DEV)
    acc = torch.empty((m, n), dtype=torch.int32, device=DEV) if want_acc else None
    _native.check(_native.load().cmi_gemm_w8a8(ptr(xq), ptr(wq), ptr(xs), ptr(ws), ptr(y), ptr(acc),
                                               m, n, k, ldy, stream()), "gemm_w8a8")
    return acc, y


def w4_repack(packed, scale, k, gs=128):
    """Device layout of an int4 weight: rows of cmi_w4_device_k(k, gs) codes."""
    n = packed.shape[1]
    kd = int(_native.load().cmi_w4_device_k(k, gs))
    w4 = torch.empty((n, kd // 2), dtype=torch.uint8, device=DEV)
    ws = torch.empty((n, kd // gs), dtype=torch.float32, device=DEV)
    _native.check(_native.load().cmi_w4_repack(ptr(packed), ptr(scale), ptr(w4), ptr(ws), n, k, gs,
                                               stream()), "w4_repack")
    return w4, ws


def w4a8(w4, ws, xq, xs, k, gemm: bool, want_acc=True, gs=128):
    m = xq.shape[0]
    n = w4.shape[0]
    y = torch.empty((m, n), dtype=torch.bfloat16, device=DEV)
    gacc = torch.empty((m, k // gs, n), dtype=torch.int32, device=DEV) if want_acc else None
    lib = _native.load()
    fn = lib.cmi_gemm_w4a8 if gemm else lib.cmi_gemv_w4a8
    _native.check(fn(ptr(w4), ptr(ws), ptr(xq), ptr(xs), ptr(y), ptr(gacc), m, n, k, gs, stream()),
                  "gemm_w4a8" if gemm else "gemv_w4a8")
    return gacc, y


def gemv_w4a8_bf16(w4, ws, x, k, gs=128):
    """Fused quantiser + W4A8 GEMV; returns (group sums, y, xq used, xs used)."""
    m = x.shape[0]
    n = w4.shape[0]
    y = torch.empty((m, n), dtype=torch.bfloat16, device=DEV)
    gacc = torch.empty((m, k // gs, n), dtype=torch.int32, device=DEV)
    xq = torch.empty((m, k), dtype=torch.int8, device=DEV)
    xs = torch.empty(m, dtype=torch.float32, device=DEV)
    _native.check(_native.load().cmi_gemv_w4a8_bf16(ptr(w4), ptr(ws), ptr(x), ptr(y), ptr(gacc), ptr(xq),
                                                    ptr(xs), m, n, k, gs, stream()), "gemv_w4a8_bf16")
    return gacc, y, xq, xs


def gemv_w4a16(w4, ws, x, k, gs=128):
    """int4 weight-only GEMV on one unquantised bf16 row x [K] -> y [N]."""
    n = w4.shape[0]
    y = torch.empty(n, dtype=torch.bfloat16, device=DEV)
    _native.check(_native.load().cmi_gemv_w4a16(ptr(w4), ptr(ws), ptr(x), ptr(y), n, k, gs, stream()), "gemv_w4a16")
    return y
