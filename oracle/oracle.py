"""ctypes front end of the CPU oracle (``oracle/coffin_oracle.c``).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, by ``__graft_entry__.smoke``
and by the ``cpu_baseline`` leg of ``bench.py``.  The product package never
imports it.

All arrays are numpy; bf16 travels as ``uint16`` bit patterns.  Each wrapper
names the reference lines its C function restates; the arithmetic itself is
documented in the C file.
"""

from __future__ import annotations

import ctypes
import subprocess
from pathlib import Path

import numpy as np

_DIR = Path(__file__).resolve().parent
_LIB_PATH = _DIR / "libcoffin_oracle.so"
_lib = None


def build(force: bool = False) -> Path:
    """Compile the C oracle next to its source and return the library path."""
    if force or not _LIB_PATH.exists():
        subprocess.run(["make", "-C", str(_DIR)] + (["-B"] if force else []),
                       check=True, capture_output=True)
    return _LIB_PATH


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        build()
        _lib = ctypes.CDLL(str(_LIB_PATH))
        _lib.orc_num_threads.restype = ctypes.c_int
    return _lib


def _p(a: np.ndarray | None):
    if a is None:
        return ctypes.c_void_p(0)
    assert a.flags["C_CONTIGUOUS"], "oracle inputs must be contiguous"
    return ctypes.c_void_p(a.ctypes.data)


def _i(v: int) -> ctypes.c_int64:
    return ctypes.c_int64(int(v))


def num_threads() -> int:
    return int(lib().orc_num_threads())


def set_num_threads(n: int) -> None:
    lib().orc_set_num_threads(ctypes.c_int(int(n)))


# ------------------------------------------------------------------ bf16 (R10)

def bf16_from_f32(x: np.ndarray) -> np.ndarray:
    """fp32 -> bf16 bits, RNE.  backends/corex/kernels/corex_scalar.h:37-41."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, dtype=np.uint16)
    lib().orc_bf16_from_f32(_p(x), _p(out), _i(x.size))
    return out


def bf16_to_f32(x: np.ndarray) -> np.ndarray:
    """bf16 bits -> fp32.  backends/corex/kernels/corex_scalar.h:31-34."""
    x = np.ascontiguousarray(x, dtype=np.uint16)
    out = np.empty(x.shape, dtype=np.float32)
    lib().orc_bf16_to_f32(_p(x), _p(out), _i(x.size))
    return out


# ------------------------------------------------------------- weight formats

def qweight_quantize(w: np.ndarray) -> tuple[np.ndarray, np.ndarray]:
    """R0, int8_weights.py:328-332.  w fp32 [N,K] -> (wq int8 [N,K], scale fp32 [N])."""
    w = np.ascontiguousarray(w, dtype=np.float32)
    n, k = w.shape
    wq = np.empty((n, k), dtype=np.int8)
    scale = np.empty(n, dtype=np.float32)
    lib().orc_qweight_quantize(_p(w), _i(n), _i(k), _p(wq), _p(scale))
    return wq, scale


def qweight_dequant_bf16(wq: np.ndarray, scale: np.ndarray) -> np.ndarray:
    """int8_weights.py:359 with dtype=bf16; returns bf16 bits [N,K]."""
    n, k = wq.shape
    out = np.empty((n, k), dtype=np.uint16)
    lib().orc_qweight_dequant_bf16(_p(wq), _p(scale), _i(n), _i(k), _p(out))
    return out


def w4_quantize(w: np.ndarray, group_size: int = 128) -> tuple[np.ndarray, np.ndarray]:
    """R7, tools/quant_disk_w4a8.py:45-89.  -> (packed u8 [ceil(Kpad/2),N], scale [G,N])."""
    w = np.ascontiguousarray(w, dtype=np.float32)
    n, k = w.shape
    g = -(-k // group_size)
    ke = (g * group_size + 1) // 2 * 2
    packed = np.empty((ke // 2, n), dtype=np.uint8)
    scale = np.empty((g, n), dtype=np.float32)
    lib().orc_w4_quantize(_p(w), _i(n), _i(k), _i(group_size), _p(packed), _p(scale))
    return packed, scale


def w4_dequant_f32(packed: np.ndarray, scale: np.ndarray, k: int,
                   group_size: int = 128) -> np.ndarray:
    """tools/quant_disk_w4a8.py:118-128 / w4a8_weights.py:84-99.  -> fp32 [N,K]."""
    n = packed.shape[1]
    out = np.empty((n, k), dtype=np.float32)
    lib().orc_w4_dequant_f32(_p(packed), _p(scale), _i(n), _i(k), _i(group_size), _p(out))
    return out


# --------------------------------------------------------- activation quant R3

def quant_division_mismatches(amax_lo: int = 0, amax_hi: int = 0x7F80, check_quotient: bool = True) -> int:
    """Pairs (row absmax, element) for which the kernels' division-free rounding
    (one reciprocal per row, two fused multiply-adds per element) differs from
    ``rint(x / s)`` of backends/reference/__init__.py:386-389; exhaustive over bf16."""
    fn = lib().orc_quant_division_mismatches
    fn.restype = ctypes.c_int64
    return int(fn(ctypes.c_int32(amax_lo), ctypes.c_int32(amax_hi), ctypes.c_int32(int(check_quotient))))


def quant_act_i8(x_bf16: np.ndarray) -> tuple[np.ndarray, np.ndarray]:
    """R3, backends/reference/__init__.py:386-389.  x bf16 bits [M,K] -> (q, s)."""
    m, k = x_bf16.shape
    q = np.empty((m, k), dtype=np.int8)
    s = np.empty(m, dtype=np.float32)
    lib().orc_quant_act_i8(_p(x_bf16), _i(m), _i(k), _p(q), _p(s))
    return q, s


# ------------------------------------------------------------------- linears

def linear_qweight(wq, scale, x_bf16) -> np.ndarray:
    """R1, backends/reference/__init__.py:93-95 with a QWeight.  -> bf16 bits [M,N]."""
    n, k = wq.shape
    m = x_bf16.shape[0]
    y = np.empty((m, n), dtype=np.uint16)
    lib().orc_linear_qweight(_p(wq), _p(scale), _p(x_bf16), _i(m), _i(n), _i(k), _p(y))
    return y


def linear_w4weight(packed, scale, x_bf16, k: int, group_size: int = 128) -> np.ndarray:
    """R8, reference._linear on a W4A8Weight (unquantised activations)."""
    n = packed.shape[1]
    m = x_bf16.shape[0]
    y = np.empty((m, n), dtype=np.uint16)
    lib().orc_linear_w4weight(_p(packed), _p(scale), _p(x_bf16), _i(m), _i(n), _i(k),
                              _i(group_size), _p(y))
    return y


def gemv_w8a16_exact(wq, scale, x_bf16) -> np.ndarray:
    """R2 evaluated exactly (double): scale[n]*sum_k wq*x, fp32 [M,N]."""
    n, k = wq.shape
    m = x_bf16.shape[0]
    y = np.empty((m, n), dtype=np.float32)
    lib().orc_gemv_w8a16_exact(_p(wq), _p(scale), _p(x_bf16), _i(m), _i(n), _i(k), _p(y))
    return y


def gemm_w8a8(xq, wq, xs, ws, want_acc: bool = True, want_y: bool = True):
    """R4.  -> (acc int32 [M,N] or None, y bf16 bits [M,N] or None)."""
    m, k = xq.shape
    n = wq.shape[0]
    acc = np.empty((m, n), dtype=np.int32) if want_acc else None
    y = np.empty((m, n), dtype=np.uint16) if want_y else None
    lib().orc_gemm_w8a8(_p(xq), _p(wq), _p(xs), _p(ws), _i(m), _i(n), _i(k), _p(acc),
                        _p(y), _i(n))
    return acc, y


def linear_w4a8(xq, xs, packed, ws, k: int, group_size: int = 128,
                want_group_acc: bool = False):
    """R5/R6.  -> (group_acc int32 [M,G,N] or None, y bf16 bits [M,N])."""
    m = xq.shape[0]
    n = packed.shape[1]
    g = -(-k // group_size)
    gacc = np.empty((m, g, n), dtype=np.int32) if want_group_acc else None
    y = np.empty((m, n), dtype=np.uint16)
    lib().orc_linear_w4a8(_p(xq), _p(xs), _p(packed), _p(ws), _i(m), _i(n), _i(k),
                          _i(group_size), _p(gacc), _p(y))
    return gacc, y


# --------------------------------------------------------------- torch bridge

def bits(t) -> np.ndarray:
    """torch bf16 tensor (CPU) -> uint16 bit-pattern array, same shape."""
    import torch
    assert t.dtype == torch.bfloat16
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def from_bits(a: np.ndarray):
    """uint16 bit-pattern array -> torch bf16 tensor (CPU)."""
    import torch
    return torch.from_numpy(np.ascontiguousarray(a).view(np.int16)).view(torch.bfloat16)



# ------------------------------------------------------- fused quant producers

def silu_bf16(g_bf16: np.ndarray) -> np.ndarray:
    """bf16 bits of silu(g), fp32 arithmetic (backends/reference/__init__.py:253-268)."""
    g = np.ascontiguousarray(g_bf16, dtype=np.uint16)
    out = np.empty_like(g)
    lib().orc_silu_bf16(_p(g), _p(out), _i(g.size))
    return out


def silu_mul_quant(gate: np.ndarray, up: np.ndarray, quant: bool = True):
    """``silu_mul`` then ``kv_quant`` (backends/protocol.py:274-278).  gate, up: bf16 bits
    [M,K] -> (out bf16 bits [M,K], q int8 [M,K] or None, s fp32 [M] or None)."""
    m, k = gate.shape
    out = np.empty((m, k), dtype=np.uint16)
    q = np.empty((m, k), dtype=np.int8) if quant else None
    s = np.empty(m, dtype=np.float32) if quant else None
    lib().orc_silu_mul_quant(_p(np.ascontiguousarray(gate)), _p(np.ascontiguousarray(up)), _i(m), _i(k),
                             _i(k), _i(k), _p(out), _p(q), _p(s))
    return out, q, s


def rms_norm(x: np.ndarray, w: np.ndarray, eps: float = 1e-6, add: np.ndarray | None = None):
    """Reference RMSNorm (backends/reference/__init__.py:169-198), after the residual add of
    :224-250 when ``add`` is given.  x, add: bf16 bits [M,N]; w: bf16 bits [N] ->
    (y bf16 bits [M,N], x after the add, bf16 bits [M,N])."""
    m, n = x.shape
    xs = np.array(x, dtype=np.uint16, order="C", copy=True)
    y = np.empty((m, n), dtype=np.uint16)
    a = None if add is None else np.ascontiguousarray(add, dtype=np.uint16)
    lib().orc_rms_norm(_p(xs), _p(a), _p(np.ascontiguousarray(w, dtype=np.uint16)), _i(m), _i(n),
                       _i(n), _i(n), ctypes.c_float(eps), _p(y))
    return y, xs
