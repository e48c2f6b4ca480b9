"""ctypes binding of ``libcoffin_mi355.so`` (the C ABI in ``include/coffin_mi355.h``).

This is the stub that takes the place of the reference's pybind modules
(backends/corex/kernels/__init__.py:156-163, backends/hip/shim.py:57-64): raw
device pointers, sizes and the current HIP stream go in, an ``int`` status comes
out and is turned into a Python exception here.  There is no CPU fallback: when
the library is missing or a call fails, the caller gets an error.
"""

from __future__ import annotations

import ctypes
from pathlib import Path

LIB_PATH = Path(__file__).resolve().parent / "libcoffin_mi355.so"

ABI_VERSION = 3

OK, E_ARG, E_UNSUPPORTED, E_HIP = 0, 1, 2, 3

_vp, _ci, _cs = ctypes.c_void_p, ctypes.c_int, ctypes.c_char_p
_i64, _sz, _f32 = ctypes.c_int64, ctypes.c_size_t, ctypes.c_float

#: name -> argtypes, exactly the declarations of include/coffin_mi355.h.
SIGNATURES: dict[str, list] = {
    "cmi_set_option": [_cs, _ci],
    "cmi_quant_act_i8": [_vp, _vp, _vp, _ci, _ci, _vp],
    "cmi_gemv_w8a16": [_vp, _vp, _vp, _vp, _ci, _ci, _ci, _vp],
    "cmi_gemv_w8a16_mfma": [_vp, _vp, _vp, _vp, _ci, _ci, _ci, _vp],
    "cmi_linear_w8a16": [_vp, _vp, _vp, _vp, _ci, _ci, _ci, _ci, _vp],
    "cmi_w4_repack": [_vp, _vp, _vp, _vp, _ci, _ci, _ci, _vp],
    "cmi_gemv_w4a8": [_vp, _vp, _vp, _vp, _vp, _vp, _ci, _ci, _ci, _ci, _vp],
    "cmi_gemv_w4a16": [_vp, _vp, _vp, _vp, _ci, _ci, _ci, _vp],
    "cmi_gemv_w4a8_bf16": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _ci, _ci, _ci, _ci, _vp],
    "cmi_gemm_w8a8": [_vp, _vp, _vp, _vp, _vp, _vp, _ci, _ci, _ci, _ci, _vp],
    "cmi_gemm_w4a8": [_vp, _vp, _vp, _vp, _vp, _vp, _ci, _ci, _ci, _ci, _vp],
    "cmi_linear_w8a8_bf16": [_vp, _vp, _vp, _vp, _ci, _ci, _ci, _ci, _vp, _sz, _vp],
    "cmi_linear_w4a8_bf16": [_vp, _vp, _vp, _vp, _ci, _ci, _ci, _ci, _vp, _sz, _vp],
    "cmi_linear_w4a8_bf16_static": [_vp, _vp, _vp, _vp, _ci, _ci, _ci, _ci, _vp],
    "cmi_silu_mul_quant": [_vp, _vp, _vp, _vp, _vp, _ci, _ci, _i64, _i64, _i64, _vp],
    "cmi_rms_norm_i8": [_vp, _vp, _vp, _vp, _vp, _ci, _ci, _i64, _i64, _f32, _vp],
    "cmi_add_rms_norm_i8": [_vp, _vp, _vp, _vp, _vp, _vp, _ci, _ci, _i64, _i64, _i64, _f32, _vp],
    "cmi_embed_rows_i8": [_vp, _vp, _vp, _vp, _ci, _ci, _ci, _vp],
    "cmi_embed_rows_w4": [_vp, _vp, _vp, _vp, _ci, _ci, _ci, _ci, _vp],
}

#: Entry points that do not return a status.
OTHER_RESTYPES = {"cmi_linear_workspace_bytes": ([_ci, _ci], _sz),
                  "cmi_linear_w8a8_workspace_bytes": ([_ci, _ci, _ci], _sz),
                  "cmi_stream_capture_id": ([_vp], ctypes.c_longlong),
                  "cmi_w4_device_k": ([_ci, _ci], _ci)}


class NativeError(RuntimeError):
    """A C-ABI call returned a non-zero status."""

    def __init__(self, code: int, message: str) -> None:
        super().__init__(message)
        self.code = code


_lib: ctypes.CDLL | None = None
_load_error: str | None = None


def load() -> ctypes.CDLL:
    """Load the shared library once; raise ``RuntimeError`` when it cannot be used."""
    global _lib, _load_error
    if _lib is not None:
        return _lib
    if _load_error is not None:
        raise RuntimeError(_load_error)
    try:
        # torch ships its own HIP runtime under the same soname as the system
        # one; importing torch first makes the kernels bind to the runtime that
        # owns torch's device memory and streams, whatever the import order of
        # the caller.
        import torch  # noqa: F401
        if not LIB_PATH.exists():
            raise OSError(f"{LIB_PATH} is missing; build it with `python -m coffin_amd.build`")
        lib = ctypes.CDLL(str(LIB_PATH))
        lib.cmi_abi_version.restype = _ci
        lib.cmi_last_error.restype = ctypes.c_char_p
        version = int(lib.cmi_abi_version())
        if version != ABI_VERSION:
            raise OSError(f"{LIB_PATH} has ABI {version}, this package expects {ABI_VERSION}")
        for name, argtypes in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.argtypes = argtypes
            fn.restype = _ci
        for name, (argtypes, restype) in OTHER_RESTYPES.items():
            fn = getattr(lib, name)
            fn.argtypes = argtypes
            fn.restype = restype
    except (OSError, AttributeError) as exc:
        # Memoised: a failed load is reported the same way on every call instead
        # of being retried on the decode path.
        _load_error = f"coffin_amd native library unusable: {exc}"
        raise RuntimeError(_load_error) from exc
    _lib = lib
    return lib


def available() -> bool:
    """True when the shared library loads (says nothing about a GPU being present)."""
    try:
        load()
    except RuntimeError:
        return False
    return True


def last_error() -> str:
    return load().cmi_last_error().decode("utf-8", "replace")


def check(status: int, what: str) -> None:
    """Turn a status code into the exception the adapter contract asks for."""
    if status == OK:
        return
    message = f"{what}: {last_error()}"
    if status in (E_ARG, E_UNSUPPORTED):
        raise ValueError(message)
    raise NativeError(status, message)
