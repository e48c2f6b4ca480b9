"""The slice of coffin's backend contract that the quantized-linear path touches.

When this package runs inside a coffin checkout the vendor file binds to coffin's
own ``backends.protocol`` / ``backends.vendor`` classes; everywhere else (this
repository's tests, the benchmark, a GPU box without the reference tree) these
stand-ins carry the same names, fields and error behaviour for the nine table
entries on the path:

* ``Ops`` -- backends/protocol.py:130-541: a frozen table keyed by op name,
  ``None`` = "no kernel here", ``from_mapping`` rejects unknown names
  (:520-541) and non-callables (:504-517).
* ``Caps`` -- backends/protocol.py:47-127, only the fields a linear backend sets.
* ``Detection`` / ``VendorSpec`` -- backends/vendor.py:80-101, :162-240.
"""

from __future__ import annotations

from dataclasses import dataclass, fields
from typing import Any, Callable, ClassVar, Mapping

import torch

OpFn = Callable[..., Any]

#: Claim strengths of backends/vendor.py:68-78.
CLAIM_NONE, CLAIM_NAMESPACE, CLAIM_NAME = 0, 1, 2


@dataclass(frozen=True)
class Ops:
    """Op table restricted to the entries this backend implements."""

    linear: OpFn | None = None           # linear(w, x) -> y, x [K] or [C,K]   (protocol.py:147)
    linear_m: OpFn | None = None         # linear_m(w, x[M,K]) -> [M,N]        (protocol.py:151)
    linear_m_verify: OpFn | None = None  # same shape, verify batches          (protocol.py:155)
    linear_prefill: OpFn | None = None   # linear_prefill(w, x[C,K]) -> [C,N]  (protocol.py:159)
    kv_quant: OpFn | None = None         # kv_quant(x, out_q, out_s) -> out_q  (protocol.py:258)
    silu_mul: OpFn | None = None         # silu_mul(gate, up, out) -> out      (protocol.py:273)
    silu_mul_quant: OpFn | None = None   # (gate, up, out, out_q, out_s) -> out (protocol.py:278)
    rms_norm: OpFn | None = None         # rms_norm(x, w, stride=0, eps=1e-6) -> y (protocol.py:243)
    add_rms_norm: OpFn | None = None     # (x, add, w, out, stride=0, eps=1e-6) -> out (protocol.py:248)

    NAMES: ClassVar[tuple[str, ...]]

    def __post_init__(self) -> None:
        for f in fields(self):
            value = getattr(self, f.name)
            if value is not None and not callable(value):
                raise TypeError(f"op {f.name!r} must be a callable or None, "
                                f"got {type(value).__name__}")

    @classmethod
    def from_mapping(cls, mapping: Mapping[str, OpFn | None]) -> "Ops":
        unknown = sorted(set(mapping) - set(cls.NAMES))
        if unknown:
            raise ValueError(f"unknown op(s): {', '.join(unknown)}; "
                             f"known: {', '.join(cls.NAMES)}")
        return cls(**{name: mapping.get(name) for name in cls.NAMES})

    def as_dict(self) -> dict[str, OpFn | None]:
        return {name: getattr(self, name) for name in self.NAMES}

    def implemented(self) -> tuple[str, ...]:
        return tuple(n for n, fn in self.as_dict().items() if fn is not None)

    def missing(self) -> tuple[str, ...]:
        return tuple(n for n, fn in self.as_dict().items() if fn is None)


Ops.NAMES = tuple(f.name for f in fields(Ops))


@dataclass(frozen=True)
class Caps:
    """What a backend is on this host (backends/protocol.py:47-127, linear-path fields)."""

    name: str
    device: str
    device_index: int = 0
    device_name: str = ""
    arch: str = ""
    native: frozenset = frozenset()
    act_dtype: torch.dtype = torch.bfloat16
    weight_dtype: torch.dtype = torch.bfloat16
    graph: bool = False
    autotune: bool = False
    int8_weights: bool = False
    weight_layout: str = "nk"


@dataclass(frozen=True)
class Detection:
    """How a vendor recognises its card (backends/vendor.py:80-101)."""

    namespace: str
    name_markers: tuple[str, ...] = ()
    hip: bool = False


@dataclass(frozen=True)
class VendorSpec:
    """A platform declaration (backends/vendor.py:162-240), same field names and checks."""

    name: str
    detection: Detection
    act_dtype: torch.dtype = torch.bfloat16
    weight_dtype: torch.dtype = torch.bfloat16
    graph: bool = False
    autotune: bool = False
    int8_weights: bool = False
    batch_attn: bool = False
    attn_split: int = 1
    weight_layout: str = "nk"
    priority: int = 100
    notes: str = ""
    has_kernels: bool = False
    build_ops: Callable[[], Any] | None = None

    def validate(self) -> None:
        if not self.name:
            raise ValueError("a vendor spec needs a name")
        if not self.detection.namespace:
            raise ValueError(f"{self.name}: detection.namespace is required")
        if self.weight_layout not in ("nk", "kn"):
            raise ValueError(f"{self.name}: weight_layout must be 'nk' or 'kn', "
                             f"got {self.weight_layout!r}")
        if self.attn_split < 1:
            raise ValueError(f"{self.name}: attn_split must be >= 1")
        if self.has_kernels and self.build_ops is None:
            raise ValueError(f"{self.name}: has_kernels is True but no build_ops was given")


def detect(detection: Detection) -> int:
    """Claim strength of this host for ``detection`` (backends/vendor.py:125-159)."""
    module = getattr(torch, detection.namespace, None)
    if module is None:
        return CLAIM_NONE
    try:
        if not module.is_available():
            return CLAIM_NONE
    except Exception:
        return CLAIM_NONE
    if detection.hip and getattr(torch.version, "hip", None) is None:
        return CLAIM_NONE
    if not detection.name_markers:
        return CLAIM_NAMESPACE
    try:
        name = str(module.get_device_name(0)).lower()
    except Exception:
        return CLAIM_NONE
    if name and any(marker.lower() in name for marker in detection.name_markers):
        return CLAIM_NAME
    return CLAIM_NONE
