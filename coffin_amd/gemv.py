"""Callers of the path: per-projection ``GEMV`` objects and same-input fusion.

Restates the regime choice of ops/gemv.py:37-243.  A ``GEMV`` holds one
``[N, K]`` weight (plain tensor, ``QWeight`` or ``W4A8Weight``) and picks a
table entry purely by row count; a ``GEMVGroup`` concatenates projections that
share their input along the output axis so one wide weight read replaces several
narrow ones, and splits the result back.

================  ======================================  ====================
method            rows                                    table entry
================  ======================================  ====================
``__call__``      any (``[K]`` or ``[C, K]``)             ``linear``
``linear_m``      1 -> ``linear`` on ``x[0]``; else       ``linear_m``
``linear_m_verify``  1 -> ``linear`` on ``x[0]``; else    ``linear_m_verify``
``prefill``       1 -> ``linear``; 2..8 -> ``linear_m``;  ``linear_prefill``
                  more
================  ======================================  ====================
"""

from __future__ import annotations

import torch

from coffin_amd import backend as _backend

#: Widest verify window the model captures; up to here a chunk shares one weight
#: read through ``linear_m`` instead of going to the GEMM (ops/gemv.py:126-134).
SMALL_BATCH_ROWS = 8


def _is_q8(w) -> bool:
    return hasattr(w, "wq") and hasattr(w, "scale")


def _is_w4(w) -> bool:
    return hasattr(w, "packed") and hasattr(w, "group_size")


class GEMV:
    """One ``[N, K]`` projection evaluated the way decode does it."""

    def __init__(self, w, bench: bool = True, ops=None) -> None:
        """``bench`` is accepted and ignored, as in the reference (ops/gemv.py:46-59).

        ``ops`` is any object with the four ``linear*`` attributes; default is
        this package's native adapters.
        """
        del bench
        self.q = w if _is_q8(w) else None
        self.q4 = w if _is_w4(w) else None
        quant = self.q if self.q is not None else self.q4
        self.N, self.K = (quant.n, quant.k) if quant is not None else w.shape
        self.w = w
        self.ops = ops if ops is not None else _backend

    def __call__(self, x: torch.Tensor) -> torch.Tensor:
        return self.ops.linear(self.w, x)

    def linear_m(self, x: torch.Tensor) -> torch.Tensor:
        # A one-row batch would come back 1-D from the backend; keep the row axis
        # so a group can still split along dim 1.
        if x.shape[0] == 1:
            return self(x[0]).unsqueeze(0)
        return self.ops.linear_m(self.w, x)

    def linear_m_verify(self, x: torch.Tensor) -> torch.Tensor:
        if x.shape[0] == 1:
            return self(x[0]).unsqueeze(0)
        return self.ops.linear_m_verify(self.w, x)

    def prefill(self, x: torch.Tensor) -> torch.Tensor:
        rows = x.shape[0]
        if rows == 1:
            return self(x[0]).unsqueeze(0)
        if rows <= SMALL_BATCH_ROWS:
            return self.ops.linear_m(self.w, x)
        return self.ops.linear_prefill(self.w, x)


class GEMVGroup:
    """Projections ``[N_i, K]`` sharing one input, fused into a single weight."""

    def __init__(self, ws: list, bench: bool = True, ops=None) -> None:
        head = ws[0]
        if _is_w4(head):
            if not all(_is_w4(w) for w in ws):
                raise ValueError("fused projections must use the same weight format")
            self.sizes = [int(w.n) for w in ws]
            fused = type(head).cat_output(ws)
        elif _is_q8(head):
            if not all(_is_q8(w) for w in ws):
                raise ValueError("fused projections must use the same weight format")
            self.sizes = [int(w.n) for w in ws]
            # One preallocated destination filled in place: torch.cat would keep
            # every source and the result alive together.
            total = sum(self.sizes)
            wq = torch.empty((total, head.k), dtype=head.wq.dtype, device=head.wq.device)
            scale = torch.empty(total, dtype=head.scale.dtype, device=head.scale.device)
            at = 0
            for w in ws:
                wq[at:at + w.n].copy_(w.wq)
                scale[at:at + w.n].copy_(w.scale)
                at += w.n
            fused = type(head)(wq, scale)
        else:
            self.sizes = [int(w.shape[0]) for w in ws]
            fused = torch.empty((sum(self.sizes), head.shape[1]), dtype=head.dtype,
                                device=head.device)
            at = 0
            for w in ws:
                fused[at:at + w.shape[0]].copy_(w)
                at += w.shape[0]
        self.g = GEMV(fused, bench, ops)

    def __call__(self, x: torch.Tensor):
        return self.g(x).split(self.sizes, dim=-1)

    def linear_m(self, x: torch.Tensor):
        if x.shape[0] == 1:
            return [part.unsqueeze(0) for part in self(x[0])]
        return self.g.linear_m(x).split(self.sizes, dim=1)

    def linear_m_verify(self, x: torch.Tensor):
        if x.shape[0] == 1:
            return [part.unsqueeze(0) for part in self(x[0])]
        return self.g.linear_m_verify(x).split(self.sizes, dim=1)

    def prefill(self, x: torch.Tensor):
        if x.shape[0] == 1:
            return [part.unsqueeze(0) for part in self(x[0])]
        return self.g.prefill(x).split(self.sizes, dim=1)


def _proj(sd: dict, prefixes: list[str], bench: bool = True):
    """``GEMV`` for one checkpoint prefix, ``GEMVGroup`` for several (ops/gemv.py:246-262)."""
    ws = [sd[p + ".weight"] for p in prefixes]
    return GEMV(ws[0], bench) if len(ws) == 1 else GEMVGroup(ws, bench)
