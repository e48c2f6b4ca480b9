"""Quantized weight containers with the attribute surface coffin's callers read.

``QWeight`` restates int8_weights.py:249-385 (``wq`` int8 [N,K], ``scale`` fp32
[N], ``n``, ``k``, ``quantize``, ``dequant``, ``rows``); ``W4A8Weight`` restates
w4a8_weights.py:28-99 (``packed`` uint8 [ceil(K/2),N], ``scale`` fp32 [G,N],
``k``, ``n``, ``group_size``, ``cat_output``, ``rows``, ``to``) and
``quantize_projection`` / ``dequantize_projection`` restate
tools/quant_disk_w4a8.py:45-128.  The backend adapter dispatches on attributes,
not on these classes, so coffin's own objects are accepted unchanged.

The encoders run in torch on whatever device the dense weight lives on; they
are load-time code, not part of the hot path.
"""

from __future__ import annotations

import torch

#: Rows quantised per fp32 temporary, so a wide ``lm_head`` never needs a full
#: fp32 copy (int8_weights.py:334-344 chunks for the same reason).
_CHUNK_ROWS = 16384


class QWeight:
    """int8 ``[N, K]`` weight with one fp32 absmax scale per output row."""

    __slots__ = ("wq", "scale", "n", "k", "batch_family")

    def __init__(self, wq: torch.Tensor, scale: torch.Tensor, batch_family: str | None = None) -> None:
        self.wq = wq
        self.scale = scale
        self.n, self.k = (int(d) for d in wq.shape)
        #: ``None`` (the process-wide setting), ``"dot"`` or ``"mfma"``: the kernel family every
        #: weight-only call on this weight uses (``coffin_amd.backend.configure``); read by the
        #: adapter when the weight is first used.  Not an attribute of the reference's class.
        self.batch_family = batch_family

    @classmethod
    def quantize(cls, w: torch.Tensor, chunk_rows: int = _CHUNK_ROWS) -> "QWeight":
        """scale = max(amax_k|w|, 1e-8)/127; wq = clamp(rne(w/scale), -127, 127)."""
        n = int(w.shape[0])
        wq = torch.empty(tuple(w.shape), dtype=torch.int8, device=w.device)
        scale = torch.empty(n, dtype=torch.float32, device=w.device)
        for lo in range(0, max(n, 1), chunk_rows):
            hi = min(n, lo + chunk_rows)
            block = w[lo:hi].to(torch.float32)
            s = block.abs().amax(dim=-1).clamp_min(1e-8) / 127.0
            wq[lo:hi] = torch.round(block / s.unsqueeze(1)).clamp_(-127, 127).to(torch.int8)
            scale[lo:hi] = s
        return cls(wq, scale)

    @classmethod
    def from_kn(cls, wt: torch.Tensor, scale: torch.Tensor) -> "QWeight":
        """Wrap an int8 ``[K, N]`` buffer without copying (int8_weights.py:271-305).

        ``wq`` becomes the transposed view, strides ``(1, N)``.  The MI355X
        kernels stream ``[N, K]`` rows, so the backend adapter makes its own
        row-major copy of such a weight the first time it is used.
        """
        if wt.dim() != 2 or wt.dtype != torch.int8:
            raise ValueError(f"packed int8 weight must be 2-D int8, got "
                             f"{tuple(wt.shape)} {wt.dtype}")
        if scale.dim() != 1 or scale.dtype != torch.float32:
            raise ValueError("scale must be 1-D fp32")
        if int(scale.numel()) != int(wt.shape[1]):
            raise ValueError(f"scale holds {scale.numel()} values for N = {int(wt.shape[1])}")
        if not wt.is_contiguous():
            raise ValueError("packed [K, N] weight must be contiguous")
        return cls(wt.t(), scale)

    def dequant(self, dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
        """Dense ``[N, K]``: one fp32 product, one narrowing (int8_weights.py:359)."""
        return (self.wq.to(torch.float32) * self.scale.unsqueeze(1)).to(dtype)

    def rows(self, idx: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
        return self.wq.index_select(0, idx), self.scale.index_select(0, idx)

    def nbytes(self) -> int:
        return self.wq.numel() + 4 * self.scale.numel()

    def __repr__(self) -> str:
        return f"QWeight({self.n}x{self.k} int8)"


def quantize_projection(w: torch.Tensor, group_size: int = 128
                        ) -> tuple[torch.Tensor, torch.Tensor]:
    """Pack a dense ``[N,K]`` weight into ``uint8 [ceil(Kpad/2), N]`` + ``fp32 [G, N]``.

    Per (group of ``group_size`` along K, output n): scale = max(amax,1e-8)/7,
    q = clamp(rne(w/scale), -8, 7), code = q + 8; even k in the low nibble.  K is
    padded with zeros (code 8) to whole groups and to an even length.
    """
    if w.dim() != 2:
        raise ValueError(f"projection must be 2-D, got {tuple(w.shape)}")
    if group_size <= 0:
        raise ValueError(f"group_size must be positive, got {group_size}")
    n, k = (int(d) for d in w.shape)
    groups = -(-k // group_size)
    kpad = groups * group_size
    keven = kpad + (kpad & 1)
    packed = torch.empty((keven // 2, n), dtype=torch.uint8, device=w.device)
    scales = torch.empty((groups, n), dtype=torch.float32, device=w.device)
    for lo in range(0, n, _CHUNK_ROWS):
        hi = min(n, lo + _CHUNK_ROWS)
        block = torch.zeros((hi - lo, keven), dtype=torch.float32, device=w.device)
        block[:, :k] = w[lo:hi]
        grouped = block[:, :kpad].view(hi - lo, groups, group_size)
        s = grouped.abs().amax(dim=-1).clamp_min(1e-8) / 7.0
        q = torch.round(grouped / s.unsqueeze(-1)).clamp_(-8, 7)
        codes = torch.full((hi - lo, keven), 8, dtype=torch.int32, device=w.device)
        codes[:, :kpad] = q.view(hi - lo, kpad).to(torch.int32) + 8
        byte = codes[:, 0::2] | (codes[:, 1::2] << 4)
        packed[:, lo:hi] = byte.to(torch.uint8).t()
        scales[:, lo:hi] = s.t()
    return packed.contiguous(), scales.contiguous()


def _unpack_rows(packed_cols: torch.Tensor, k: int) -> torch.Tensor:
    """``uint8 [ceil(K/2), R]`` -> signed codes ``int16 [R, K]``."""
    b = packed_cols.t().to(torch.int16)
    out = torch.empty((b.shape[0], b.shape[1] * 2), dtype=torch.int16, device=b.device)
    out[:, 0::2] = b & 0xF
    out[:, 1::2] = (b >> 4) & 0xF
    return out[:, :k] - 8


def dequantize_projection(packed: torch.Tensor, scales: torch.Tensor, *, k: int,
                          group_size: int = 128) -> torch.Tensor:
    """Inverse of :func:`quantize_projection`: fp32 ``[N, K]`` = (code-8) * scale[g, n]."""
    if packed.dim() != 2 or packed.dtype != torch.uint8:
        raise ValueError("packed weight must be a 2-D uint8 tensor")
    if scales.dim() != 2 or scales.dtype != torch.float32:
        raise ValueError("scales must be a 2-D fp32 tensor")
    if k <= 0 or group_size <= 0:
        raise ValueError("K and group_size must be positive")
    n = int(packed.shape[1])
    groups = -(-k // group_size)
    if tuple(scales.shape) != (groups, n):
        raise ValueError(f"scales must have shape {(groups, n)}, got {tuple(scales.shape)}")
    if packed.shape[0] * 2 < k:
        raise ValueError("packed weight is shorter than K")
    gid = torch.arange(k, device=packed.device) // group_size
    return _unpack_rows(packed, k).to(torch.float32) * scales.t().index_select(1, gid)


class W4A8Weight:
    """Group-symmetric int4 weight, logical ``[N, K]``, stored K-major and nibble packed."""

    __slots__ = ("group_size", "k", "n", "packed", "scale")

    def __init__(self, packed: torch.Tensor, scale: torch.Tensor, *, k: int,
                 group_size: int = 128) -> None:
        if packed.dim() != 2 or packed.dtype != torch.uint8 or not packed.is_contiguous():
            raise ValueError("packed weight must be contiguous 2-D uint8 [ceil(K/2), N]")
        if scale.dim() != 2 or scale.dtype != torch.float32 or not scale.is_contiguous():
            raise ValueError("scale must be contiguous 2-D fp32 [groups, N]")
        if k <= 0 or group_size <= 0:
            raise ValueError("K and group_size must be positive")
        n = int(packed.shape[1])
        groups = -(-k // group_size)
        if packed.shape[0] * 2 < k or tuple(scale.shape) != (groups, n):
            raise ValueError("packed weight or scale shape does not match K/group_size")
        self.packed, self.scale = packed, scale
        self.k, self.n, self.group_size = int(k), n, int(group_size)

    @classmethod
    def quantize(cls, w: torch.Tensor, group_size: int = 128) -> "W4A8Weight":
        packed, scale = quantize_projection(w, group_size)
        return cls(packed, scale, k=int(w.shape[1]), group_size=group_size)

    @property
    def shape(self) -> tuple[int, int]:
        return self.n, self.k

    def nbytes(self) -> int:
        return self.packed.numel() + self.scale.numel() * self.scale.element_size()

    @classmethod
    def cat_output(cls, weights: list["W4A8Weight"]) -> "W4A8Weight":
        """Fuse projections that share K along the output axis (w4a8_weights.py:58-82)."""
        head = weights[0]
        for w in weights:
            if (w.k != head.k or w.group_size != head.group_size
                    or w.packed.device != head.packed.device):
                raise ValueError("W4A8 weights must share K, group_size, and device")
        packed = torch.cat([w.packed for w in weights], dim=1).contiguous()
        scale = torch.cat([w.scale for w in weights], dim=1).contiguous()
        return cls(packed, scale, k=head.k, group_size=head.group_size)

    def rows(self, ids: torch.Tensor) -> torch.Tensor:
        """Dequantised fp32 rows ``[len(ids), K]`` (embedding-style gather)."""
        ids = ids.reshape(-1)
        q = _unpack_rows(self.packed.index_select(1, ids), self.k).to(torch.float32)
        gid = torch.arange(self.k, device=self.packed.device) // self.group_size
        return q * self.scale.index_select(1, ids).t().index_select(1, gid)

    def to(self, dtype: torch.dtype) -> torch.Tensor:
        """Dense contiguous ``[N, K]`` in ``dtype`` (what the torch reference multiplies)."""
        every = torch.arange(self.n, device=self.packed.device)
        return self.rows(every).to(dtype).contiguous()
