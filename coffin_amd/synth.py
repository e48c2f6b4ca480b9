"""Seeded synthetic operands for the parity tests, the smoke check and the benchmark.

Distributions follow the benchmark configurations: weights ``N(0, 0.02)``
quantized with absmax scales that are rounded to fp16 and stored as fp32 (so a
"fp16 scale" and the reference's fp32 scale storage are the same numbers);
activations ``N(0, 1)`` in bf16, optionally with 1 % of the elements multiplied
by 20 before the cast (prefill outliers).  A ``torch.Generator`` drives
everything; tests seed it with 1234 like tests/test_backends.py:444.
"""

from __future__ import annotations

import torch

from coffin_amd.weights import QWeight, W4A8Weight

#: (name, N, K) of the int8 projections of one Qwen3.5-4B-shaped decode layer.
DECODE_LAYER = (
    ("q_proj", 4096, 2560), ("k_proj", 1024, 2560), ("v_proj", 1024, 2560),
    ("o_proj", 2560, 4096), ("gate_proj", 9728, 2560), ("up_proj", 9728, 2560),
    ("down_proj", 2560, 9728),
)
#: Same layer as its callers issue it: q/k/v and gate/up fused along N.
DECODE_LAYER_FUSED = (
    ("qkv_proj", 6144, 2560), ("o_proj", 2560, 4096),
    ("gate_up_proj", 19456, 2560), ("down_proj", 2560, 9728),
)
LM_HEAD = ("lm_head", 151936, 2560)


def generator(seed: int = 1234, device: str | torch.device = "cpu") -> torch.Generator:
    return torch.Generator(device=device).manual_seed(seed)


def _fp16_round(s: torch.Tensor) -> torch.Tensor:
    return s.to(torch.float16).to(torch.float32)


def dense_weight(n: int, k: int, gen: torch.Generator) -> torch.Tensor:
    return torch.randn((n, k), generator=gen, device=gen.device, dtype=torch.float32) * 0.02


def int8_weight(n: int, k: int, gen: torch.Generator, chunk_rows: int = 8192) -> QWeight:
    """Per-row absmax int8 weight with fp16-representable scales."""
    wq = torch.empty((n, k), dtype=torch.int8, device=gen.device)
    scale = torch.empty(n, dtype=torch.float32, device=gen.device)
    for lo in range(0, n, chunk_rows):
        hi = min(n, lo + chunk_rows)
        w = dense_weight(hi - lo, k, gen)
        s = _fp16_round(w.abs().amax(dim=1).clamp_min(1e-8) / 127.0).clamp_min(2.0 ** -24)
        wq[lo:hi] = torch.round(w / s.unsqueeze(1)).clamp_(-127, 127).to(torch.int8)
        scale[lo:hi] = s
    return QWeight(wq, scale)


def int4_weight(n: int, k: int, gen: torch.Generator, group_size: int = 128,
                chunk_rows: int = 8192) -> W4A8Weight:
    """Group-128 int4 weight (contract layout) with fp16-representable scales."""
    assert k % group_size == 0 and k % 2 == 0
    groups = k // group_size
    packed = torch.empty((k // 2, n), dtype=torch.uint8, device=gen.device)
    scale = torch.empty((groups, n), dtype=torch.float32, device=gen.device)
    for lo in range(0, n, chunk_rows):
        hi = min(n, lo + chunk_rows)
        w = dense_weight(hi - lo, k, gen).view(hi - lo, groups, group_size)
        s = _fp16_round(w.abs().amax(dim=-1).clamp_min(1e-8) / 7.0).clamp_min(2.0 ** -24)
        codes = (torch.round(w / s.unsqueeze(-1)).clamp_(-8, 7).to(torch.int32) + 8).view(hi - lo, k)
        packed[:, lo:hi] = (codes[:, 0::2] | (codes[:, 1::2] << 4)).to(torch.uint8).t()
        scale[:, lo:hi] = s.t()
    return W4A8Weight(packed.contiguous(), scale.contiguous(), k=k, group_size=group_size)


def activations(m: int, k: int, gen: torch.Generator, outliers: bool = False) -> torch.Tensor:
    x = torch.randn((m, k), generator=gen, device=gen.device, dtype=torch.float32)
    if outliers:
        mask = torch.rand((m, k), generator=gen, device=gen.device) < 0.01
        x = torch.where(mask, x * 20.0, x)
    return x.to(torch.bfloat16)


def gemv_bytes(m: int, n: int, k: int) -> int:
    """Algorithmic bytes of one int8 weight-only GEMV: weight + fp16 scales + bf16 in/out."""
    return n * k + 2 * n + 2 * m * k + 2 * m * n


def w4_gemv_bytes(m: int, n: int, k: int, group_size: int = 128) -> int:
    """Algorithmic bytes of one W4A8 GEMV on bf16 activations."""
    return (k // 2) * n + 2 * (k // group_size) * n + 2 * m * k + 2 * m * n


def gemm_ops(m: int, n: int, k: int) -> int:
    """int8 operations of one GEMM (a multiply-accumulate counts as two)."""
    return 2 * m * n * k


def quant_bytes(m: int, k: int) -> int:
    return 3 * m * k + 4 * m
