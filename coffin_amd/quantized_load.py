"""Read coffin's pre-quantised checkpoint directories for a row-major (``"nk"``) backend.

coffin writes two on-disk formats (tools/quant_disk.py, tools/quant_disk_w4a8.py; read back by
quantized_load.py:46-51,186-330):

* ``coffin-int8-kn-v1`` -- every quantizable projection as ``int8 [K, N]`` plus a
  ``<key>#scale`` tensor ``fp32 [N]``;
* ``coffin-w4a8-kn-v1`` -- ``uint8 [ceil(K/2), N]`` (low nibble = even k) plus
  ``fp32 [ceil(K/group), N]`` group scales;

both with a ``quant_index.json`` that records, per tensor, its kind, shapes, shard file and scale
key.  coffin's own loader refuses these directories for every backend whose kernels want
``[N, K]`` rows (quantized_load.py:123-141), because it hands out the ``[K, N]`` buffer as a
transposed *view*.  This module is the loader for such a backend: the int8 buffer is transposed
once, on the device it was read to, into the contiguous ``[N, K]`` the GEMV / GEMM kernels stream
(the ``[K, N]`` copy is dropped), and int4 weights keep the contract layout, which
``cmi_w4_repack`` re-lays out on first use.  Nothing is dequantised; dense tensors pass through.

The index is checked before anything is built (format, shapes, dtypes, scale lengths, the
``config.json`` digest): a mismatch would otherwise show up as a shape error many layers later,
or not at all.
"""

from __future__ import annotations

import hashlib
import json
from pathlib import Path
from typing import Any, Callable, Iterable

import torch

from coffin_amd.weights import QWeight, W4A8Weight

INDEX_NAME = "quant_index.json"
FORMAT_INT8 = "coffin-int8-kn-v1"
FORMAT_W4A8 = "coffin-w4a8-kn-v1"
#: Prefixes read by default: the text model, the multi-token-prediction head and an untied lm_head
#: (quantized_load.py:247-249).
DEFAULT_PREFIXES = ("model.language_model.", "mtp.", "lm_head.")

_DTYPES = {"bfloat16": torch.bfloat16, "float16": torch.float16, "float32": torch.float32}


def is_quantized_dir(model_dir: str | Path) -> bool:
    """A directory is pre-quantised exactly when it holds the index file."""
    return (Path(model_dir) / INDEX_NAME).is_file()


def read_index(model_dir: str | Path) -> dict:
    """Parse ``quant_index.json``; unknown formats are refused (bytes laid out differently would
    read back as plausible int8 numbers)."""
    path = Path(model_dir) / INDEX_NAME
    index = json.loads(path.read_text(encoding="utf-8"))
    if index.get("format") not in (FORMAT_INT8, FORMAT_W4A8):
        raise ValueError(f"{path}: unsupported quantized format {index.get('format')!r}")
    if not isinstance(index.get("tensors"), dict):
        raise ValueError(f"{path}: index holds no tensor table")
    return index


def _check_config_digest(model_dir: Path, index: dict) -> None:
    want = index.get("source_config_sha256") or ""
    config = model_dir / "config.json"
    if not want or not config.is_file():
        return
    have = hashlib.sha256(config.read_bytes()).hexdigest()
    if have != want:
        raise ValueError(f"{config} does not belong to these weights "
                         f"(sha256 {have[:12]} != {want[:12]}): the directory mixes two checkpoints")


def _int8_rows(key: str, wt: torch.Tensor, scale: torch.Tensor, meta: dict) -> QWeight:
    """``int8 [K, N]`` + ``fp32 [N]`` from disk -> ``QWeight`` with contiguous ``[N, K]`` rows."""
    if wt.dim() != 2 or wt.dtype != torch.int8:
        raise ValueError(f"{key}: expected a 2-D int8 weight, got {tuple(wt.shape)} {wt.dtype}")
    k, n = int(wt.shape[0]), int(wt.shape[1])
    if [k, n] != list(meta.get("shape") or []):
        raise ValueError(f"{key}: index says shape {meta.get('shape')}, shard holds {[k, n]}")
    if scale.dim() != 1 or scale.dtype != torch.float32 or scale.numel() != n:
        raise ValueError(f"{key}: scale must be fp32 [{n}], got {tuple(scale.shape)} {scale.dtype}")
    return QWeight(wt.t().contiguous(), scale.contiguous())


def _int4_groups(key: str, packed: torch.Tensor, scale: torch.Tensor, meta: dict) -> W4A8Weight:
    if list(packed.shape) != list(meta.get("packed_shape") or []) \
            or list(scale.shape) != list(meta.get("scale_shape") or []):
        raise ValueError(f"{key}: index says packed {meta.get('packed_shape')} / scale "
                         f"{meta.get('scale_shape')}, shard holds {list(packed.shape)} / {list(scale.shape)}")
    return W4A8Weight(packed.contiguous(), scale.contiguous(), k=int(meta["k"]),
                      group_size=int(meta["group_size"]))


def load(model_dir: str | Path, *, device: torch.device | str, quant: bool = True,
         prefixes: Iterable[str] = DEFAULT_PREFIXES, keep: Callable[[str], bool] | None = None,
         weight_dtype: torch.dtype | None = None) -> dict[str, Any]:
    """State dict of a pre-quantised directory, tensors read straight to ``device``.

    ``quant=True``: projections come back as ``QWeight`` (``[N, K]`` int8 rows, fp32 row scales)
    or ``W4A8Weight``; ``quant=False`` dequantises them to ``weight_dtype`` (default: the dtype
    the index records).  ``keep(key)`` filters further (only the layers a caller needs).  Fused
    expert stacks (``q8-moe`` / ``q4-moe``) are not part of this backend's path and are refused.
    """
    from safetensors import safe_open

    model_dir = Path(model_dir)
    index = read_index(model_dir)
    _check_config_digest(model_dir, index)
    stored = index.get("weight_dtype")
    if weight_dtype is None:
        if stored not in _DTYPES:
            raise ValueError(f"{model_dir}: index records dtype {stored!r}, which this loader does not know")
        weight_dtype = _DTYPES[stored]
    elif str(weight_dtype).split(".")[-1] != stored:
        raise ValueError(f"{model_dir}: weights were quantised from {stored}, this load asked for "
                         f"{str(weight_dtype).split('.')[-1]}; the integer codes cannot be reused across dtypes")
    prefixes = tuple(prefixes)
    wanted = {key: meta for key, meta in index["tensors"].items()
              if key.startswith(prefixes) and (keep is None or keep(key))}
    if not wanted:
        raise ValueError(f"{model_dir}: index holds no tensor under prefixes {prefixes}")
    by_shard: dict[str, list[str]] = {}
    for key, meta in wanted.items():
        by_shard.setdefault(meta["shard"], []).append(key)

    out: dict[str, Any] = {}
    for shard in sorted(by_shard):
        path = model_dir / shard
        if not path.is_file():
            raise FileNotFoundError(f"{model_dir}: index names {shard}, which is missing")
        with safe_open(str(path), framework="pt", device=str(torch.device(device))) as handle:
            present = set(handle.keys())
            for key in by_shard[shard]:
                meta = wanted[key]
                if key not in present:
                    raise ValueError(f"{path}: index names {key}, shard does not hold it")
                kind = meta.get("kind")
                if kind in ("q8", "q4"):
                    scale_key = meta.get("scale_key")
                    if scale_key not in present:
                        raise ValueError(f"{path}: {key} has no scale tensor {scale_key}; the codes "
                                         f"without their scales dequantise to a different model")
                    build = _int8_rows if kind == "q8" else _int4_groups
                    w = build(key, handle.get_tensor(key), handle.get_tensor(scale_key), meta)
                    out[key] = w if quant else (w.dequant(weight_dtype) if kind == "q8" else w.to(weight_dtype))
                elif kind in ("q8-moe", "q4-moe"):
                    raise ValueError(f"{path}: {key} is a fused expert stack ({kind}); expert weights are "
                                     f"outside the quantized-linear path this backend serves")
                else:
                    out[key] = handle.get_tensor(key)
    return out
