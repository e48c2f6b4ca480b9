"""Vendor declaration for AMD Instinct MI355X (gfx950): the drop-in registration door.

Copy (or symlink) this file to ``backends/vendors/mi355x.py`` of a coffin checkout
with the ``coffin_amd`` package importable; ``COFFIN_BACKEND=mi355x`` then selects
it and auto-probing prefers it on an MI355X because a device-name match (claim 2)
outranks the ROCm-build gate of the built-in gfx906 backend
(backends/vendors/__init__.py:8-16, backends/discovery.py:63-91,
backends/registry.py:102-110,139-157).

Import is side-effect free: no library load, no allocation, no device call.  The
kernels are loaded on the first ``build_ops()`` call; a missing or unusable
library yields an empty table there (the resolver then fills every entry from
the torch reference, backends/vendor.py:353-363) instead of crashing selection.
"""

from __future__ import annotations

import torch

try:  # inside a coffin checkout: bind to the real contract classes
    from backends.protocol import Ops
    from backends.vendor import Detection, VendorSpec
except ImportError:  # standalone: the package's own mirror of the same names
    from coffin_amd.contract import Detection, Ops, VendorSpec

#: ISA the kernels are compiled for.
ARCH = "gfx950"


def _device_is_gfx950() -> bool:
    try:
        props = torch.cuda.get_device_properties(0)
    except Exception:
        return False
    return str(getattr(props, "gcnArchName", "")).split(":")[0] == ARCH


def build_ops() -> "Ops":
    """Native entries for the quantized-linear path, or an empty table if unusable."""
    try:
        if not _device_is_gfx950():
            return Ops()
        from coffin_amd import _native, backend
        _native.load()
        return Ops.from_mapping(backend.native_table())
    except Exception:
        return Ops()


def configure(**settings) -> dict:
    """Process-wide switches of the native entries, e.g. ``configure(batch_family="mfma")`` for a
    deployment that decodes static batches (see ``coffin_amd.backend.configure``).  The contract's
    ``VendorSpec`` has no field for backend options, so the door is this module-level function of
    the vendor file; environment variables (``COFFIN_AMD_BATCH_MFMA`` ...) give the initial values."""
    from coffin_amd import backend
    return backend.configure(**settings)


SPEC = VendorSpec(
    name="mi355x",
    detection=Detection(
        namespace="cuda",
        # Boards report "AMD Instinct MI355X".  A host without the amdgpu id table
        # reports the generic "AMD Radeon Graphics" for every AMD part; claiming
        # that name would take non-gfx950 devices away from the backend written
        # for them, so such hosts select this backend by name
        # (COFFIN_BACKEND=mi355x).  build_ops() checks the ISA either way.
        name_markers=("mi355", "mi350"),
        hip=True,
    ),
    act_dtype=torch.bfloat16,
    weight_dtype=torch.bfloat16,
    # The adapters are capture-safe once a warm-up step has touched every weight (they launch on the
    # current stream, never synchronise and keep no per-call host state); a captured 129-projection
    # decode step runs in 0.82 ms against 0.98 ms launched eagerly (7 us of host time per call
    # in front of a 6.3 us kernel), so decode should be captured.
    graph=True,
    autotune=False,
    int8_weights=True,
    batch_attn=False,
    attn_split=1,
    weight_layout="nk",
    priority=50,
    notes="native: linear, linear_m, linear_m_verify, linear_prefill, kv_quant, silu_mul, "
          "silu_mul_quant, rms_norm, add_rms_norm; everything else runs the torch reference",
    has_kernels=True,
    build_ops=build_ops,
)
