"""MI355X (gfx950) quantized-linear backend: hand-written HIP kernels behind a C ABI.

Drop-in for the ``linear`` / ``linear_m`` / ``linear_m_verify`` / ``linear_prefill``
/ ``kv_quant`` entries of MuWinds/coffin's backend table (backends/protocol.py:147-159,
:252-258) for ``QWeight`` and ``W4A8Weight`` storage.
"""

__all__ = ["__version__"]
__version__ = "0.1.0"
