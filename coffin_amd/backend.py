"""Adapters behind the ``linear*`` / ``kv_quant`` table entries on MI355X.

Each module-level function whose name is a contract name is that op's native
entry (the name-is-registration rule of backends/protocol.py:582-612); the
vendor file collects them into the ``Ops`` table.  Signatures, return shapes
and error behaviour follow backends/protocol.py:143-159,252-258 and the corex
adapters they stand in for (backends/corex/__init__.py:396-425 ``linear``,
:495-546 ``_gemv_rows``, :576-651 ``_w4_rows``, :1557-1609 ``_w8a8_rows``,
:1612-1670 ``linear_prefill``).

Routing, by storage type first (never by op name), then by row count:

=================  ==========================  =================================
weight             rows                        kernel
=================  ==========================  =================================
QWeight (int8)     linear, linear_m            int8 weight-only dot-product GEMV, 16
                                               rows at a time (row r == linear(x[r]))
QWeight            >= 3, linear_m_verify and   weight-only GEMV on the matrix pipe,
                   linear_prefill below 64     16 rows at a time
QWeight            >= 64, linear_prefill       per-token quant + W8A8 MFMA GEMM
QWeight            >= 2, linear_m_verify with  per-token quant + W8A8 (weight read
                   COFFIN_AMD_W8A8_VERIFY=1    once up to 16 rows, tiled beyond)
W4A8Weight         1..16                       per-token quant + W4A8 GEMV
W4A8Weight         > 16                        per-token quant + W4A8 MFMA GEMM
plain tensor       any                         torch ``F.linear`` (not quantized,
                                               outside this backend's scope)
=================  ==========================  =================================

Everything launches on torch's current stream; nothing synchronises or reads
device memory on the host.  Outputs are fresh tensors; ``xq``/``xs`` scratch is
private and cached by shape; weights are borrowed and never modified (the int4
re-layout is a private copy made once per weight).
"""

from __future__ import annotations

import os
import weakref
from collections import OrderedDict

import torch
import torch.nn.functional as F

from coffin_amd import _native

#: Widest batch the GEMV kernels take in one launch.
GEMV_MAX_ROWS = 16
#: The matrix-pipe weight-only GEMV takes this many (the weight is read once, the activation rows
#: go through in chunks of 16 inside the kernel: same bits as 16-row calls).
GEMV_MFMA_MAX_ROWS = 64
#: From this many rows ``linear_prefill`` quantizes activations and runs the
#: int8 MFMA GEMM (the reference's corex backend draws the same line at 64,
#: backends/corex/__init__.py:633,1655-1659).
PREFILL_MIN_ROWS = 64

#: ``linear_m_verify`` on int8 weights may answer with W8A8 arithmetic (per-token
#: int8 activations) instead of the weight-only GEMV: the contract allows it
#: (backends/protocol.py:152-155) and corex keeps the same switch, off by default,
#: as ``COFFIN_COREX_W8A8_DP4A_VERIFY`` (backends/corex/__init__.py:119-131,
#: 450-494).  Off by default here too, so verify and decode share their numerics
#: unless asked; on, a 16-row verify of a 2560 -> 9728 projection takes 8 us
#: instead of 32 (the weight is read once, the sums run on the matrix pipe).
W8A8_VERIFY = os.environ.get("COFFIN_AMD_W8A8_VERIFY", "0").strip() == "1"
#: Static-batch decode owes its users "row r of a batch equals the single-row call on x[r]", bit
#: for bit (models/qwen35/batch.py:19-22: a batched and an unbatched request must give the same
#: numbers), so ``linear`` and ``linear_m`` on int8 weights stay on the dot-product GEMV, whose
#: summation order depends on K only.  ``linear_m_verify`` (which may use a path of its own,
#: backends/protocol.py:152-155) and short ``linear_prefill`` chunks do not carry that obligation
#: and take the matrix-pipe GEMV from three rows up: 1.5-2.8 times faster at 8-16 rows, same
#: weight-only arithmetic, last-place differences from fp32 summation order.
#: ``COFFIN_AMD_BATCH_MFMA=1`` moves *every* int8 weight-only call -- ``linear`` included, one row
#: included -- to the matrix-pipe GEMV: the contract holds again (one kernel family, a row's bits
#: independent of its batch), static batches of 4-16 requests run 1.05-2.8 times faster, and
#: single-stream decode pays for it (7.9 us instead of 6.3 us for 2560 -> 9728).  A deployment choice.
BATCH_MFMA = os.environ.get("COFFIN_AMD_BATCH_MFMA", "0").strip() == "1"
#: int4 weights are answered with W4A8 arithmetic (per-token int8 activations), which is what coffin
#: runs on its native backends.  ``COFFIN_AMD_W4A16=1`` keeps the activations unquantised instead for
#: decode-sized calls (up to ``W4A16_MAX_ROWS`` rows, K <= ``W4A16_MAX_K``): the int4 weight-only GEMV, i.e. the
#: arithmetic of the reference's torch path for an int4 weight (backends/reference/__init__.py:93-95)
#: up to fp32 summation order; one launch per row, so it is meant for single-stream decode.
W4A16 = os.environ.get("COFFIN_AMD_W4A16", "0").strip() == "1"
W4A16_MAX_ROWS = 4
W4A16_MAX_K = 32768
#: Rows from which the matrix-pipe GEMV beats the dot-product one (measured on every layer shape).
MFMA_MIN_ROWS = 3
#: ``rms_norm`` / ``add_rms_norm`` / ``silu_mul`` also leave their output rows quantised (int8 +
#: scale) in private scratch, and a ``linear*`` call on that very output -- W4A8 at any row count,
#: W8A8 prefill -- takes them from there instead of quantising the bf16 rows again: the
#: reference's own call sequence (``ops/norm.py:87`` then ``ops/gemv.py:75``;
#: ``models/qwen35/blocks.py:69``) then runs the projection kernels on quantised rows, as a caller
#: of ``rms_norm_i8`` + ``linear_quantized`` would.  Same bits (the producers quantise the stored
#: bf16 values with the quantiser's arithmetic).  ``COFFIN_AMD_HANDOVER=0`` or
#: ``configure(handover=False)`` switches it off.
HANDOVER = os.environ.get("COFFIN_AMD_HANDOVER", "1").strip() != "0"
#: Largest block of rows (bytes of int8) a producer leaves behind.
HANDOVER_MAX_BYTES = 128 << 20
#: Fewest rows a producer hands over.  A single row is not worth it: at one row every kernel here
#: runs at its launch floor, quantising costs about 1 us wherever it is done (a second
#: workgroup-wide reduction in the producer: rms_norm 2.6 -> 3.6 us, silu_mul 2.9 -> 4.6 us), and the
#: one-row GEMVs that quantise for themselves lose only 0.4 / 1.1 / 1.9 us to it (qkv / gate_up /
#: down): the 129-projection step measured 1.042 ms handed against 1.058 ms not.  From two rows up
#: the projection would otherwise launch the quantiser in front of its kernel (2.5 .. 4 us).
HANDOVER_MIN_ROWS = 2

_FAMILIES = {"dot": 0, "mfma": 1}


def configure(*, batch_family: str | None = None, w8a8_verify: bool | None = None,
              w4a16: bool | None = None, handover: bool | None = None) -> dict:
    """Process-wide switches of this backend, settable after import (the environment variables
    above give the initial values).  Returns the settings in force.

    ``batch_family``: ``"dot"`` -- ``linear`` / ``linear_m`` on int8 weights run the dot-product
    GEMV (fastest single row; 4-16 rows are vector-ALU bound) -- or ``"mfma"`` -- every int8
    weight-only call, single rows included, runs the matrix-pipe GEMV (4-16 rows 1.05-2.8 times
    faster, a single row slower).  Either way row r of a batch carries the bits of the single-row
    call (models/qwen35/batch.py:19-22): the rule needs one family per weight, not a particular
    one.  A weight object may carry its own choice in an attribute ``batch_family`` (read when the
    weight is first used), e.g. ``"mfma"`` for the projections of a model served in static batches.
    """
    global BATCH_MFMA, W8A8_VERIFY, W4A16, HANDOVER
    if batch_family is not None:
        if batch_family not in _FAMILIES:
            raise ValueError(f"batch_family must be 'dot' or 'mfma', got {batch_family!r}")
        BATCH_MFMA = batch_family == "mfma"
    if w8a8_verify is not None:
        W8A8_VERIFY = bool(w8a8_verify)
    if w4a16 is not None:
        W4A16 = bool(w4a16)
    if handover is not None:
        HANDOVER = bool(handover)
        _drop_handed()
    return {"batch_family": "mfma" if BATCH_MFMA else "dot", "w8a8_verify": W8A8_VERIFY, "w4a16": W4A16,
            "handover": HANDOVER}


def _vp(address: int) -> int:
    """Pointer argument: the entry points declare ``void *`` (``argtypes``), so a plain int passes."""
    return address


def _ptr(t: torch.Tensor | None) -> int:
    return t.data_ptr() if t is not None else 0


# The adapters run once per projection and token; what they do on the host is part of the decode
# path (corex measured 36 us per call for its W4A8 adapter, backends/corex/__init__.py:580-585).
# ``torch.cuda.current_stream()`` builds a Stream object through three layers of Python (several
# microseconds); the raw getter behind it returns the handle directly.
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_raw_device = getattr(torch._C, "_cuda_getDevice", None)


def _stream() -> int:
    """Handle of torch's current stream on the current device."""
    if _raw_stream is not None:
        return _raw_stream(_current_device())
    return torch.cuda.current_stream().cuda_stream


def _current_device() -> int:
    return _raw_device() if _raw_device is not None else torch.cuda.current_device()


def _is_w4(w) -> bool:
    return hasattr(w, "packed") and hasattr(w, "group_size")


def _is_q8(w) -> bool:
    return hasattr(w, "wq") and hasattr(w, "scale")


def _on_gpu(t: torch.Tensor) -> bool:
    return t.device.type == "cuda"


# --------------------------------------------------------------- private state

class _Arena:
    """One grow-only block of device memory per (purpose, device) that is never handed back.

    A captured HIP graph holds raw addresses of whatever scratch its kernels were launched with
    (quantised rows, split-K arrival counters and partial tiles), so scratch that a later call
    could free -- a pool that evicts by shape, say -- would be rewritten under a replay once the
    allocator reuses it.  Here a request larger than the block allocates a new block of at least
    twice the size and *retires* the old one: it stays allocated until the process ends, so every
    address ever handed out stays valid, and the memory held is at most twice the largest request.
    Calls are serialised on one stream by contract (backends/corex/__init__.py:656-658), so one
    block serves every shape: a projection's scratch is dead when the next projection starts.
    Growth allocates, which a stream capture must not do: the warm-up step that precedes a capture
    (engine/llm_engine.py:116) sizes the block, and growth under capture raises."""

    _ROUND = 1 << 20

    def __init__(self, purpose: str) -> None:
        self.purpose = purpose
        self.blocks: dict = {}      # device index -> uint8 tensor
        self.retired: list = []     # outgrown blocks, kept alive for graphs that captured them

    def take(self, nbytes: int, device: torch.device) -> int:
        """Address of at least ``nbytes`` bytes (256-byte aligned) on ``device``."""
        block = self.blocks.get(device.index)
        if block is None or block.numel() < nbytes:
            if device.type == "cuda" and torch.cuda.is_current_stream_capturing():
                raise RuntimeError(f"coffin_amd: {self.purpose} scratch must grow to {nbytes} bytes inside a "
                                   "graph capture; run one eager step over the same shapes before capturing")
            size = max(nbytes, 2 * block.numel() if block is not None else 0)
            size = (size + self._ROUND - 1) // self._ROUND * self._ROUND
            if block is not None:
                self.retired.append(block)
            block = torch.empty(size, dtype=torch.uint8, device=device)
            self.blocks[device.index] = block
        return block.data_ptr()


#: Workspace of the fused quantiser + projection entries (quantised rows, scales, split-K room).
_WORKSPACE = _Arena("projection")
#: (rows, n, k) -> bytes the library asks for; a few integers per distinct shape.
_WORKSPACE_BYTES: dict = {}


def _scratch(rows: int, k: int, device: torch.device, n: int = 0):
    """``(address, bytes)`` of the workspace for one projection; with ``n`` (int8 weights) sized so
    that the W8A8 entry may split K where that pays."""
    key = (rows, n, k)
    nbytes = _WORKSPACE_BYTES.get(key)
    if nbytes is None:
        lib = _native.load()
        nbytes = int(lib.cmi_linear_w8a8_workspace_bytes(rows, n, k) if n else lib.cmi_linear_workspace_bytes(rows, k))
        if len(_WORKSPACE_BYTES) >= 65536:
            _WORKSPACE_BYTES.clear()
        _WORKSPACE_BYTES[key] = nbytes
    return _WORKSPACE.take(nbytes, device), nbytes


#: id(source tensor) -> device-layout copy, dropped when the source dies
#: (same ownership rule as backends/corex/pack.py:323-359).
_REPACKED: dict = {}


def _memo(source: torch.Tensor, make):
    key = id(source)
    hit = _REPACKED.get(key)
    if hit is not None and hit[0]() is source:
        return hit[1]
    value = make()
    ref = weakref.ref(source, lambda _r, key=key: _REPACKED.pop(key, None))
    _REPACKED[key] = (ref, value)
    return value


def _q8_operands(w):
    """``(wq int8 [N,K] contiguous, scale fp32 [N] contiguous)`` for a QWeight-like."""
    wq, scale = w.wq, w.scale
    if wq.dtype != torch.int8 or wq.dim() != 2:
        raise ValueError(f"int8 weight must be 2-D int8, got {tuple(wq.shape)} {wq.dtype}")
    if not wq.is_contiguous():
        # e.g. a [K,N]-stored weight exposed as a transposed view: one private
        # row-major copy, made once.
        wq = _memo(w.wq, lambda: w.wq.contiguous())
    if scale.dtype != torch.float32 or not scale.is_contiguous():
        scale = _memo(w.scale, lambda: w.scale.to(torch.float32).contiguous())
    return wq, scale


def _w4_check(w) -> None:
    """Refuse a W4A8Weight-like whose buffers are not what the re-layout kernel reads.

    The adapter accepts any object with ``packed`` / ``scale`` / ``k`` / ``n`` / ``group_size``;
    the kernel reads ``K/2 * N`` bytes and ``K/gs * N`` floats from raw addresses, so dtype,
    contiguity, device and shape are checked here (the reference's own class checks the same in
    its constructor, w4a8_weights.py:35-44).
    """
    n, k, gs = int(w.n), int(w.k), int(w.group_size)
    packed, scale = w.packed, w.scale
    if packed.dtype != torch.uint8 or packed.dim() != 2 or not packed.is_contiguous():
        raise ValueError(f"int4 weight: packed must be contiguous 2-D uint8, got "
                         f"{tuple(packed.shape)} {packed.dtype}")
    if packed.shape[1] != n or gs < 1 or packed.shape[0] * 2 < -(-k // gs) * gs:
        raise ValueError(f"int4 weight: packed {tuple(packed.shape)} does not hold K={k} x N={n} codes")
    if scale.dtype != torch.float32 or scale.dim() != 2 or not scale.is_contiguous():
        raise ValueError(f"int4 weight: scale must be contiguous 2-D fp32, got "
                         f"{tuple(scale.shape)} {scale.dtype}")
    if tuple(scale.shape) != (-(-k // gs), n):
        raise ValueError(f"int4 weight: scale {tuple(scale.shape)} does not match "
                         f"[{-(-k // gs)}, {n}] (K={k}, group size {gs})")
    if packed.device.type != "cuda" or scale.device != packed.device:
        raise ValueError(f"int4 weight: packed on {packed.device} and scale on {scale.device} "
                         f"must share a GPU")


def _kernels_take(w) -> bool:
    """Whether the native kernels are built for this quantized weight's shape.

    int4: group sizes 64, 128 and 256, any K (rows are padded to whole groups on the device);
    int8: K a multiple of 16.  Other shapes are answered by the torch statement of the op (the
    reference's corex adapter likewise falls back for group sizes its GEMM does not take,
    backends/corex/__init__.py:633).
    """
    if _is_w4(w):
        gs, k = int(w.group_size), int(w.k)
        # whole groups in storage, as the encoder writes them (tools/quant_disk_w4a8.py:60-66)
        return gs in (64, 128, 256) and k >= 1 and int(w.packed.shape[0]) * 2 >= -(-k // gs) * gs
    return int(w.wq.shape[-1]) % 16 == 0


def _w4_operands(w):
    """Device layout ``(w4 uint8 [N,Kd/2], ws fp32 [N,Kd/gs])`` of a W4A8Weight-like, built once
    (``Kd``: K rounded up to whole groups and whole 128-element steps, ``cmi_w4_device_k``)."""
    def make():
        _w4_check(w)
        n, k, gs = int(w.n), int(w.k), int(w.group_size)
        lib = _native.load()
        kd = int(lib.cmi_w4_device_k(k, gs))
        w4 = torch.empty((n, kd // 2), dtype=torch.uint8, device=w.packed.device)
        ws = torch.empty((n, kd // gs), dtype=torch.float32, device=w.packed.device)
        with torch.cuda.device(w.packed.device):
            _native.check(lib.cmi_w4_repack(_ptr(w.packed), _ptr(w.scale), _ptr(w4), _ptr(ws),
                                            n, k, gs, _stream()), "w4 re-layout")
        return w4, ws
    return _memo(w.packed, make)


# ------------------------------------------------- quantised rows handed forward

class _Handed:
    """The latest producer output and where its quantised rows are.  ``tensor`` is a strong
    reference on purpose: while it lives no other allocation can have its address, so an
    activation with the same address, layout and version counter *is* this tensor's memory."""

    __slots__ = ("tensor", "version", "ptr", "rows", "k", "ld", "dev", "xq", "xs", "capture")


_HANDED: _Handed | None = None
_HANDOVER_ARENA = _Arena("quantised-row hand-over")
#: Producers start leaving quantised rows behind once a projection has quantised activations in
#: this process (a model of plain or weight-only int8 decode never pays for rows nobody reads).
_QUANT_CONSUMER_SEEN = False


def _round256(v: int) -> int:
    return (v + 255) // 256 * 256


def _drop_handed() -> None:
    global _HANDED
    _HANDED = None


def _drop_handed_if_written(*written) -> None:
    """Forget the handed rows when one of this backend's own ops writes into their tensor (torch
    ops announce their writes through the version counter; these kernels do not)."""
    h = _HANDED
    if h is None:
        return
    home = h.tensor.untyped_storage().data_ptr()
    for t in written:
        if t is not None and t.device == h.dev and t.untyped_storage().data_ptr() == home:
            _drop_handed()
            return


def _capture_id(stream: int) -> int:
    return int(_native.load().cmi_stream_capture_id(stream))


def _hand_target(rows: int, k: int, device: torch.device):
    """``(xq address, xs address)`` for a producer of ``rows x k`` outputs, or ``None`` when it
    should not leave quantised rows behind."""
    if not (HANDOVER and _QUANT_CONSUMER_SEEN) or rows < HANDOVER_MIN_ROWS or rows * k > HANDOVER_MAX_BYTES:
        return None
    try:
        base = _HANDOVER_ARENA.take(_round256(rows * k) + _round256(4 * rows), device)
    except RuntimeError:
        return None                      # would have to grow inside a capture: this call goes without
    return base, base + _round256(rows * k)


def _hand_over(t: torch.Tensor, rows: int, k: int, ld: int, target, stream: int) -> None:
    global _HANDED
    h = _Handed()
    h.tensor, h.version, h.ptr, h.rows, h.k, h.ld, h.dev = t, t._version, t.data_ptr(), rows, k, ld, t.device
    h.xq, h.xs = target
    # a graph must not read rows that a kernel outside it wrote (nor the other way round): the
    # consumer has to be recorded into the same capture as the producer, or both run eagerly
    h.capture = _capture_id(stream)
    _HANDED = h


def _handed_rows(x: torch.Tensor, rows: int, k: int, stream: int):
    """The quantised copy of ``x`` left by the producer that wrote it, or ``None``."""
    h = _HANDED
    if h is None or x.data_ptr() != h.ptr or rows != h.rows or k != h.k or x._version != h.version \
            or x.device != h.dev:
        return None
    if x.stride(-1) != 1 or (x.dim() == 2 and rows > 1 and x.stride(0) != h.ld):
        return None
    if _capture_id(stream) != h.capture:
        return None
    return h.xq, h.xs


# ------------------------------------------------------------------- kernels

def _quantize_rows(act: torch.Tensor, xq: torch.Tensor, xs: torch.Tensor, rows: int, k: int) -> None:
    rc = _native.load().cmi_quant_act_i8(act.data_ptr(), xq.data_ptr(), xs.data_ptr(), rows, k, _stream())
    if rc:
        _native.check(rc, "quant_act_i8")


class _Record:
    """What the adapters need of one quantized weight, resolved once: operand addresses in
    device layout, shape, device.  Holds no strong reference to the caller's tensors."""

    __slots__ = ("kind", "src", "src2", "a", "b", "n", "k", "kd", "gs", "dev", "family")


#: id(weight object) -> _Record; an entry is trusted only while the tensors it was
#: built from are still the ones the weight object holds.
_RECORDS: OrderedDict = OrderedDict()
_RECORDS_MAX = 8192


def _lookup(w) -> _Record | None:
    key = id(w)
    rec = _RECORDS.get(key)
    if rec is None:
        return None
    try:
        first = w.wq if rec.kind == 8 else w.packed
        if rec.src() is first and rec.src2() is w.scale:
            _RECORDS.move_to_end(key)
            return rec
    except AttributeError:
        pass
    return None


def _make_record(w) -> _Record:
    # A weight is resolved (and an int4 weight re-laid out into a private copy) on its first use.
    # Under stream capture that copy would live in the graph's memory pool and the re-layout would
    # be replayed with every step: the callers' warm-up step (the reference's engine runs one
    # before it captures, engine/llm_engine.py:116) must have touched every weight already.
    if torch.cuda.is_available() and torch.cuda.is_current_stream_capturing():
        raise RuntimeError("coffin_amd: first use of a quantized weight inside graph capture; "
                           "run one eager step over every projection before capturing")
    rec = _Record()
    if _is_w4(w):
        w4, ws = _w4_operands(w)
        rec.kind, rec.src, rec.a, rec.b = 4, weakref.ref(w.packed), w4.data_ptr(), ws.data_ptr()
        rec.n, rec.k, rec.gs, rec.dev = int(w.n), int(w.k), int(w.group_size), w.packed.device
        rec.kd = 2 * int(w4.shape[1])
    else:
        wq, scale = _q8_operands(w)
        rec.kind, rec.src, rec.a, rec.b = 8, weakref.ref(w.wq), wq.data_ptr(), scale.data_ptr()
        rec.n, rec.k, rec.gs, rec.dev = int(wq.shape[0]), int(wq.shape[1]), 0, w.wq.device
        rec.kd = rec.k
    family = getattr(w, "batch_family", None)
    if family is not None and family not in _FAMILIES:
        raise ValueError(f"batch_family of a weight must be 'dot' or 'mfma', got {family!r}")
    rec.family = family
    rec.src2 = weakref.ref(w.scale)
    _RECORDS.pop(id(w), None)                     # a stale entry under a reused id
    while len(_RECORDS) >= _RECORDS_MAX:
        _RECORDS.popitem(last=False)              # least recently used weight goes first
    _RECORDS[id(w)] = rec
    return rec


def _gemv_q8(rec: _Record, act: torch.Tensor, rows: int, out: torch.Tensor, mfma: bool = False) -> None:
    """Weight-only projection, one native call for any number of rows.  ``mfma``: the call site may
    use the matrix-pipe family (verify, short prefill chunks: from ``MFMA_MIN_ROWS`` rows); a weight
    or a process whose family is "mfma" uses it for every call, single rows included."""
    n, k = rec.n, rec.k
    whole = rec.family == "mfma" if rec.family is not None else BATCH_MFMA
    fast = (whole or (mfma and rows >= MFMA_MIN_ROWS)) and k % 128 == 0
    rc = _native.load().cmi_linear_w8a16(rec.a, rec.b, act.data_ptr(), out.data_ptr(), rows, n, k,
                                         1 if fast else 0, _stream())
    if rc:
        _native.check(rc, "linear_w8a16")


def _gemm_q8(rec: _Record, act: torch.Tensor, rows: int, out: torch.Tensor) -> None:
    global _QUANT_CONSUMER_SEEN
    _QUANT_CONSUMER_SEEN = True
    n, k = rec.n, rec.k
    work, nbytes = _scratch(rows, k, act.device, n)
    rc = _native.load().cmi_linear_w8a8_bf16(act.data_ptr(), rec.a, rec.b, out.data_ptr(), rows, n, k, n,
                                             work, nbytes, _stream())
    if rc:
        _native.check(rc, "linear_w8a8_bf16")


def _rows_w4(rec: _Record, act: torch.Tensor, rows: int, out: torch.Tensor) -> None:
    """Quantiser + W4A8 GEMV or GEMM in one native call; the library picks the route (one launch
    with the quantiser folded into the GEMV for one or two rows, else two launches)."""
    global _QUANT_CONSUMER_SEEN
    _QUANT_CONSUMER_SEEN = True
    n, k = rec.n, rec.k
    work, nbytes = _scratch(rows, rec.kd, act.device)
    rc = _native.load().cmi_linear_w4a8_bf16(rec.a, rec.b, act.data_ptr(), out.data_ptr(), rows, n, k, rec.gs,
                                             work, nbytes, _stream())
    if rc:
        _native.check(rc, "linear_w4a8_bf16")


def _rows_quantised(rec: _Record, xq: int, xs: int, rows: int, out: torch.Tensor, stream: int) -> None:
    """Projection of rows that are already int8 + scale (addresses): W4A8 GEMV / GEMM or the W8A8 GEMM."""
    lib = _native.load()
    if rec.kind == 4:
        fn = lib.cmi_gemv_w4a8 if rows <= 16 else lib.cmi_gemm_w4a8
        rc = fn(rec.a, rec.b, xq, xs, out.data_ptr(), None, rows, rec.n, rec.k, rec.gs, stream)
    else:
        rc = lib.cmi_gemm_w8a8(xq, rec.a, xs, rec.b, out.data_ptr(), None, rows, rec.n, rec.k, rec.n, stream)
    if rc:
        _native.check(rc, "projection of quantised rows")


def _splits_k(rows: int, n: int, k: int, device: torch.device) -> bool:
    """Whether the W8A8 entry would be given room to split K for this shape (it then needs the
    quantiser's launch in front of it, which clears the arrival counters)."""
    return _scratch(rows, k, device, n)[1] != _scratch(rows, k, device)[1]


def _rows_w4a16(rec: _Record, act: torch.Tensor, rows: int, out: torch.Tensor) -> None:
    """int4 weight-only GEMV on unquantised activations, one launch per row."""
    n, k = rec.n, rec.k
    lib = _native.load()
    stream = _stream()
    x0, y0 = act.data_ptr(), out.data_ptr()
    for r in range(rows):
        rc = lib.cmi_gemv_w4a16(rec.a, rec.b, x0 + r * k * 2, y0 + r * n * 2, n, k, rec.gs, stream)
        if rc:
            _native.check(rc, "gemv_w4a16")


# ------------------------------------------------------------------ dispatch

def _dense(w, x: torch.Tensor) -> torch.Tensor:
    """Unquantized or non-bf16 call: the torch statement of the op, on x's device.

    Same arithmetic as backends/reference/__init__.py:93-95; used for plain
    tensors and for activation dtypes the kernels are not built for.
    """
    compute = torch.promote_types(x.dtype, torch.bfloat16)
    if _is_q8(w):
        dense = (w.wq.to(torch.float32) * w.scale.unsqueeze(1)).to(compute)
    elif _is_w4(w):
        dense = w.to(compute)
    else:
        dense = w.to(compute)
    return F.linear(x.to(compute), dense).to(x.dtype)


def _project(w, x: torch.Tensor, prefill: bool, min_rows: int = PREFILL_MIN_ROWS,
             mfma: bool = False) -> torch.Tensor:
    rec = _lookup(w)
    if rec is None and not (_is_w4(w) or _is_q8(w)):
        return _dense(w, x)
    dev = x.device
    if dev.type != "cuda":
        # A CPU tensor cannot reach the kernels and this backend has no CPU
        # path for quantized weights: refuse instead of answering slowly.
        raise ValueError("coffin_amd: quantized weights need activations on the GPU, "
                         f"got {x.device}")
    if x.dtype != torch.bfloat16 or (rec is None and not _kernels_take(w)):
        return _dense(w, x)
    k = rec.k if rec is not None else int(w.k)
    nd = x.dim()
    if nd not in (1, 2) or x.shape[-1] != k:
        raise ValueError(f"projection expects [K] or [M, K] activations with K={k}, "
                         f"got {tuple(x.shape)}")
    wdev = rec.dev if rec is not None else (w.packed if _is_w4(w) else w.wq).device
    if dev != wdev:
        raise ValueError(f"weight on {wdev} and activation on {x.device} must share a device")
    if _current_device() != dev.index:
        with torch.cuda.device(dev):
            return _project(w, x, prefill, min_rows, mfma)
    if rec is None:
        rec = _make_record(w)
    rows = 1 if nd == 1 else x.shape[0]
    # a [K] activation is one row answered as [N]: no view juggling on the decode path
    out = torch.empty((rec.n,) if nd == 1 else (rows, rec.n), dtype=torch.bfloat16, device=dev)
    if rows == 0:
        return out
    w4a16 = rec.kind == 4 and W4A16 and rows <= W4A16_MAX_ROWS and rec.k <= W4A16_MAX_K and rec.gs == 128 and rec.kd == rec.k
    quantising = (rec.kind == 4 and not w4a16) or (rec.kind == 8 and prefill and rows >= min_rows)
    if quantising and _HANDED is not None and rec.kd == rec.k:
        # the rows a producer of this backend left behind for exactly this tensor
        stream = _stream()
        handed = _handed_rows(x, rows, rec.k, stream)
        if handed is not None and (rec.kind == 4 or not _splits_k(rows, rec.n, rec.k, dev)):
            _rows_quantised(rec, handed[0], handed[1], rows, out, stream)
            return out
    act = x if x.is_contiguous() else x.contiguous()
    if rec.kind == 4:
        if w4a16:
            _rows_w4a16(rec, act, rows, out)
        else:
            _rows_w4(rec, act, rows, out)
    elif prefill and rows >= min_rows:
        _gemm_q8(rec, act, rows, out)
    else:
        _gemv_q8(rec, act, rows, out, mfma)
    return out


def linear(w, x: torch.Tensor) -> torch.Tensor:
    """``linear(w, x) -> y``: ``x`` ``[K]`` or ``[C, K]``, ``y`` ``[N]`` or ``[C, N]``, dtype of ``x``."""
    return _project(w, x, prefill=False)


def linear_m(w, x: torch.Tensor) -> torch.Tensor:
    """``linear_m(w, x[M, K]) -> [M, N]``: one weight read serves all rows; row r carries the bits
    of ``linear(w, x[r])`` (in either kernel family: both entries switch together, see :func:`configure`)."""
    return _project(w, x, prefill=False)


def linear_m_verify(w, x: torch.Tensor) -> torch.Tensor:
    """Speculative-verify batches.

    int8 weights: weight-only arithmetic on the matrix-pipe GEMV from three rows up (a row's
    bits do not depend on the batch, but are not those of ``linear``); with ``W8A8_VERIFY``
    set, at least two bf16 rows on the GPU take quantiser + W8A8 instead (same conditions as
    backends/corex/__init__.py:462-485: ``QWeight`` only, rows >= 2).  int4 weights: as
    ``linear_m`` (exact integer sums, one summation order everywhere).
    """
    if (W8A8_VERIFY and _is_q8(w) and x.dim() == 2 and x.shape[0] >= 2 and _on_gpu(x)
            and x.dtype == torch.bfloat16 and int(w.k) % 16 == 0 and x.shape[-1] == int(w.k)):
        return _project(w, x, prefill=True, min_rows=2)
    return _project(w, x, prefill=False, mfma=True)


def linear_prefill(w, x: torch.Tensor) -> torch.Tensor:
    """``linear_prefill(w, x[C, K]) -> [C, N]``: the GEMM regime (W8A8 from 64 rows up; shorter
    chunks of int8 weights stay weight-only, on the matrix-pipe GEMV)."""
    return _project(w, x, prefill=True, mfma=True)


def linear_quantized(w, xq: torch.Tensor, xs: torch.Tensor) -> torch.Tensor:
    """Projection of rows that arrive already quantised: ``xq`` int8 ``[M, K]`` and ``xs`` fp32
    ``[M]`` as written by :func:`rms_norm_i8` / :func:`silu_mul_quant` / :func:`kv_quant`, result
    bf16 ``[M, N]`` -- W8A8 for an int8 weight, W4A8 for an int4 one, bit for bit what
    ``linear_prefill`` (int8, from 64 rows) or ``linear`` (int4) returns for the bf16 rows those
    were quantised from, without reading them again.  Not a table entry of the contract (the
    reference consumes quantised rows inside its own MoE ops, models/qwen35/moe.py:306-307,
    backends/corex/__init__.py:736-760); offered to callers that fuse a norm or an activation with
    the projection behind it."""
    if not (_is_w4(w) or _is_q8(w)):
        raise ValueError("linear_quantized needs a quantized weight")
    if xq.dim() != 2 or xq.dtype != torch.int8 or xs.dtype != torch.float32 or xs.numel() != xq.shape[0]:
        raise ValueError("linear_quantized expects xq int8 [M, K] and xs fp32 [M]")
    if not (_on_gpu(xq) and xs.device == xq.device and xq.is_contiguous() and xs.is_contiguous()):
        raise ValueError("linear_quantized: xq and xs must be contiguous on one GPU")
    rec = _lookup(w)
    if rec is None:
        if not _kernels_take(w):
            raise ValueError("linear_quantized: the kernels are not built for this weight's shape")
        wdev = (w.packed if _is_w4(w) else w.wq).device
        if wdev != xq.device:
            raise ValueError(f"weight on {wdev} and activation on {xq.device} must share a device")
        if _current_device() != xq.device.index:
            with torch.cuda.device(xq.device):
                return linear_quantized(w, xq, xs)
        rec = _make_record(w)
    if rec.dev != xq.device:
        raise ValueError(f"weight on {rec.dev} and activation on {xq.device} must share a device")
    if _current_device() != xq.device.index:
        with torch.cuda.device(xq.device):
            return linear_quantized(w, xq, xs)
    rows, k = xq.shape
    if k != rec.k:
        raise ValueError(f"linear_quantized expects K={rec.k}, got {k}")
    if rec.kd != rec.k:
        raise ValueError(f"linear_quantized: this weight's rows are padded to {rec.kd} on the device; "
                         "pass bf16 rows to linear*, which pads the quantised rows itself")
    out = torch.empty((rows, rec.n), dtype=torch.bfloat16, device=xq.device)
    if rows == 0:
        return out
    _rows_quantised(rec, xq.data_ptr(), xs.data_ptr(), rows, out, _stream())
    return out


def kv_quant(x: torch.Tensor, out_q: torch.Tensor, out_s: torch.Tensor) -> torch.Tensor:
    """Per-row symmetric int8 quantisation into caller-owned ``out_q`` / ``out_s``.

    ``s = max(amax|x|, 1e-5)/127``, ``q = clamp(rne(x/s), -127, 127)``
    (backends/reference/__init__.py:386-389).  bf16 rows on the GPU run the
    kernel; other inputs take the same formula in torch.
    """
    if x.dim() != 2 or tuple(out_q.shape) != tuple(x.shape) or out_s.numel() != x.shape[0]:
        raise ValueError("kv_quant expects x [M, N], out_q [M, N], out_s [M]")
    native_ok = (_on_gpu(x) and x.dtype == torch.bfloat16 and x.is_contiguous()
                 and out_q.dtype == torch.int8 and out_q.is_contiguous()
                 and out_s.dtype == torch.float32 and out_s.is_contiguous()
                 and out_q.device == x.device and out_s.device == x.device)
    if not native_ok:
        xf = x.to(torch.float32)
        s = xf.abs().amax(dim=-1).clamp_min(1e-5) / 127.0
        out_s.copy_(s.reshape(out_s.shape))
        out_q.copy_(torch.round(xf / s.unsqueeze(-1)).clamp_(-127, 127).to(torch.int8))
        return out_q
    _drop_handed_if_written(out_q, out_s)
    with torch.cuda.device(x.device):
        _quantize_rows(x, out_q, out_s, x.shape[0], x.shape[1])
    return out_q


def _rows_view(t: torch.Tensor):
    """``(rows, width, row pitch)`` of ``[K]``, ``[rows, K]`` or ``[..., K]`` whose rows are
    ``K`` contiguous elements at one pitch; ``None`` for any other layout."""
    if t.dim() == 1:
        return (1, t.shape[0], t.shape[0]) if t.stride(0) == 1 or t.shape[0] <= 1 else None
    if t.dim() > 2:
        try:
            t = t.view(-1, t.shape[-1])          # leading axes that collapse without a copy
        except RuntimeError:
            return None
    if t.dim() != 2 or (t.shape[1] > 1 and t.stride(1) != 1):
        return None
    return t.shape[0], t.shape[1], (t.stride(0) if t.shape[0] > 1 else max(t.stride(0), t.shape[1]))


def _silu_mul_native(gate, up, out, out_q, out_s, hand: bool = False) -> bool:
    """Run the fused kernel when every tensor is one it takes; False leaves the call to torch
    (other dtypes or devices, rows that are not ``K`` contiguous elements at one pitch).  ``hand``:
    with no ``out_q`` of the caller's, leave the quantised rows behind for the projection that
    follows (see ``HANDOVER``)."""
    tensors = [t for t in (gate, up, out, out_q, out_s) if t is not None]
    if not all(_on_gpu(t) and t.device == gate.device for t in tensors):
        return False
    if not (gate.dtype == up.dtype == out.dtype == torch.bfloat16):
        return False
    if out_q is not None and not (out_q.dtype == torch.int8 and out_q.is_contiguous()
                                  and out_s.dtype == torch.float32 and out_s.is_contiguous()):
        return False
    views = [_rows_view(t) for t in (gate, up, out)]
    if any(v is None for v in views):
        return False
    (rows, k, ldg), (_, _, ldu), (_, _, ldo) = views
    if rows == 0 or k == 0:
        return True
    q_ptr, s_ptr = _ptr(out_q), _ptr(out_s)
    with torch.cuda.device(gate.device):
        stream = _stream()
        target = _hand_target(rows, k, gate.device) if hand and out_q is None and out.dim() <= 2 else None
        if target is not None:
            q_ptr, s_ptr = target
        rc = _native.load().cmi_silu_mul_quant(gate.data_ptr(), up.data_ptr(), out.data_ptr(), q_ptr, s_ptr,
                                               rows, k, ldg, ldu, ldo, stream)
        if rc:
            _native.check(rc, "silu_mul_quant")
        if target is not None:
            _hand_over(out, rows, k, ldo, target, stream)
    return True


def silu_mul(gate: torch.Tensor, up: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """``silu_mul(gate, up, out) -> out``: ``out = silu(gate) * up`` into a caller-owned buffer
    that may alias ``up`` (backends/protocol.py:265-273, backends/reference/__init__.py:253-268).
    Registered together with :func:`silu_mul_quant` so that the two share one arithmetic.  Any
    leading shape (``[...]`` in the contract): layouts the kernel does not take go to torch."""
    if gate.shape != up.shape or out.shape != gate.shape:
        raise ValueError("silu_mul needs gate, up and out of one shape")
    _drop_handed()
    if not _silu_mul_native(gate, up, out, None, None, hand=True):
        out.copy_(F.silu(gate) * up)
    return out


def silu_mul_quant(gate: torch.Tensor, up: torch.Tensor, out: torch.Tensor, out_q: torch.Tensor,
                   out_s: torch.Tensor) -> torch.Tensor:
    """``silu_mul_quant(gate, up, out, out_q, out_s) -> out``: the SwiGLU product written as bf16
    and, in the same pass, quantised per row to int8 (``out_q`` + ``out_s``) -- bit for bit what
    ``silu_mul`` followed by ``kv_quant`` gives, because the absmax is taken over the stored bf16
    values (backends/protocol.py:274-278, backends/corex/__init__.py:1038-1071)."""
    if gate.shape != up.shape or gate.dim() != 2:
        raise ValueError("silu_mul_quant needs two same-shaped [rows, K] inputs")
    if tuple(out.shape) != tuple(gate.shape) or tuple(out_q.shape) != tuple(gate.shape) \
            or out_s.numel() != gate.shape[0]:
        raise ValueError("silu_mul_quant expects out [rows, K], out_q [rows, K], out_s [rows]")
    _drop_handed()
    if not _silu_mul_native(gate, up, out, out_q, out_s):
        out.copy_(F.silu(gate) * up)
        kv_quant(out if out.is_contiguous() else out.contiguous(), out_q, out_s)
    return out


def rms_norm_i8(x: torch.Tensor, w: torch.Tensor, out_q: torch.Tensor, out_s: torch.Tensor,
                eps: float = 1e-6, add: torch.Tensor | None = None,
                out: torch.Tensor | None = None) -> torch.Tensor:
    """RMSNorm (after ``x += add`` when ``add`` is given) quantised per row in the same pass.

    Not a table entry of the contract: the reference binds ``rms_norm_i8`` / ``add_rms_norm_i8``
    in its kernel extension only (backends/corex/kernels/norm.cu:257-350).  Same bits as
    ``rms_norm`` / ``add_rms_norm`` written as bf16 and then quantised by ``kv_quant``
    (backends/reference/__init__.py:169-198,224-250).  bf16 rows on the GPU only.
    ``out`` (optional) also receives the bf16 normalised rows.  Returns ``out_q``.
    """
    if x.dim() != 2 or not _on_gpu(x) or x.dtype != torch.bfloat16 or x.stride(1) != 1:
        raise ValueError("rms_norm_i8 expects bf16 [M, N] rows on the GPU with a unit innermost stride")
    m, n = x.shape
    gain = w if (w.dtype == torch.bfloat16 and w.is_contiguous()) else _memo(w, lambda: w.to(torch.bfloat16).contiguous())
    if gain.numel() != n or tuple(out_q.shape) != (m, n) or out_s.numel() != m:
        raise ValueError("rms_norm_i8 expects w [N], out_q [M, N], out_s [M]")
    if not (out_q.dtype == torch.int8 and out_q.is_contiguous() and out_s.dtype == torch.float32
            and out_s.is_contiguous() and out_q.device == x.device and gain.device == x.device):
        raise ValueError("rms_norm_i8: out_q must be contiguous int8 and out_s contiguous fp32 on x's device")
    ldx = x.stride(0) if m > 1 else max(x.stride(0), n)
    lib = _native.load()
    _drop_handed()
    y_ptr, ldy = 0, n
    if out is not None:
        if tuple(out.shape) != (m, n) or out.dtype != torch.bfloat16 or out.stride(1) != 1 or out.device != x.device:
            raise ValueError("rms_norm_i8: out must be bf16 [M, N] on x's device")
        y_ptr, ldy = out.data_ptr(), (out.stride(0) if m > 1 else max(out.stride(0), n))
    with torch.cuda.device(x.device):
        if add is None:
            rc = lib.cmi_rms_norm_i8(x.data_ptr(), gain.data_ptr(), y_ptr, out_q.data_ptr(), out_s.data_ptr(),
                                     m, n, ldx, ldy, float(eps), _stream())
        else:
            if tuple(add.shape) != (m, n) or add.dtype != torch.bfloat16 or add.stride(1) != 1 \
                    or add.device != x.device:
                raise ValueError("rms_norm_i8: add must be bf16 [M, N] on x's device")
            lda = add.stride(0) if m > 1 else max(add.stride(0), n)
            rc = lib.cmi_add_rms_norm_i8(x.data_ptr(), add.data_ptr(), gain.data_ptr(), y_ptr, out_q.data_ptr(),
                                         out_s.data_ptr(), m, n, ldx, lda, ldy, float(eps), _stream())
    if rc:
        _native.check(rc, "rms_norm_i8")
    return out_q


def _norm_native(x: torch.Tensor, w: torch.Tensor) -> bool:
    return (_on_gpu(x) and x.dtype == torch.bfloat16 and x.dim() == 2 and (x.shape[1] == 1 or x.stride(1) == 1)
            and w.device == x.device and w.numel() == x.shape[1])


def _gain_bf16(w: torch.Tensor) -> torch.Tensor:
    return w if (w.dtype == torch.bfloat16 and w.is_contiguous()) else _memo(w, lambda: w.to(torch.bfloat16).contiguous())


def rms_norm(x: torch.Tensor, w: torch.Tensor, stride: int = 0, eps: float = 1e-6) -> torch.Tensor:
    """``rms_norm(x, w, stride=0, eps=1e-6) -> y``: zero-centred RMSNorm over the last axis of a 2-D
    block (backends/protocol.py:238-243, backends/reference/__init__.py:169-198).  Registered so that
    ``rms_norm`` followed by ``kv_quant`` and :func:`rms_norm_i8` are one arithmetic (the kernel is
    the same, with and without the quantised outputs).  ``stride`` is informational, as in the
    reference: the row pitch is read from ``x``."""
    del stride
    if not _norm_native(x, w):
        xf = x.to(torch.float32)
        scale = torch.rsqrt(xf.pow(2).mean(dim=-1, keepdim=True) + eps)
        return (xf * scale).to(x.dtype) * w.to(x.dtype)
    m, n = x.shape
    y = torch.empty((m, n), dtype=torch.bfloat16, device=x.device)
    _drop_handed()
    if m == 0:
        return y
    gain = _gain_bf16(w)
    with torch.cuda.device(x.device):
        stream = _stream()
        target = _hand_target(m, n, x.device)
        q_ptr, s_ptr = target if target is not None else (0, 0)
        rc = _native.load().cmi_rms_norm_i8(x.data_ptr(), gain.data_ptr(), y.data_ptr(), q_ptr, s_ptr, m, n,
                                            x.stride(0) if m > 1 else max(x.stride(0), n), n, float(eps), stream)
        if rc:
            _native.check(rc, "rms_norm")
        if target is not None:
            _hand_over(y, m, n, n, target, stream)
    return y


def add_rms_norm(x: torch.Tensor, add: torch.Tensor, w: torch.Tensor, out: torch.Tensor, stride: int = 0,
                 eps: float = 1e-6) -> torch.Tensor:
    """``add_rms_norm(x, add, w, out, stride=0, eps=1e-6) -> out``: ``x += add`` in place, then the
    RMSNorm of the sum into ``out`` (backends/protocol.py:244-248, backends/reference/__init__.py:224-250)."""
    del stride
    ok = (_norm_native(x, w) and add.shape == x.shape and add.dtype == torch.bfloat16 and add.device == x.device
          and (add.shape[1] == 1 or add.stride(1) == 1) and out.shape == x.shape and out.dtype == torch.bfloat16
          and out.device == x.device and (out.shape[1] == 1 or out.stride(1) == 1))
    if not ok:
        x.add_(add)
        out.copy_(rms_norm(x, w, 0, eps))
        return out
    m, n = x.shape
    _drop_handed()
    if m == 0:
        return out
    gain = _gain_bf16(w)
    pitch = lambda t: t.stride(0) if m > 1 else max(t.stride(0), n)
    with torch.cuda.device(x.device):
        stream = _stream()
        target = _hand_target(m, n, x.device)
        q_ptr, s_ptr = target if target is not None else (0, 0)
        rc = _native.load().cmi_add_rms_norm_i8(x.data_ptr(), add.data_ptr(), gain.data_ptr(), out.data_ptr(), q_ptr,
                                                s_ptr, m, n, pitch(x), pitch(add), pitch(out), float(eps), stream)
        if rc:
            _native.check(rc, "add_rms_norm")
        if target is not None:
            _hand_over(out, m, n, pitch(out), target, stream)
    return out


def embed_rows(w, ids: torch.Tensor) -> torch.Tensor:
    """Rows ``ids`` of a quantized embedding matrix as bf16 ``[T, K]``: only the gathered rows are
    dequantised (ops/embed.py:64-81; ``QWeight.rows`` int8_weights.py:361-372,
    ``W4A8Weight.rows`` w4a8_weights.py:84-94).  Ids outside the vocabulary give NaN rows."""
    rec = _lookup(w)
    if rec is None:
        if not (_is_w4(w) or _is_q8(w)):
            raise ValueError("embed_rows expects a QWeight or W4A8Weight")
        if _is_w4(w) and not _kernels_take(w):
            raise ValueError("embed_rows: int4 rows are gathered for group sizes 64, 128 and 256")
        rec = _make_record(w)
    if rec.dev.type != "cuda":
        raise ValueError(f"coffin_amd: a quantized embedding is gathered on the GPU, weight is on {rec.dev}")
    if ids.device != rec.dev:
        raise ValueError(f"weight on {rec.dev} and ids on {ids.device} must share a device")
    flat = ids.reshape(-1)
    if flat.dtype != torch.int64 or not flat.is_contiguous():
        flat = flat.to(torch.int64).contiguous()
    t = flat.numel()
    out = torch.empty((t, rec.k), dtype=torch.bfloat16, device=rec.dev)
    lib = _native.load()
    with torch.cuda.device(rec.dev):
        if rec.kind == 4:
            rc = lib.cmi_embed_rows_w4(rec.a, rec.b, flat.data_ptr(), out.data_ptr(), t, rec.n, rec.k, rec.gs,
                                       _stream())
        else:
            rc = lib.cmi_embed_rows_i8(rec.a, rec.b, flat.data_ptr(), out.data_ptr(), t, rec.n, rec.k, _stream())
    if rc:
        _native.check(rc, "embed_rows")
    return out


#: Contract names this module answers natively.
NATIVE_NAMES = ("linear", "linear_m", "linear_m_verify", "linear_prefill", "kv_quant",
                "silu_mul", "silu_mul_quant", "rms_norm", "add_rms_norm")


def native_table() -> dict:
    """``{contract name: adapter}`` for the vendor file's ``build_ops``."""
    return {name: globals()[name] for name in NATIVE_NAMES}
