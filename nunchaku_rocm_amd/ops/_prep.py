"""One-time re-layouts of weights.

The kernels read a LoRA-down weight ``(K, R)`` transposed, ``(R, K)``, so that MFMA operands are K-contiguous.  The
operator signatures take the natural layout (as the reference does), so the transposed copy is made on first use and
kept for as long as the weight tensor lives, is not modified in place and keeps its storage.

A cache entry holds a reference to the storage it was made from.  Assigning ``param.data = other`` changes neither the
parameter object nor its version counter, and without that reference the allocator could hand the freed block to the
next tensor of the same size, which would then look like the cached source; with it, an equal storage address means
the same storage.

A copy is made on the stream that is current at its first use.  A later use on another stream waits for the event
recorded behind that launch (until it has completed once); the copy itself stays allocated while it is cached.
"""

from __future__ import annotations

import weakref

import torch

from .. import _lib

_cache: dict[int, tuple] = {}


class _Ready:
    """Orders the first uses of a freshly made copy on other streams behind the launch that made it."""

    __slots__ = ("stream", "event")

    def __init__(self, device: torch.device):
        cur = torch.cuda.current_stream(device)
        self.stream = cur.cuda_stream
        self.event = torch.cuda.Event()
        self.event.record(cur)

    def wait(self, device: torch.device) -> None:
        if self.event is None:
            return
        if self.event.query():
            self.event = None
            return
        cur = torch.cuda.current_stream(device)
        if cur.cuda_stream != self.stream:
            cur.wait_event(self.event)


def _source_of(t: torch.Tensor) -> tuple:
    """What identifies the bytes a copy was derived from: version counter, the storage (kept alive) and the view."""
    return (t._version, t.untyped_storage(), t.storage_offset(), tuple(t.shape), tuple(t.stride()))


def _same_source(src: tuple, t: torch.Tensor) -> bool:
    version, storage, offset, shape, stride = src
    return (version == t._version and storage.data_ptr() == t.untyped_storage().data_ptr() and offset == t.storage_offset()
            and shape == tuple(t.shape) and stride == tuple(t.stride()))  # fmt: skip


def invalidate(t: torch.Tensor) -> None:
    """Drop the derived copies of ``t`` (for callers that rewrite a weight through a path the version counter misses)."""
    _cache.pop(id(t), None)
    _ldb_cache.pop(id(t), None)
    _rotary_cache.pop(id(t), None)
    _planes_cache.pop(id(t), None)
    _pinned.pop(id(t), None)


def lora_down_t(lora_down: torch.Tensor) -> torch.Tensor:
    key = id(lora_down)
    hit = _cache.get(key)
    if hit is not None:
        ref, src, t, ready = hit
        if ref() is lora_down and _same_source(src, lora_down):
            ready.wait(t.device)
            return t
    K, R = lora_down.shape
    src = lora_down if lora_down.stride(1) == 1 else lora_down.contiguous()
    t = torch.empty(R, K, dtype=lora_down.dtype, device=lora_down.device)
    lib = _lib.load()
    with torch.cuda.device(t.device):
        _lib.check(lib.svdq_transpose_lora_down(src.data_ptr(), t.data_ptr(), K, R, src.stride(0), _lib.stream_of(src)))
        ready = _Ready(t.device)
    try:
        ref = weakref.ref(lora_down, lambda _r, k=key: _cache.pop(k, None))
        _cache[key] = (ref, _source_of(lora_down), t, ready)
    except TypeError:
        pass
    return t


_ldb_cache: dict[int, tuple] = {}


def lora_down_blocked(lora_down: torch.Tensor, ldt: torch.Tensor) -> torch.Tensor | None:
    """The transposed LoRA-down weight ``ldt`` ``(R2, N)`` in the order the GELU + requantization epilogue reads it
    (``svdq_block_lora_down``), cached under the weight ``lora_down`` like the transposed copy itself."""
    key = id(lora_down)
    hit = _ldb_cache.get(key)
    if hit is not None:
        ref, src, t, ready = hit
        if ref() is lora_down and _same_source(src, lora_down):
            ready.wait(t.device)
            return t
    if torch.cuda.is_current_stream_capturing():
        return None  # no new copies while a graph is being recorded
    R2, N = ldt.shape
    lib = _lib.load()
    t = torch.empty(lib.svdq_lora_down_blocked_bytes(N, R2) // 2, dtype=ldt.dtype, device=ldt.device)
    with torch.cuda.device(t.device):
        _lib.check(lib.svdq_block_lora_down(ldt.data_ptr(), t.data_ptr(), N, R2, _lib.dtype_code(ldt.dtype), _lib.stream_of(ldt)))
        ready = _Ready(t.device)
    try:
        ref = weakref.ref(lora_down, lambda _r, k=key: _ldb_cache.pop(k, None))
        _ldb_cache[key] = (ref, _source_of(lora_down), t, ready)
    except TypeError:
        pass
    return t


_rotary_cache: dict[int, tuple] = {}


def rotary_blocked(rotary_emb: torch.Tensor, rot2d: torch.Tensor) -> torch.Tensor | None:
    """The rotary table in the order the Q/K RMSNorm + RoPE epilogue reads it (``svdq_block_rotary``).  ``rotary_emb`` is
    the tensor the caller passed (the cache key: a model passes the same table to every block and step), ``rot2d`` its
    ``(rows, 128)`` fp32 view with unit inner stride."""
    key = id(rotary_emb)
    hit = _rotary_cache.get(key)
    if hit is not None:
        ref, src, t, ready, rows = hit
        if ref() is rotary_emb and _same_source(src, rotary_emb) and rows == rot2d.shape[0]:
            ready.wait(t.device)
            return t
    if torch.cuda.is_current_stream_capturing():
        return None  # no new copies while a graph is being recorded: the epilogue reads the table itself
    lib = _lib.load()
    rows = rot2d.shape[0]
    t = torch.empty(lib.svdq_rotary_blocked_bytes(rows) // 4, dtype=torch.float32, device=rot2d.device)
    with torch.cuda.device(t.device):
        _lib.check(lib.svdq_block_rotary(rot2d.data_ptr(), t.data_ptr(), rows, rot2d.stride(0), _lib.stream_of(rot2d)))
        ready = _Ready(t.device)
    try:
        ref = weakref.ref(rotary_emb, lambda _r, k=key: _rotary_cache.pop(k, None))
        _rotary_cache[key] = (ref, _source_of(rotary_emb), t, ready, rows)
    except TypeError:
        pass
    return t


_planes_cache: dict[int, tuple] = {}
_pinned: dict[int, tuple] = {}  # id(weight parameter) -> (weakref, planes): a weight whose packed bytes were released


def pin_weight_planes(qweight: torch.Tensor, planes: torch.Tensor) -> None:
    """Make ``planes`` the working copy of ``qweight`` for good, whatever storage ``qweight`` points at from now on (its
    packed bytes are about to be released: the fp8 main loop never reads them).  Undone by :func:`unpin_weight_planes`."""
    key = id(qweight)
    _pinned[key] = (weakref.ref(qweight, lambda _r, k=key: _pinned.pop(k, None)), planes)
    _planes_cache.pop(key, None)


def unpin_weight_planes(qweight: torch.Tensor) -> None:
    _pinned.pop(id(qweight), None)


def pinned_weight_planes(qweight: torch.Tensor) -> torch.Tensor | None:
    hit = _pinned.get(id(qweight))
    return hit[1] if hit is not None and hit[0]() is qweight else None


def weight_planes(qweight: torch.Tensor, wscales: torch.Tensor) -> torch.Tensor | None:
    """The GEMM's working copy of a packed ``(N, K/2)`` weight (``svdq_split_weight_planes``): six-bit fp6 codes in
    MFMA lane order, followed by the weight scales and the per-group terms that take the offset of signed activations
    out again.  Made on first use and kept while both tensors live unmodified.  Costs ``0.75 * N * K`` bytes (one and a
    half times the packed weight) plus ``6 * N * K / 64`` bytes.  ``None`` when the offset terms do not fit the 16-bit
    type (fp16 scales of about 17 and more): the caller then uses the packed weight.  Reading that status word waits for
    the re-layout once, when the copy is made."""
    pinned = pinned_weight_planes(qweight)
    if pinned is not None:
        return pinned
    key = id(qweight)
    hit = _planes_cache.get(key)
    if hit is not None:
        ref, src, src_s, t, ready = hit
        if ref() is qweight and _same_source(src, qweight) and _same_source(src_s, wscales):
            if t is not None:
                ready.wait(t.device)
            return t
    N, K = qweight.shape[0], qweight.shape[1] * 2
    lib = _lib.load()
    t = torch.empty(lib.svdq_weight_planes_bytes(N, K), dtype=torch.uint8, device=qweight.device)
    with torch.cuda.device(t.device):
        _lib.check(lib.svdq_split_weight_planes(qweight.data_ptr(), wscales.data_ptr(), t.data_ptr(), N, K, qweight.stride(0),
                                                wscales.stride(0), _lib.dtype_code(wscales.dtype), _lib.stream_of(qweight)))  # fmt: skip
        ready = _Ready(t.device)
        if int(t[-16:-12].view(torch.int32).item()) != 0:  # a piece of an offset term is not finite
            t = None
    try:
        ref = weakref.ref(qweight, lambda _r, k=key: _planes_cache.pop(k, None))
        _planes_cache[key] = (ref, _source_of(qweight), _source_of(wscales), t, ready)
    except TypeError:
        pass
    return t
