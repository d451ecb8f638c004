"""One-time re-layout of LoRA-down weights.

The kernels read a LoRA-down weight ``(K, R)`` transposed, ``(R, K)``, so that MFMA operands are K-contiguous.  The
operator signatures take the natural layout (as the reference does), so the transposed copy is made on first use and
kept for as long as the weight tensor lives and is not modified in place.
"""

from __future__ import annotations

import weakref

import torch

from .. import _lib

_cache: dict[int, tuple] = {}


def lora_down_t(lora_down: torch.Tensor) -> torch.Tensor:
    key = id(lora_down)
    hit = _cache.get(key)
    if hit is not None:
        ref, version, data_ptr, t = hit
        if ref() is lora_down and version == lora_down._version and data_ptr == lora_down.data_ptr():
            return t
    K, R = lora_down.shape
    if lora_down.stride(1) != 1:
        lora_down = lora_down.contiguous()
    t = torch.empty(R, K, dtype=lora_down.dtype, device=lora_down.device)
    lib = _lib.load()
    _lib.check(
        lib.svdq_transpose_lora_down(
            lora_down.data_ptr(), t.data_ptr(), K, R, lora_down.stride(0), _lib.stream_of(lora_down)
        )
    )
    try:
        ref = weakref.ref(lora_down, lambda _r, k=key: _cache.pop(k, None))
        _cache[key] = (ref, lora_down._version, lora_down.data_ptr(), t)
    except TypeError:
        pass
    return t
