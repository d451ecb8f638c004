"""Unmasked 16-bit attention (reference: nunchaku/ops/dispatch.py:51-99, nunchaku/ops/triton/attention.py:120-169)."""

from __future__ import annotations

import torch
import torch.nn.functional as F

from .. import _lib

_HEAD_DIMS = (128, 64)  # the head dimensions the kernel is built for (FLUX / Qwen-Image, SDXL-class models)


def attention_fp16(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, o: torch.Tensor, scale: float) -> None:
    """
    Fused scaled-dot-product attention without a mask, written into ``o``.

    q : (B, H, TokensQ, D);  k, v : (B, H, TokensKV, D);  o : (B, TokensQ, H * D);  D = 128 or 64;  fp16 or bf16, last
    dimension contiguous.  ``scale`` is the softmax scale, normally ``D ** -0.5``.
    """
    B, H, Tq, D = q.shape
    Tkv = k.shape[2]
    assert k.shape == (B, H, Tkv, D) and v.shape == (B, H, Tkv, D)
    assert o.shape == (B, Tq, H * D), f"unexpected output shape {tuple(o.shape)}"
    _lib.require_cuda(q, k, v, o)
    if not (q.dtype == k.dtype == v.dtype == o.dtype):
        raise ValueError("q, k, v and o must share one dtype")
    if any(t.stride(-1) != 1 for t in (q, k, v, o)):
        raise ValueError("the last dimension of q, k, v and o must be contiguous")
    if D not in _HEAD_DIMS:
        raise NotImplementedError(f"attention_fp16: head dimension {D} is not supported (128 and 64 only)")
    lib = _lib.load()
    args = _lib.AttentionArgs(
        q=q.data_ptr(), k=k.data_ptr(), v=v.data_ptr(), o=o.data_ptr(),
        sqb=q.stride(0), sqh=q.stride(1), sqm=q.stride(2),
        skb=k.stride(0), skh=k.stride(1), skn=k.stride(2),
        svb=v.stride(0), svh=v.stride(1), svn=v.stride(2),
        sob=o.stride(0), som=o.stride(1),
        B=B, H=H, Tq=Tq, Tkv=Tkv, D=D, dtype=_lib.dtype_code(q.dtype), scale=float(scale),
    )  # fmt: skip
    with torch.cuda.device(q.device):
        _lib.check(lib.svdq_attention_fp16(args, _lib.stream_of(q)))


def _covered(query: torch.Tensor, key: torch.Tensor, value: torch.Tensor) -> bool:
    return (
        query.is_cuda
        and query.dtype in (torch.float16, torch.bfloat16)
        and key.dtype == value.dtype == query.dtype
        and query.shape[-1] in _HEAD_DIMS
        and key.shape[2] > 0
        and all(t.stride(-1) == 1 and t.data_ptr() % 16 == 0 and all(s % 8 == 0 for s in t.stride()[:-1]) for t in (query, key, value))
    )  # fmt: skip


def scaled_dot_product_attention(
    query: torch.Tensor, key: torch.Tensor, value: torch.Tensor, attn_mask: torch.Tensor | None = None
) -> torch.Tensor:
    """
    Drop-in for ``F.scaled_dot_product_attention`` on ``(B, H, T, D)`` inputs (no dropout, not causal).  Unmasked
    fp16 / bf16 attention with head dimension 128 or 64 runs on the HIP kernel; what the kernel does not cover (a mask,
    fp32, another head dimension, a strided head dimension) goes to torch, as in the reference.
    """
    if attn_mask is not None or not _covered(query, key, value):
        return F.scaled_dot_product_attention(query, key, value, attn_mask=attn_mask, dropout_p=0.0, is_causal=False)
    B, H, T, D = query.shape
    out = torch.empty(B, T, H * D, dtype=query.dtype, device=query.device)
    attention_fp16(query, key, value, out, D**-0.5)
    return out.view(B, T, H, D).transpose(1, 2)
