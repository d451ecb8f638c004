"""Block-level elementwise step fused into one kernel: the gated residual update
(reference: nunchaku/models/transformers/transformer_flux_v2.py:233-234, :241-243, :326-330, separate torch kernels
there).  An addition to the reference's operator set."""

from __future__ import annotations

import torch

from .. import _lib


def gated_residual(
    x: torch.Tensor,
    gate: torch.Tensor,
    y: torch.Tensor,
    y2: torch.Tensor | None = None,
    out: torch.Tensor | None = None,
    want_stats: bool = False,
    eps: float = 1e-6,
    clip: float = 0.0,
) -> tuple[torch.Tensor, torch.Tensor | None]:
    """
    ``out = x + gate[:, None] * (y [+ y2])`` for ``x``, ``y`` of shape ``(B, S, C)`` and ``gate`` ``(B, C)`` (any element
    stride), every step rounded to the 16-bit dtype as the separate torch kernels would.  With ``want_stats`` also
    returns the ``(B * S, 2)`` float32 row statistics ``(mean, 1 / sqrt(var + eps))`` of ``out``, ready for the ``norm=``
    prologue of the next quantizer.  ``clip > 0`` limits ``out`` to ``[-clip, clip]`` first (the reference model's
    ``clip(-65504, 65504)`` of fp16 runs).  Returns ``(out, stats)``.
    """
    _lib.require_cuda(x, gate, y, y2, out)
    B, S, C = x.shape
    if y.shape != x.shape or (y2 is not None and y2.shape != x.shape) or gate.shape != (B, C):
        raise ValueError(f"shapes: x {tuple(x.shape)}, y {tuple(y.shape)}, gate {tuple(gate.shape)}")
    if not (x.dtype == y.dtype == gate.dtype) or (y2 is not None and y2.dtype != x.dtype):
        raise ValueError("x, gate, y and y2 must share one 16-bit dtype")

    def rows(t):
        t2 = t.reshape(B * S, C)
        return t2 if t2.stride(1) == 1 and t2.stride(0) % 8 == 0 and t2.data_ptr() % 16 == 0 else t2.contiguous()

    x2, ya = rows(x), rows(y)
    yb = rows(y2) if y2 is not None else None
    if yb is not None and yb.stride(0) != ya.stride(0):
        ya, yb = ya.contiguous(), yb.contiguous()
    if out is None:
        out = torch.empty(B, S, C, dtype=x.dtype, device=x.device)
    o2 = out.view(B * S, C)
    if gate.stride(1) < 1 or (gate.stride(1) == 1 and (gate.stride(0) % 8 or gate.data_ptr() % 16)):
        gate = gate.contiguous()
    stats = torch.empty(B * S, 2, dtype=torch.float32, device=x.device) if want_stats else None
    with torch.cuda.device(x.device):
        _lib.check(_lib.load().svdq_gated_residual(
            x2.data_ptr(), gate.data_ptr(), ya.data_ptr(), _lib.ptr(yb), o2.data_ptr(), _lib.ptr(stats), B * S, C,
            x2.stride(0), ya.stride(0), o2.stride(0), S if B > 1 else 0, gate.stride(0), gate.stride(1),
            _lib.dtype_code(x.dtype), float(eps), float(clip), _lib.stream_of(x)))  # fmt: skip
    return out, stats
