"""Activation quantizer operator (reference: nunchaku/ops/quantize.py:11-88)."""

from __future__ import annotations

import torch

from .. import _lib
from ._prep import lora_down_t as _lora_down_t


def _ceil_divide(a: int, b: int) -> int:
    return (a + b - 1) // b


def layer_norm_stats(input: torch.Tensor, eps: float = 1e-6) -> torch.Tensor:
    """Per-row ``(mean, 1 / sqrt(var + eps))`` of a 16-bit ``(..., K)`` tensor as ``(M, 2)`` float32: the statistics of
    ``LayerNorm(K, elementwise_affine=False, eps=eps)``, for the ``norm=`` prologue of the quantizer (one call can
    serve several quantizations of the same rows)."""
    inp = input.reshape(-1, input.shape[-1])
    _lib.require_cuda(inp)
    if inp.stride(1) != 1 or inp.stride(0) % 8 or inp.data_ptr() % 16:
        inp = inp.contiguous()
    stats = torch.empty(inp.shape[0], 2, dtype=torch.float32, device=inp.device)
    with torch.cuda.device(inp.device):
        _lib.check(_lib.load().svdq_row_stats(inp.data_ptr(), stats.data_ptr(), inp.shape[0], inp.shape[1], inp.stride(0),
                                              _lib.dtype_code(inp.dtype), float(eps), _lib.stream_of(inp)))  # fmt: skip
    return stats


def _norm_args(norm, inp: torch.Tensor, M: int, K: int, eps: float):
    """``norm = (scale, shift[, stats])`` -> (stats, scale, shift, rows_per_batch, ld, stride) for the C call.  scale
    and shift are used where they lie when they share their strides (as the slices of one adaLN projection do)."""
    scale, shift = norm[0], norm[1]
    stats = norm[2] if len(norm) > 2 and norm[2] is not None else layer_norm_stats(inp, eps)
    if scale.dim() == 1:
        scale, shift = scale[None], shift[None]
    batches = scale.shape[0]
    if scale.shape != (batches, K) or shift.shape != scale.shape or scale.dtype != inp.dtype or shift.dtype != inp.dtype:
        raise ValueError("norm scale and shift must both be (K,) or (batches, K) of the input dtype")
    if M % batches or (batches > 1 and (M // batches) % 16):
        raise ValueError(f"{M} rows do not split into {batches} batches of a multiple of 16 rows")
    if stats.dtype != torch.float32 or stats.shape != (M, 2) or not stats.is_contiguous():
        raise ValueError("norm stats must be a contiguous (M, 2) float32 tensor")
    if scale.stride() != shift.stride() or scale.stride(1) < 1 or (batches > 1 and scale.stride(0) < 0):
        scale, shift = scale.contiguous(), shift.contiguous()
    return stats, scale, shift, (M // batches if batches > 1 else 0), scale.stride(0), scale.stride(1)


def quantize_w4a4_act_fuse_lora(
    input: torch.Tensor,
    output: torch.Tensor | None = None,
    oscales: torch.Tensor | None = None,
    lora_down: torch.Tensor | None = None,
    lora_act_out: torch.Tensor | None = None,
    smooth: torch.Tensor | None = None,
    fuse_glu: bool = False,
    fp4: bool = False,
    fuse_gelu: bool = False,
    shift_value: float = 0.0,
    unsigned: bool = False,
    norm: tuple | None = None,
    norm_eps: float = 1e-6,
    out_blocked: bool | int = False,
) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """
    Backend-level quantizer with the reference's full option set (reference:
    nunchaku/ops/triton/gemm_w4a4.py:1521-1565): no row padding, outputs allocated when not given, ``unsigned`` /
    ``shift_value`` for activations known to be non-negative after a shift, ``fuse_gelu`` = tanh-GELU of the input
    first (what the GEMM's fused GELU epilogue computes, for outputs that were produced unfused).

    ``norm=(scale, shift)`` or ``(scale, shift, stats)`` (no counterpart in the reference, which runs these as separate
    torch kernels): what is quantized and LoRA-projected is ``layer_norm(input) * scale + shift`` (no affine,
    ``eps=norm_eps``, every step rounded to the input dtype), with ``scale`` / ``shift`` of shape ``(K,)`` or
    ``(batches, K)`` (rows split evenly over the batches) and ``stats`` from :func:`layer_norm_stats`.

    ``out_blocked=True`` (no counterpart in the reference): ``output`` keeps its shape but holds the codes in the order
    the GEMM's fp8 main loop reads them (``svdq_quantize_args.out_blocked``; pass it on with ``act_blocked=True``); it
    must be contiguous with a multiple of 32 rows.  :func:`nunchaku_rocm_amd.layout.unblock_activations` undoes it.
    ``out_blocked=2``: ``output`` is ``(rows, 3K/4)`` bytes of fp6 codes (sign << 5 | magnitude, the same integers) in
    lane order, for the GEMM's ``act_blocked=2`` (:func:`nunchaku_rocm_amd.layout.unblock_activations_f6`).
    ``out_blocked=3`` (K a multiple of 512): as ``2``, and ``oscales`` -- contiguous ``(K/64, rows)``, rows a multiple of
    32 -- holds the scales in the GEMM's own order too (``svdq_quantize_args.scales_blocked``, for ``act_blocked=3``;
    :func:`nunchaku_rocm_amd.layout.unblock_scales`).
    """
    if fp4:
        raise NotImplementedError("NVFP4 quantization is not implemented (int4 only)")
    if fuse_gelu and fuse_glu:
        raise NotImplementedError("fuse_gelu together with fuse_glu")
    inp = input.reshape(-1, input.shape[-1])
    _lib.require_cuda(inp, output, oscales, lora_down, lora_act_out, smooth)
    M = inp.shape[0]
    K = inp.shape[1] // 2 if fuse_glu else inp.shape[1]
    if K % 64:
        raise ValueError(f"K={K} must be a multiple of the group size 64")
    rank = lora_down.shape[1] if lora_down is not None else 0
    out_blocked = int(out_blocked)
    kb = K * 3 // 4 if out_blocked >= 2 else K // 2  # bytes of codes per row
    if output is None:
        output = torch.empty(_ceil_divide(M, 32) * 32 if out_blocked else M, kb, dtype=torch.uint8, device=inp.device)
    if oscales is None:
        oscales = torch.empty(K // 64, output.shape[0] if out_blocked == 3 else M, dtype=inp.dtype, device=inp.device)
    if lora_act_out is None and lora_down is not None:
        lora_act_out = torch.empty(M, rank, dtype=torch.float32, device=inp.device)

    if inp.stride(1) != 1 or inp.stride(0) % 8 or inp.data_ptr() % 16:
        inp = inp.contiguous()
    if output.element_size() != 1 or output.stride(1) != 1 or output.shape[0] < M:
        raise ValueError("output must be a (>= M, K/2) byte tensor with unit inner stride")
    if out_blocked and (not output.is_contiguous() or output.shape[0] % 32 or output.shape[1] != kb or output.data_ptr() % 16):
        raise ValueError("out_blocked needs a contiguous (rows, K/2) output (2: (rows, 3K/4)) with rows a multiple of 32")
    if out_blocked == 3 and (K % 512 or not oscales.is_contiguous() or oscales.shape != (K // 64, output.shape[0]) or oscales.data_ptr() % 16):
        raise ValueError("out_blocked=3 needs K % 512 == 0 and contiguous (K/64, rows) oscales over output's rows")
    if oscales.dtype != inp.dtype or oscales.stride(1) != 1 or oscales.shape[1] < M or oscales.shape[0] < K // 64:
        raise ValueError("oscales must be (K/64, >= M) of the input dtype with unit inner stride")
    if rank and (lora_act_out.dtype != torch.float32 or lora_act_out.stride(1) != 1 or lora_act_out.shape[0] < M):
        raise ValueError("lora_act_out must be (>= M, R) float32 with unit inner stride")
    if smooth is not None and (smooth.dtype != inp.dtype or not smooth.is_contiguous() or smooth.numel() != K):
        raise ValueError("smooth must be a contiguous (K,) tensor of the input dtype")
    if lora_down is not None and (lora_down.dtype != inp.dtype or lora_down.shape[0] != K):
        raise ValueError("lora_down must be (K, R) of the input dtype")

    nstats = nscale = nshift = None
    nrows, nld, nstride = 0, 0, 1
    if norm is not None:
        if fuse_glu or fuse_gelu:
            raise NotImplementedError("norm= cannot be combined with fuse_glu / fuse_gelu")
        nstats, nscale, nshift, nrows, nld, nstride = _norm_args(norm, inp, M, K, norm_eps)
    args = _lib.QuantizeArgs(
        norm_stats=_lib.ptr(nstats),
        norm_scale=_lib.ptr(nscale),
        norm_shift=_lib.ptr(nshift),
        norm_rows_per_batch=nrows,
        norm_ld=nld,
        norm_stride=nstride,
        x=inp.data_ptr(),
        smooth=_lib.ptr(smooth),
        lora_down_t=_lora_down_t(lora_down).data_ptr() if rank else None,
        out=output.data_ptr(),
        scales=oscales.data_ptr(),
        lora_act=lora_act_out.data_ptr() if rank else None,
        M=M,
        K=K,
        R=rank,
        ld_x=inp.stride(0),
        ld_out=output.stride(0),
        ld_scales=oscales.stride(0),
        ld_lora_act=lora_act_out.stride(0) if rank else 0,
        dtype=_lib.dtype_code(inp.dtype),
        is_unsigned=int(unsigned),
        prologue=_lib.PRE_GLU if fuse_glu else (_lib.PRE_GELU if fuse_gelu else _lib.PRE_NONE),
        shift=float(shift_value),
        out_blocked=min(out_blocked, 2),
        scales_blocked=int(out_blocked == 3),
    )
    with torch.cuda.device(inp.device):
        _lib.check(_lib.load().svdq_quantize_act(args, _lib.stream_of(inp)))
    return output, oscales, lora_act_out


def quantize_w4a4_act(
    input: torch.Tensor,
    output: torch.Tensor | None = None,
    oscales: torch.Tensor | None = None,
    fp4: bool = False,
) -> tuple[torch.Tensor, torch.Tensor]:
    """Per-group-64 symmetric int4 quantization without smoothing or LoRA (reference:
    nunchaku/ops/triton/gemm_w4a4.py:1568-1577): ``(codes (M, K/2) uint8, scales (K/64, M))``."""
    out, scales, _ = quantize_w4a4_act_fuse_lora(input, output, oscales, fp4=fp4)
    return out, scales


def quantize_w4a4_wgt(
    input: torch.Tensor,
    output: torch.Tensor | None = None,
    oscales: torch.Tensor | None = None,
    fp4: bool = False,
) -> tuple[torch.Tensor, torch.Tensor]:
    """The same arithmetic applied to a weight ``(N, K)`` (reference: nunchaku/ops/triton/gemm_w4a4.py:1580-1592): the
    result ``(codes (N, K/2), scales (K/64, N))`` is the natural layout the GEMM reads as ``wgt`` / ``wscales``."""
    out, scales, _ = quantize_w4a4_act_fuse_lora(input, output, oscales, fp4=fp4)
    return out, scales


def svdq_quantize_w4a4_act_fuse_lora_cuda(
    input: torch.Tensor,
    output: torch.Tensor | None = None,
    oscales: torch.Tensor | None = None,
    lora_down: torch.Tensor | None = None,
    lora_act_out: torch.Tensor | None = None,
    smooth: torch.Tensor | None = None,
    fuse_glu: bool = False,
    fp4: bool = False,
    pad_size: int = 256,
    norm: tuple | None = None,
    norm_eps: float = 1e-6,
    out_blocked: bool | int = False,
) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """
    Quantize activations to int4 (per-group-64 absmax, after dividing by ``smooth``) and compute the LoRA
    down-projection ``input @ lora_down`` in the same pass (reference: nunchaku/ops/quantize.py:11-88).

    Same signature and return value as the reference operator: ``(output (M_pad, C/2) uint8,
    oscales (C/64, M_pad) input.dtype, lora_act_out (M_pad, R) float32)`` with ``C = input.shape[1]`` and
    ``M_pad = ceil(M / pad_size) * pad_size``.  Only rows ``< M`` are written; pad rows keep whatever the freshly
    allocated buffers held.

    Unlike the reference wrapper (which dereferences ``lora_down.shape`` unconditionally), ``lora_down=None`` is
    accepted and returns ``lora_act_out`` with zero columns.  ``norm`` / ``norm_eps``: the LayerNorm + modulate
    prologue described in :func:`quantize_w4a4_act_fuse_lora` (an addition; ``None`` = the reference's behaviour).
    ``out_blocked``: see there as well (an addition; ``False`` = the reference's ``(M_pad, C/2)`` matrix; ``2`` =
    ``(M_pad, 3C/4)`` fp6 codes).
    """
    if fp4:
        raise NotImplementedError("NVFP4 quantization is not implemented (int4 only)")
    if input.dim() != 2:
        raise ValueError(f"input must be 2-D (M, K), got {tuple(input.shape)}")
    batch_size, channels = input.shape
    rank = lora_down.shape[1] if lora_down is not None else 0
    batch_size_pad = _ceil_divide(batch_size, pad_size) * pad_size
    if output is None:
        kb = (channels // 2 if fuse_glu else channels) * 3 // 4 if int(out_blocked) >= 2 else channels // 2
        output = torch.empty(batch_size_pad, kb, dtype=torch.uint8, device=input.device)
    if oscales is None:
        assert channels % 64 == 0
        oscales = torch.empty(channels // 64, batch_size_pad, dtype=input.dtype, device=input.device)
    if lora_act_out is None:
        lora_act_out = torch.empty(batch_size_pad, rank, dtype=torch.float32, device=input.device)
    quantize_w4a4_act_fuse_lora(input, output, oscales, lora_down, lora_act_out if rank else None, smooth, fuse_glu, fp4,
                                norm=norm, norm_eps=norm_eps, out_blocked=out_blocked)
    return output, oscales, lora_act_out
