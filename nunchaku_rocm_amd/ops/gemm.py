"""W4A4 GEMM operator (reference: nunchaku/ops/gemm.py:12-207 and the dispatcher nunchaku/ops/triton/gemm_w4a4.py:1003-1314)."""

from __future__ import annotations

import torch

from .. import _lib
from ._prep import lora_down_blocked as _lora_down_blocked
from ._prep import lora_down_t as _lora_down_t
from ._prep import pinned_weight_planes as _pinned_weight_planes
from ._prep import rotary_blocked as _rotary_blocked
from ._prep import weight_planes as _weight_planes

# Which weights get the GEMM's working copy (fp6 codes in MFMA lane order with their scales and offset terms, cached per
# tensor, see _prep.weight_planes; 0.84 bytes per weight next to the packed weight's 0.5; without it the GEMM is 36 %
# slower, 240 against 176 us at the FLUX QKV shape): "parameters" = weights that are nn.Parameter (module weights, which
# live long), "all" = any weight tensor (a temporary pays the re-layout on every call), "none" = the GEMM unpacks the
# packed weight itself (int8 main loop, no extra memory).
USE_WEIGHT_PLANES = "parameters"

# The Q/K RMSNorm + RoPE epilogue reads the rotary table through a copy in the order its lanes want it (made once per
# table tensor and cached, 16 KB per 32 rows): 1 KB per load instruction instead of 32-byte pieces of 32 rows, which was
# most of that epilogue's cost.  False = read the (rows, 128) table itself (same results).
USE_BLOCKED_ROTARY = True

# The modules and composite operators (SVDQW4A4Linear.forward, fused_gelu_mlp, fused_qkv_norm_rottary, fused_swiglu_mlp)
# pass quantized activations from the quantizer, or from a requantizing epilogue, to the GEMM in the order the fp8 main
# loop's lanes read them (out_blocked / act_blocked / qout_blocked): 1 KB per load instruction instead of 16-byte pieces
# of 32 rows.  True: as fp6 codes (ACT_CODES_F6: the matrix instruction takes them as they are -- fp6 x fp6, no nibble
# unpack, no offset term for signed activations; 8 % of a GEMM launch on signed, 4 % on unsigned activations).  1: the
# matrix's bytes in lane order (3 %; the same results as the matrix, bit for bit).  False: the reference's (M, K/2)
# matrix everywhere.  The operators themselves (svdq_quantize_w4a4_act_fuse_lora_cuda, svdq_gemm_w4a4_cuda) keep the
# matrix unless asked.
USE_BLOCKED_ACTIVATIONS = True

# The GELU + requantization epilogue reads the next layer's LoRA-down weight through a copy in the order its matrix
# instructions want it (made once per weight and cached, as large as the weight): 1 KB per load instruction instead of
# 8-byte pieces of 32 rows.  False = read the transposed (R2, N) copy (same results).
USE_BLOCKED_LORA_DOWN = True
# values of ``act_blocked`` / ``out_blocked`` / ``qout_blocked`` beyond False / True: fp6 codes in lane order, and the same with
# the activation scales in the GEMM's own order as well (eight groups of a row side by side; K a multiple of 512)
ACT_CODES_F6 = 2
ACT_CODES_F6_SCALES = 3

# True sends the requantizing epilogues' LoRA-down partial sums to the buffer built into the library
# (svdq_gemm_w4a4_static_scratch) instead of a torch allocation per call: for callers that may not allocate, e.g. while
# a HIP graph is being captured.  The buffer holds 16 MiB (about M * N / 128 * R2 * 4 bytes are needed) and is shared
# by every call on the GPU, so calls on two streams must not overlap.
STATIC_SCRATCH = False


def prepare_static_scratch(device=None) -> None:
    """Look up the built-in buffer on ``device`` (default: the current one) now, outside any graph capture; the first
    ``STATIC_SCRATCH`` call on a device would otherwise do it (``svdq_gemm_w4a4_static_scratch_prepare``)."""
    with torch.cuda.device(device):
        _lib.check(_lib.load().svdq_gemm_w4a4_static_scratch_prepare())


def set_fp8_loop_variant(variant: int) -> None:
    """Which build of the fp8 main loop every following GEMM on pre-split weights uses: -1 = chosen by the number of tiles
    (default), 0 = three workgroups per CU, 1 = two per CU with software-pipelined steps.  The two give identical bits; the
    switch exists for tuning and for tests (``svdq_gemm_w4a4_set_variant``)."""
    _lib.check(_lib.load().svdq_gemm_w4a4_set_variant(int(variant)))


def working_copy(wgt: torch.Tensor, wscales: torch.Tensor) -> torch.Tensor | None:
    """The re-laid-out copy of ``wgt`` the fp8 main loop reads (made and cached on first use), or ``None`` when this
    weight runs through the int8 main loop: not a parameter (see ``USE_WEIGHT_PLANES``), rows not 16-byte aligned, or
    fp16 scales too large for the copy's 16-bit offset terms."""
    planes = _pinned_weight_planes(wgt)  # a module whose packed weight was released: this copy is all there is
    if planes is None:
        want_planes = USE_WEIGHT_PLANES == "all" or (USE_WEIGHT_PLANES == "parameters" and isinstance(wgt, torch.nn.Parameter))
        planes = _weight_planes(wgt, wscales) if want_planes and wgt.stride(0) % 16 == 0 else None
    return planes


def takes_blocked_activations(wgt: torch.Tensor, wscales: torch.Tensor, rows: int) -> int:
    """How a GEMM on this weight should be fed its activations: 0 = the (M, K/2) matrix, 1 = its bytes in the fp8 main
    loop's own order, 2 (``ACT_CODES_F6``) = fp6 codes in that order, 3 (``ACT_CODES_F6_SCALES``, K a multiple of 512) = those
    with the activation scales in the loop's own order too -- the value for ``out_blocked`` / ``qout_blocked`` of the
    producer and ``act_blocked`` of this GEMM.  Non-zero when the switch is on, the weight has a working copy and the
    (padded) row count is a multiple of 32."""
    if not USE_BLOCKED_ACTIVATIONS or rows % 32 or working_copy(wgt, wscales) is None:
        return 0
    if USE_BLOCKED_ACTIVATIONS is True:
        return ACT_CODES_F6_SCALES if (wgt.shape[1] * 2) % 512 == 0 else ACT_CODES_F6
    return int(USE_BLOCKED_ACTIVATIONS)


HEAD_DIM = 128
GELU_SHIFT = 0.171875


def svdq_gemm_w4a4_cuda(
    act: torch.Tensor,
    wgt: torch.Tensor,
    out: torch.Tensor | None = None,
    qout: torch.Tensor | None = None,
    ascales: torch.Tensor | None = None,
    wscales: torch.Tensor | None = None,
    oscales: torch.Tensor | None = None,
    poolout: torch.Tensor | None = None,
    lora_act_in: torch.Tensor | None = None,
    lora_up: torch.Tensor | None = None,
    lora_down: torch.Tensor | None = None,
    lora_act_out: torch.Tensor | None = None,
    norm_q: torch.Tensor | None = None,
    norm_k: torch.Tensor | None = None,
    rotary_emb: torch.Tensor | None = None,
    bias: torch.Tensor | None = None,
    smooth_factor: torch.Tensor | None = None,
    out_vk: torch.Tensor | None = None,
    out_linearattn: torch.Tensor | None = None,
    act_unsigned: bool = False,
    lora_scales: list[float] | None = None,
    fuse_silu: bool = False,
    fp4: bool = False,
    alpha: float | None = 1.0,
    wcscales: torch.Tensor | None = None,
    out_q: torch.Tensor | None = None,
    out_k: torch.Tensor | None = None,
    out_v: torch.Tensor | None = None,
    attn_tokens: int = 0,
    fuse_swiglu: bool = False,
    act_blocked: bool | int = False,
    qout_blocked: bool | int = False,
):
    """
    ``out = deq(act) @ deq(wgt).T + lora_act_in @ lora_up.T + bias`` on packed int4 operands with per-group-64 scales,
    written in place; positional order is the reference operator's (29 arguments; ``fuse_swiglu`` is keyword-only
    in spirit and selects the SwiGLU requantizing epilogue of the reference's Triton-level ``gemm_w4a4``).

    * ``norm_q``/``norm_k``/``rotary_emb``: fused per-head RMSNorm + RoPE on the Q and K thirds of ``out``.
    * ``qout``/``oscales`` (+ ``smooth_factor``, ``lora_down``, ``lora_act_out``): fused GELU, next layer's LoRA-down
      and unsigned int4 requantization; ``out`` may then be ``None``.
    * ``act`` may have more (padded) rows than ``out``; only ``out.shape[0]`` rows are written.
    * ``act_blocked`` / ``qout_blocked`` (no counterpart in the reference): ``act`` holds its codes in the order the fp8
      main loop reads them, as the quantizer writes them with ``out_blocked=True`` / the requantizing epilogue writes
      ``qout`` that way for the GEMM that consumes it.  Needs a weight with a working copy (see ``USE_WEIGHT_PLANES``).
      ``act_blocked=2`` (``ACT_CODES_F6``): ``act`` is ``(rows, 3K/4)`` bytes of fp6 codes in lane order, as the quantizer
      writes them with ``out_blocked=2``: the matrix instruction takes them as they are (no offset term for signed
      activations, fp6 x fp6); ``act_unsigned`` is then not looked at.  ``qout_blocked=2``: the requantizing epilogue writes
      ``qout`` as ``(rows, 3NQ/4)`` bytes of such codes.  ``3`` (``ACT_CODES_F6_SCALES``; K, or the requantized width, a
      multiple of 512): as ``2``, and ``ascales`` / ``oscales`` hold their values in the loop's own order as well
      (``svdq_gemm_args.ascales_blocked`` / ``oscales_blocked``; contiguous, rows a multiple of 32).

    Raises ``NotImplementedError`` for the arguments the reference's ROCm backend rejects as well (``poolout``,
    ``out_vk``, ``out_linearattn``, ``out_q/k/v``) and for the NVFP4-only ones (``fp4``, ``wcscales``, ``alpha != 1``,
    ``fuse_silu``).  ``lora_scales`` is accepted and ignored, as in the reference's ROCm backend.  Returns ``None``.
    """
    unsupported = {
        "poolout": poolout,
        "out_vk": out_vk,
        "out_linearattn": out_linearattn,
        "out_q": out_q,
        "out_k": out_k,
        "out_v": out_v,
    }
    active = sorted(name for name, value in unsupported.items() if value is not None)
    if active:
        raise NotImplementedError("these fused gemm_w4a4 epilogues are not implemented: " + ", ".join(active))
    if fp4 or wcscales is not None or fuse_silu or not (alpha is None or alpha == 1.0):
        raise NotImplementedError("NVFP4 options (fp4, wcscales, alpha != 1) and fuse_silu are not implemented (int4 only)")
    assert ascales is not None and wscales is not None, "W4A4 GEMM requires both scale tensors"

    act = act.reshape(-1, act.shape[-1])
    act_blocked = int(act_blocked)
    M, K, N = act.shape[0], wgt.shape[1] * 2, wgt.shape[0]
    assert act.shape[1] == (K * 3 // 4 if act_blocked >= ACT_CODES_F6 else K // 2), f"weight K mismatch: {K} vs act {tuple(act.shape)}"
    dev = _lib.require_cuda(act, wgt, out, qout, ascales, wscales, oscales, lora_act_in, lora_up, lora_down,
                            lora_act_out, norm_q, norm_k, rotary_emb, bias, smooth_factor)  # fmt: skip

    want_quant = qout is not None or oscales is not None
    want_qk = norm_q is not None or norm_k is not None or rotary_emb is not None
    if want_quant:
        assert qout is not None and oscales is not None, "qout and oscales must be given together"
        assert (lora_down is None) == (lora_act_out is None), "lora_down and lora_act_out must be given together"
        if want_qk:
            raise NotImplementedError("requantizing epilogue together with Q/K norm + RoPE")
    if want_qk:
        assert norm_q is not None and norm_k is not None and rotary_emb is not None, (
            "norm_q, norm_k, and rotary_emb must all be given together"
        )
    if fuse_swiglu:
        assert out is None and want_quant, "fuse_swiglu writes qout/oscales, not out"
    if want_quant and not want_qk and (N % 128 or M % 16 or qout.stride(-1) != 1 or (fuse_swiglu and N % 32)):
        # shapes the requantizing epilogues do not take: the unfused form, as the reference's dispatcher does
        # (nunchaku/ops/triton/gemm_w4a4.py:985-1000, 1298-1312): 16-bit GEMM output, then the activation quantizer
        from .quantize import quantize_w4a4_act_fuse_lora

        T = oscales.dtype
        x = out.reshape(-1, N) if out is not None else torch.empty(M, N, dtype=T, device=dev)
        svdq_gemm_w4a4_cuda(act, wgt, out=x, ascales=ascales, wscales=wscales, lora_act_in=lora_act_in, lora_up=lora_up,
                            bias=bias, act_unsigned=act_unsigned, act_blocked=act_blocked)  # fmt: skip
        rows = x.shape[0]
        qout2d = qout.reshape(-1, qout.shape[-1])
        la_out = lora_act_out if lora_down is not None else None
        if fuse_swiglu:
            x = x.view(rows, N // 32, 2, 16)
            y = (torch.nn.functional.silu(x[:, :, 0]) * x[:, :, 1]).reshape(rows, N // 2)
            quantize_w4a4_act_fuse_lora(y, qout2d, oscales, lora_down, la_out, smooth_factor, out_blocked=qout_blocked)
        else:
            quantize_w4a4_act_fuse_lora(x, qout2d, oscales, lora_down, la_out, smooth_factor, fuse_gelu=True,
                                        shift_value=GELU_SHIFT, unsigned=True, out_blocked=qout_blocked)  # fmt: skip
        return None

    T = out.dtype if out is not None else (oscales.dtype if oscales is not None else ascales.dtype)
    if out is None and not want_quant:
        out = torch.empty(M, N, dtype=T, device=dev)  # computed and dropped, as the reference does
    out2d = out.reshape(-1, N) if out is not None else None
    actual_m = out2d.shape[0] if out2d is not None else M
    assert actual_m <= M, f"out has more rows ({actual_m}) than act ({M})"

    has_lora = lora_act_in is not None and lora_up is not None
    R = lora_up.shape[1] if has_lora else 0

    for name, t in (("act", act), ("wgt", wgt)):
        if t.element_size() != 1 or t.stride(-1) != 1:
            raise ValueError(f"{name} must be a packed byte tensor with unit inner stride")
    for name, s, rows in (("ascales", ascales, M), ("wscales", wscales, N)):
        if s.dtype != T or s.dim() != 2 or s.shape[0] < K // 64 or s.shape[1] < rows or s.stride(1) != 1:
            raise ValueError(f"{name} must be (K/64, >= {rows}) of dtype {T}, got {tuple(s.shape)} {s.dtype}")
    if bias is not None and (bias.dtype != T or bias.dim() != 1 or bias.shape[0] < N or bias.stride(0) != 1):
        raise ValueError("bias must be a contiguous (N,) tensor of the output dtype")
    if has_lora:
        if lora_act_in.dtype != torch.float32 or lora_up.dtype != T:
            raise ValueError(f"LoRA dtypes {lora_act_in.dtype}/{lora_up.dtype}")
        if lora_up.shape[0] < N or lora_act_in.shape[0] < M or lora_act_in.shape[1] < R:
            raise ValueError("LoRA shapes")
        if lora_act_in.stride(1) != 1 or lora_up.stride(1) != 1:
            raise ValueError("LoRA tensors need unit inner stride")
    if out2d is not None and out2d.stride(1) != 1:
        raise ValueError("out not row-major")

    planes = working_copy(wgt, wscales)
    if act_blocked:
        if planes is None:
            raise ValueError("act_blocked needs a weight with a working copy (the int8 main loop reads the (M, K/2) matrix)")
        if not act.is_contiguous() or M % 32 or act.data_ptr() % 16:
            raise ValueError("act_blocked needs a contiguous act with a multiple of 32 rows")
        if act_blocked == ACT_CODES_F6_SCALES and (K % 512 or not ascales.is_contiguous() or ascales.shape != (K // 64, M) or ascales.data_ptr() % 16):
            raise ValueError("act_blocked=3 needs K % 512 == 0 and contiguous (K/64, rows) ascales over the same rows as act")
    args = _lib.GemmArgs(
        act=act.data_ptr(),
        wgt=wgt.data_ptr(),
        wgt_planes=_lib.ptr(planes),
        ascales=ascales.data_ptr(),
        wscales=wscales.data_ptr(),
        bias=_lib.ptr(bias),
        lora_act=lora_act_in.data_ptr() if R else None,
        lora_up=lora_up.data_ptr() if R else None,
        out=_lib.ptr(out2d),
        M=M,
        N=N,
        K=K,
        R=R,
        actual_m=actual_m,
        ld_act=act.stride(0),
        ld_wgt=wgt.stride(0),
        ld_ascales=ascales.stride(0),
        ld_wscales=wscales.stride(0),
        ld_lora_act=lora_act_in.stride(0) if R else 0,
        ld_lora_up=lora_up.stride(0) if R else 0,
        ld_out=out2d.stride(0) if out2d is not None else 0,
        dtype=_lib.dtype_code(T),
        act_unsigned=int(act_unsigned),
        epilogue=_lib.EPI_PLAIN,
        eps=1e-6,
        act_blocked=min(act_blocked, ACT_CODES_F6),
        ascales_blocked=int(act_blocked == ACT_CODES_F6_SCALES),
    )
    keep = [planes]  # tensors that must outlive the launch call
    lib = _lib.load()
    if want_qk:
        rot_key = rotary_emb  # the caller's tensor: what the re-laid-out copy is cached under
        if rotary_emb.dtype != torch.float32:
            rotary_emb = rotary_emb.float()  # the reference's unfused kernel reads any dtype and computes in fp32
        rot = rotary_emb.reshape(actual_m, HEAD_DIM)
        if rot.stride(1) != 1:
            rot = rot.contiguous()
        for name, w in (("norm_q", norm_q), ("norm_k", norm_k)):
            if w.dtype != T or w.numel() != HEAD_DIM or not w.is_contiguous():
                raise ValueError(f"{name} must be a contiguous ({HEAD_DIM},) tensor of the output dtype")
        keep.append(rot)
        args.epilogue = _lib.EPI_QK_NORM_ROPE
        args.norm_q, args.norm_k, args.rotary = norm_q.data_ptr(), norm_k.data_ptr(), rot.data_ptr()
        args.ld_rotary = rot.stride(0)
        if USE_BLOCKED_ROTARY and rot.data_ptr() % 16 == 0 and rot.stride(0) % 4 == 0:
            # the epilogue reads the table re-laid-out for its lanes (made once per table, see _prep)
            rb = _rotary_blocked(rot_key, rot)
            if rb is not None:
                keep.append(rb)
                args.rotary_blocked = rb.data_ptr()
    elif want_quant:
        NQ = N // 2 if fuse_swiglu else N
        qout2d = qout.reshape(-1, qout.shape[-1])
        qb = NQ * 3 // 4 if int(qout_blocked) >= ACT_CODES_F6 else NQ // 2  # bytes of codes per row
        if qout2d.element_size() != 1 or qout2d.shape[0] < M or qout2d.shape[1] != qb or qout2d.stride(1) != 1:
            raise ValueError(f"qout shape/dtype {tuple(qout.shape)} {qout.dtype}")
        if oscales.dtype != T or oscales.dim() != 2 or oscales.shape[0] != NQ // 64 or oscales.shape[1] < M or oscales.stride(1) != 1:
            raise ValueError(f"oscales shape {tuple(oscales.shape)}")
        if smooth_factor is not None and (smooth_factor.dtype != T or smooth_factor.numel() != NQ or not smooth_factor.is_contiguous()):
            raise ValueError("smooth_factor must be a contiguous (N,) tensor of the output dtype")
        R2 = lora_down.shape[1] if lora_down is not None else 0
        if R2:
            if lora_down.dtype != T or lora_down.dim() != 2 or lora_down.shape[0] != NQ:
                raise ValueError(f"lora_down shape/dtype {tuple(lora_down.shape)} {lora_down.dtype}")
            if lora_act_out.dtype != torch.float32 or lora_act_out.dim() != 2 or lora_act_out.shape[0] < M or lora_act_out.shape[1] != R2:
                raise ValueError("lora_act_out must be (>= M, R2) fp32")
            ldt = _lora_down_t(lora_down)
            epi = _lib.EPI_SWIGLU_QUANT if fuse_swiglu else _lib.EPI_GELU_QUANT
            keep.append(ldt)
            args.lora_down_t, args.lora_act_out = ldt.data_ptr(), lora_act_out.data_ptr()
            if USE_BLOCKED_LORA_DOWN and not fuse_swiglu and N % 128 == 0:
                ldb = _lora_down_blocked(lora_down, ldt)  # the GELU epilogue's own order (made once per weight, see _prep)
                if ldb is not None:
                    keep.append(ldb)
                    args.lora_down_blocked = ldb.data_ptr()
            if not STATIC_SCRATCH:
                nbytes = lib.svdq_gemm_w4a4_scratch_bytes(M, N, R2, epi)
                scratch = torch.empty(nbytes // 4, dtype=torch.float32, device=dev)
                keep.append(scratch)
                args.scratch = scratch.data_ptr()
            args.ld_lora_act_out = lora_act_out.stride(0)
        args.epilogue = _lib.EPI_SWIGLU_QUANT if fuse_swiglu else _lib.EPI_GELU_QUANT
        args.qout, args.oscales, args.smooth_next = qout2d.data_ptr(), oscales.data_ptr(), _lib.ptr(smooth_factor)
        args.R2, args.ld_qout, args.ld_oscales = R2, qout2d.stride(0), oscales.stride(0)
        if qout_blocked:
            if not qout2d.is_contiguous() or qout2d.shape[0] % 32 or qout2d.data_ptr() % 16:
                raise ValueError("qout_blocked needs a contiguous qout with a multiple of 32 rows")
            args.qout_blocked = min(int(qout_blocked), ACT_CODES_F6)
            if int(qout_blocked) == ACT_CODES_F6_SCALES:
                if NQ % 512 or not oscales.is_contiguous() or oscales.shape[1] != qout2d.shape[0] or oscales.data_ptr() % 16:
                    raise ValueError("qout_blocked=3 needs a requantized width that is a multiple of 512 and contiguous oscales over qout's rows")
                args.oscales_blocked = 1
        args.shift = 0.0 if fuse_swiglu else GELU_SHIFT

    with torch.cuda.device(dev):
        entry = lib.svdq_gemm_w4a4_static_scratch if STATIC_SCRATCH else lib.svdq_gemm_w4a4
        _lib.check(entry(args, _lib.stream_of(act)))
    return None


def group_acc_i32(act: torch.Tensor, wgt: torch.Tensor, group: int, act_unsigned: bool = False, fp8_path: bool = False) -> torch.Tensor:
    """Debug read-out: exact int32 accumulators ``sum_{k in group} a[m, k] * w[n, k]`` through the instruction sequence of
    the GEMM's int8 main loop (packed weights) or of its fp8 main loop (pre-split weights)."""
    act = act.reshape(-1, act.shape[-1])
    dev = _lib.require_cuda(act, wgt)
    M, K, N = act.shape[0], act.shape[1] * 2, wgt.shape[0]
    out = torch.empty(M, N, dtype=torch.int32, device=dev)
    with torch.cuda.device(dev):
        _lib.check(
            _lib.load().svdq_group_acc_i32(
                act.data_ptr(), wgt.data_ptr(), out.data_ptr(), M, N, K, act.stride(0), wgt.stride(0), group,
                int(act_unsigned), int(fp8_path), _lib.stream_of(act),
            )  # fmt: skip
        )
    return out
