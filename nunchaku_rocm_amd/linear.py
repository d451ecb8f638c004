"""Quantized linear modules with the reference's parameter names and shapes
(reference: nunchaku/models/linear.py:13-269 ``SVDQW4A4Linear``, :278-415 ``AWQW4A16Linear``), natural layout
(``qweight (N, K/2)`` low nibble = even k, ``wscales (K/64, N)``), int4 only."""

from __future__ import annotations

import torch
from torch import nn

from .ops.gemm import svdq_gemm_w4a4_cuda
from .ops.gemv import awq_gemv_w4a16_cuda
from .ops.quantize import svdq_quantize_w4a4_act_fuse_lora_cuda


class SVDQW4A4Linear(nn.Module):
    """``y = (x / smooth) .q W4^T + (x @ proj_down) @ proj_up^T + bias`` with 4-bit activations and weights."""

    def __init__(
        self,
        in_features: int,
        out_features: int,
        rank: int = 32,
        bias: bool = True,
        precision: str = "int4",
        act_unsigned: bool = False,
        torch_dtype: torch.dtype = torch.bfloat16,
        device: str | torch.device | None = None,
    ):
        super().__init__()
        if precision != "int4":
            raise NotImplementedError(f"precision {precision!r}: only int4 is implemented")
        if device is None:
            device = torch.device("cpu")
        self.in_features, self.out_features, self.rank = in_features, out_features, rank
        self.precision, self.torch_dtype, self.group_size = precision, torch_dtype, 64
        self.qweight = nn.Parameter(torch.empty(out_features, in_features // 2, dtype=torch.int8, device=device), requires_grad=False)
        self.bias = nn.Parameter(torch.empty(out_features, dtype=torch_dtype, device=device)) if bias else None
        self.wscales = nn.Parameter(torch.empty(in_features // 64, out_features, dtype=torch_dtype, device=device), requires_grad=False)
        self.smooth_factor = nn.Parameter(torch.empty(in_features, dtype=torch_dtype, device=device), requires_grad=False)
        self.smooth_factor_orig = nn.Parameter(torch.empty(in_features, dtype=torch_dtype, device=device), requires_grad=False)
        self.proj_down = nn.Parameter(torch.empty(in_features, rank, dtype=torch_dtype, device=device))
        self.proj_up = nn.Parameter(torch.empty(out_features, rank, dtype=torch_dtype, device=device))
        self.wtscale = None
        self.wcscales = None
        self.act_unsigned = act_unsigned

    @classmethod
    def from_linear(cls, linear: nn.Linear, **kwargs):
        in_features = kwargs.pop("in_features", linear.in_features)
        torch_dtype = kwargs.pop("torch_dtype", linear.weight.dtype)
        return cls(in_features=in_features, out_features=linear.out_features, bias=linear.bias is not None,
                   torch_dtype=torch_dtype, device=linear.weight.device, **kwargs)  # fmt: skip

    # ---- memory: the GEMM's working copy can stand in for the packed weight ------------------------------------------
    def release_packed_weight(self) -> bool:
        """Drop the bytes of ``qweight`` and keep only the GEMM's working copy of it (1.7 x as large; made now if it does not
        exist yet).  The fp8 main loop never reads the packed weight, so a model that would otherwise hold both (2.7 x the
        packed bytes) holds 1.7 x.  ``qweight`` keeps its shape (every row a view of one spare row); ``state_dict()`` still
        returns the packed weight, rebuilt from the copy; :meth:`restore_packed_weight` puts it back in place.  Returns
        ``False`` (and changes nothing) when the weight has no usable working copy (rows not 16-byte aligned, or fp16
        scales too large for its 16-bit offset terms)."""
        from .ops import _prep

        if _prep.pinned_weight_planes(self.qweight) is not None:
            return True
        if not self.qweight.is_cuda or self.qweight.stride(0) % 16:
            return False
        planes = _prep.weight_planes(self.qweight, self.wscales)
        if planes is None:
            return False
        _prep.pin_weight_planes(self.qweight, planes)
        self.qweight.data = torch.empty(self.in_features // 2, dtype=self.qweight.dtype, device=self.qweight.device).expand(self.out_features, -1)
        return True

    def restore_packed_weight(self) -> None:
        """Undo :meth:`release_packed_weight`: ``qweight`` holds its packed bytes again."""
        from .layout import join_weight_planes
        from .ops import _prep

        planes = _prep.pinned_weight_planes(self.qweight)
        if planes is None:
            return
        packed = join_weight_planes(planes, self.out_features, self.in_features).view(self.qweight.dtype)
        _prep.unpin_weight_planes(self.qweight)
        self.qweight.data = packed

    def _save_to_state_dict(self, destination, prefix, keep_vars):
        super()._save_to_state_dict(destination, prefix, keep_vars)
        from .ops import _prep

        planes = _prep.pinned_weight_planes(self.qweight)
        if planes is not None:  # released: hand out the packed form, rebuilt from the working copy
            from .layout import join_weight_planes

            destination[prefix + "qweight"] = join_weight_planes(planes, self.out_features, self.in_features).view(self.qweight.dtype)

    def _load_from_state_dict(self, state_dict, prefix, *args, **kwargs):
        from .ops import _prep

        if _prep.pinned_weight_planes(self.qweight) is not None:  # a new weight is coming: give it storage to land in
            _prep.unpin_weight_planes(self.qweight)
            self.qweight.data = torch.empty(self.out_features, self.in_features // 2, dtype=self.qweight.dtype, device=self.qweight.device)
        super()._load_from_state_dict(state_dict, prefix, *args, **kwargs)

    def forward(self, x: torch.Tensor, output: torch.Tensor | None = None, norm: tuple | None = None) -> torch.Tensor:
        """``norm=(scale, shift[, stats])``: apply ``layer_norm(x) * scale + shift`` inside the quantizer (an addition
        to the reference's signature; see ``ops.quantize``)."""
        batch_size, seq_len, channels = x.shape
        x = x.reshape(batch_size * seq_len, channels)
        if output is None:
            output = torch.empty(batch_size * seq_len, self.out_features, dtype=x.dtype, device=x.device)
        blocked = self.takes_blocked(batch_size * seq_len)
        quantized_x, ascales, lora_act_out = self.quantize(x, norm=norm, blocked=blocked)
        output = self.forward_quant(quantized_x, ascales, lora_act_out, output, act_blocked=blocked)
        return output.reshape(batch_size, seq_len, -1)

    def takes_blocked(self, rows: int, pad_size: int = 256) -> int:
        """How this layer's GEMM wants its quantized input for ``rows`` rows padded to ``pad_size``: the value for
        ``blocked=`` in :meth:`quantize` (or ``qout_blocked=`` of the GEMM whose epilogue produces the input) and
        ``act_blocked=`` in :meth:`forward_quant`: 0 = the reference's matrix, 1 = its bytes in the fp8 main loop's own
        order, 2 = fp6 codes in that order, 3 = those with the activation scales in that order too (``in_features`` a
        multiple of 512)."""
        from .ops.gemm import takes_blocked_activations

        return takes_blocked_activations(self.qweight, self.wscales, -(-rows // pad_size) * pad_size)

    def quantize(self, x: torch.Tensor, pad_size: int = 256, norm: tuple | None = None, blocked: bool | int = False):
        """``blocked`` (an addition to the reference's signature): the codes in the order the GEMM's fp8 main loop reads
        them (``True``), as fp6 codes in that order (``2``) or those with the scales in that order too (``3``), for
        :meth:`forward_quant` with the same ``act_blocked``;
        ``False`` = the reference's ``(M_pad, K/2)`` matrix."""
        return svdq_quantize_w4a4_act_fuse_lora_cuda(
            x, lora_down=self.proj_down, smooth=self.smooth_factor, fp4=False, pad_size=pad_size, norm=norm, out_blocked=blocked
        )

    def forward_quant(self, quantized_x, ascales, lora_act, output: torch.Tensor | None = None, act_blocked: bool | int = False) -> torch.Tensor:
        if output is None:
            output = torch.empty(quantized_x.shape[0], self.out_features, dtype=self.proj_up.dtype, device=quantized_x.device)
        svdq_gemm_w4a4_cuda(
            act=quantized_x,
            wgt=self.qweight,
            out=output,
            ascales=ascales,
            wscales=self.wscales,
            lora_act_in=lora_act,
            lora_up=self.proj_up,
            bias=self.bias,
            fp4=False,
            alpha=self.wtscale,
            wcscales=self.wcscales,
            act_unsigned=self.act_unsigned,
            act_blocked=act_blocked,
        )
        return output

    def __repr__(self):
        return (f"SVDQW4A4Linear(in_features={self.in_features}, out_features={self.out_features}, rank={self.rank}, "
                f"precision={self.precision}, act_unsigned={self.act_unsigned})")  # fmt: skip


class AWQW4A16Linear(nn.Module):
    """AWQ W4A16 linear, group 64, TinyChat-packed ``qweight (N/4, K/2) int32``; bias added after the GEMV."""

    def __init__(self, in_features: int, out_features: int, bias: bool = True, group_size: int = 64,
                 torch_dtype: torch.dtype = torch.bfloat16, device: str | torch.device | None = None):  # fmt: skip
        super().__init__()
        if device is None:
            device = torch.device("cpu")
        self.in_features, self.out_features, self.group_size = in_features, out_features, group_size
        self.qweight = nn.Parameter(torch.empty(out_features // 4, in_features // 2, dtype=torch.int32, device=device), requires_grad=False)
        self.bias = nn.Parameter(torch.empty(out_features, dtype=torch_dtype, device=device)) if bias else None
        self.wscales = nn.Parameter(torch.empty(in_features // group_size, out_features, dtype=torch_dtype, device=device), requires_grad=False)
        self.wzeros = nn.Parameter(torch.empty(in_features // group_size, out_features, dtype=torch_dtype, device=device), requires_grad=False)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        output = awq_gemv_w4a16_cuda(in_feats=x, kernel=self.qweight, scaling_factors=self.wscales, zeros=self.wzeros,
                                     m=x.shape[0], n=self.out_features, k=self.in_features, group_size=self.group_size)  # fmt: skip
        if self.bias is not None:
            view_shape = [1] * (output.ndim - 1) + [-1]
            output.add_(self.bias.view(view_shape))
        return output

    @classmethod
    def from_linear(cls, linear: nn.Linear, group_size: int = 64, torch_dtype: torch.dtype = torch.bfloat16,
                    device: str = "cpu", **kwargs):  # fmt: skip
        return cls(in_features=linear.in_features, out_features=linear.out_features, bias=linear.bias is not None,
                   group_size=group_size, torch_dtype=torch_dtype, device=device)  # fmt: skip

    def __repr__(self):
        return f"AWQW4A16Linear(in_features={self.in_features}, out_features={self.out_features}, group_size={self.group_size})"
