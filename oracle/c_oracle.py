"""ctypes access to the C restatement of the oracle (``svdq_oracle.c``); test infrastructure only."""

from __future__ import annotations

import ctypes
import os
import subprocess

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libsvdq_oracle.so")
_lib = None


def build() -> str:
    """Compile ``svdq_oracle.c`` with the Makefile beside it; returns the library path."""
    subprocess.run(["make", "-C", _HERE, "-s", "-B"], check=True)
    return _SO


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = ctypes.CDLL(_SO)
    return _lib


def _p(t: torch.Tensor | None):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else None


def _bits(t: torch.Tensor | None):
    return t.contiguous().view(torch.int16) if t is not None else None


def group_acc_i32(act: torch.Tensor, wgt: torch.Tensor, g: int, act_unsigned: bool) -> torch.Tensor:
    act, wgt = act.contiguous().view(torch.uint8), wgt.contiguous().view(torch.uint8)
    M, K, N = act.shape[0], act.shape[1] * 2, wgt.shape[0]
    p = torch.empty(M, N, dtype=torch.int32)
    lib().oracle_group_acc_i32(_p(act), _p(wgt), _p(p), M, N, K, g, int(act_unsigned))
    return p


def quantize_act(x, smooth=None, lora_down=None, unsigned=False, shift=0.0):
    assert x.dtype == torch.bfloat16
    M, K = x.shape
    R = lora_down.shape[1] if lora_down is not None else 0
    xb, sb, lb = _bits(x), _bits(smooth), _bits(lora_down)
    out = torch.empty(M, K // 2, dtype=torch.uint8)
    scales = torch.empty(K // 64, M, dtype=torch.int16)
    lora_act = torch.empty(M, max(R, 1), dtype=torch.float32)
    lib().oracle_quantize_act(
        _p(xb), _p(sb), _p(lb), _p(out), _p(scales), _p(lora_act), M, K, R, M, int(unsigned), ctypes.c_float(shift)
    )
    return out, scales.view(torch.bfloat16), (lora_act[:, :R] if R else None)


def gemm_w4a4(act, wgt, ascales, wscales, bias=None, lora_act=None, lora_up=None, act_unsigned=False):
    act, wgt = act.contiguous().view(torch.uint8), wgt.contiguous().view(torch.uint8)
    M, K, N = act.shape[0], act.shape[1] * 2, wgt.shape[0]
    R = lora_up.shape[1] if lora_up is not None else 0
    asb, wsb, bb, lub = _bits(ascales), _bits(wscales), _bits(bias), _bits(lora_up)
    la = lora_act.contiguous() if lora_act is not None else None
    out = torch.empty(M, N, dtype=torch.float32)
    lib().oracle_gemm_w4a4(
        _p(act), _p(wgt), _p(asb), _p(wsb), _p(bb), _p(la), _p(lub), _p(out), M, N, K, R,
        ascales.shape[1], wscales.shape[1], int(act_unsigned),
    )  # fmt: skip
    return out


def awq_gemv(x, packed_i16, scales, zeros):
    M, K = x.shape
    N = scales.shape[1]
    xb, sb, zb = _bits(x), _bits(scales), _bits(zeros)
    pk = packed_i16.contiguous()
    out = torch.empty(M, N, dtype=torch.float32)
    lib().oracle_awq_gemv(_p(xb), _p(pk), _p(sb), _p(zb), _p(out), M, N, K)
    return out
