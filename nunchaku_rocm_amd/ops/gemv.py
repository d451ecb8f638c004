"""AWQ W4A16 GEMV operator (reference: nunchaku/ops/gemv.py:10-56, nunchaku/ops/triton/awq.py:186-229)."""

from __future__ import annotations

import torch

from .. import _lib

_MAX_ROWS = 32  # rows one launch handles; more rows re-stream the weights per block of 32


def awq_gemv_w4a16_cuda(
    in_feats: torch.Tensor,
    kernel: torch.Tensor,
    scaling_factors: torch.Tensor,
    zeros: torch.Tensor,
    m: int,
    n: int,
    k: int,
    group_size: int = 64,
) -> torch.Tensor:
    """
    ``out = in_feats @ (q * scaling_factors + zeros).T`` with ``q`` the TinyChat-packed uint4 weight
    (``kernel`` ``(n // 4, k // 2)`` int32), group size 64.  Returns ``in_feats.shape[:-1] + (n,)`` in the input dtype.
    """
    if group_size != 64:
        raise NotImplementedError(f"group_size={group_size}: only the group-64 GEMV of the FLUX adaLN layers is implemented")
    _lib.require_cuda(in_feats, kernel, scaling_factors, zeros)
    x = in_feats.reshape(m, k)
    if x.stride(1) != 1 or x.stride(0) % 8 or x.data_ptr() % 16:
        x = x.contiguous()
    if kernel.element_size() * kernel.numel() != n * k // 2 or not kernel.is_contiguous():
        raise ValueError(f"unexpected packed AWQ weight shape {tuple(kernel.shape)} for n={n}, k={k}")
    if scaling_factors.stride(1) != 1 or zeros.stride() != scaling_factors.stride():
        raise ValueError("scaling_factors and zeros must share a row-major (k // 64, n) layout")
    if scaling_factors.dtype != x.dtype or zeros.dtype != x.dtype:
        raise ValueError("scaling_factors / zeros must have the input dtype")
    out = torch.empty(m, n, dtype=x.dtype, device=x.device)
    lib = _lib.load()
    with torch.cuda.device(x.device):
        for r0 in range(0, m, _MAX_ROWS):
            rows = min(_MAX_ROWS, m - r0)
            args = _lib.AwqGemvArgs(
                x=x[r0:].data_ptr(),
                qweight=kernel.data_ptr(),
                scales=scaling_factors.data_ptr(),
                zeros=zeros.data_ptr(),
                out=out[r0:].data_ptr(),
                M=rows,
                N=n,
                K=k,
                ld_x=x.stride(0),
                ld_scales=scaling_factors.stride(0),
                ld_out=out.stride(0),
                dtype=_lib.dtype_code(x.dtype),
            )
            _lib.check(lib.svdq_awq_gemv_w4a16(args, _lib.stream_of(x)))
    return out.reshape(*in_feats.shape[:-1], n)
