"""AWQ W4A16 operators: the group-64 GEMV, the dense decode and the GEMM built on it (reference:
nunchaku/ops/gemv.py:10-56, nunchaku/ops/dispatch.py:19-49, nunchaku/ops/triton/awq.py:83-118, 186-251)."""

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
    (``kernel`` ``(n // 4, k // 2)`` int32).  Group size 64 runs the fused GEMV kernel (weights read once for all ``m``
    rows).  Two cases take the reference's own route for everything but group size 64 (ops/triton/awq.py:226-228), still
    on the GPU: :func:`awq_dequantize` to a dense ``(n, k)`` 16-bit weight (``2 n k`` bytes, allocated per call), then a
    library matmul -- other group sizes or ``n % 32 != 0``, and shapes whose per-group tables do not fit the kernel's
    64 KB of LDS (``k = 12288`` with more than 16 rows; no FLUX shape).  Weights of 4 GiB and more are refused
    (``RuntimeError``): the kernels address them with 32-bit offsets.  Returns ``in_feats.shape[:-1] + (n,)`` in the
    input dtype.
    """
    _lib.require_cuda(in_feats, kernel, scaling_factors, zeros)
    x = in_feats.reshape(m, k)
    if group_size != 64 or n % 32:
        # as the reference (ops/triton/awq.py:226-228): decode to a dense weight, then a library matmul
        w = awq_dequantize(kernel, scaling_factors, zeros, n, k, group_size, x.dtype)
        return torch.matmul(x, w.t()).reshape(*in_feats.shape[:-1], n)
    if x.stride(1) != 1 or x.stride(0) % 8 or x.data_ptr() % 16:
        x = x.contiguous()
    if kernel.element_size() * kernel.numel() != n * k // 2 or not kernel.is_contiguous():
        raise ValueError(f"unexpected packed AWQ weight shape {tuple(kernel.shape)} for n={n}, k={k}")
    if scaling_factors.stride(1) != 1 or zeros.stride() != scaling_factors.stride():
        raise ValueError("scaling_factors and zeros must share a row-major (k // 64, n) layout")
    if scaling_factors.dtype != x.dtype or zeros.dtype != x.dtype:
        raise ValueError("scaling_factors / zeros must have the input dtype")
    if n * k // 2 >= 1 << 32:
        raise RuntimeError(f"AWQ weight of {n * k // 2} bytes: 4 GiB and more are not supported (32-bit offsets)")
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
            rc = lib.svdq_awq_gemv_w4a16(args, _lib.stream_of(x))
            if rc == _lib.E_UNSUPPORTED:
                # the kernel's per-group tables do not fit LDS (K = 12288 with more than 16 rows, longer K with fewer):
                # decode the weight and multiply on the GPU, the reference's route for everything but group size 64 (the
                # other refusal, a weight of 4 GiB and more, was raised above)
                w = awq_dequantize(kernel, scaling_factors, zeros, n, k, group_size, x.dtype)
                return torch.matmul(x, w.t()).reshape(*in_feats.shape[:-1], n)
            _lib.check(rc)
    return out.reshape(*in_feats.shape[:-1], n)


class AwqGemvBatch:
    """Several AWQ W4A16 GEMVs of one shape, all on the same input, in one launch (``svdq_awq_gemv_w4a16_batched``).

    The adaLN projections of a diffusion transformer all take ``silu(temb)`` and depend on nothing else in the model
    (nunchaku/models/normalization.py), so the model can compute them together; one 32 MB weight is too short a read to
    reach the HBM rate, many behind each other are not.  Built once from the layers' tensors (``kernels[i]``
    ``(n // 4, k // 2)`` int32, ``scales[i]`` / ``zeros[i]`` ``(k // 64, n)``); ``__call__`` copies the input into the
    batch's own buffer and returns ``(count, m, n)``, a buffer the next call overwrites.  Results are bit-identical to
    :func:`awq_gemv_w4a16_cuda` layer by layer.  Up to eight rows, group size 64.  No counterpart in the reference.
    """

    def __init__(self, kernels, scales, zeros, m: int, n: int, k: int):
        import ctypes

        if not 1 <= m <= 8:
            raise ValueError(f"m={m}: a batched launch takes up to eight rows")
        _lib.require_cuda(*kernels, *scales, *zeros)
        count, dev, dtype = len(kernels), kernels[0].device, scales[0].dtype
        if count == 0 or len(scales) != count or len(zeros) != count:
            raise ValueError("kernels, scales and zeros must be equally long, non-empty lists")
        if n * k // 2 >= 1 << 32:
            raise RuntimeError(f"AWQ weight of {n * k // 2} bytes: 4 GiB and more are not supported (32-bit offsets)")
        self.m, self.n, self.k, self.count = m, n, k, count
        self.x = torch.zeros(m, k, dtype=dtype, device=dev)
        self.out = torch.empty(count, m, n, dtype=dtype, device=dev)
        self._keep = (list(kernels), list(scales), list(zeros))
        table = (_lib.AwqGemvArgs * count)()
        for i, (q, sc, z) in enumerate(zip(kernels, scales, zeros)):
            if q.element_size() * q.numel() != n * k // 2 or not q.is_contiguous() or q.data_ptr() % 16:
                raise ValueError(f"problem {i}: unexpected packed AWQ weight {tuple(q.shape)} for n={n}, k={k}")
            for name, t in (("scales", sc), ("zeros", z)):
                if t.shape != (k // 64, n) or t.dtype != dtype or t.stride() != (n, 1) or t.data_ptr() % 16 or t.device != dev:
                    raise ValueError(f"problem {i}: {name} must be a contiguous ({k // 64}, {n}) {dtype} tensor on {dev}")
            table[i] = _lib.AwqGemvArgs(x=self.x.data_ptr(), qweight=q.data_ptr(), scales=sc.data_ptr(), zeros=z.data_ptr(),
                                        out=self.out[i].data_ptr(), M=m, N=n, K=k, ld_x=k, ld_scales=n, ld_out=n,
                                        dtype=_lib.dtype_code(dtype))  # fmt: skip
        self._first = table[0]
        raw = torch.frombuffer(bytearray(bytes(table)), dtype=torch.uint8)
        self._table = raw.to(dev)  # the device copy the kernel reads its pointers from

    def __call__(self, in_feats: torch.Tensor) -> torch.Tensor:
        self.x.copy_(in_feats.reshape(self.m, self.k))
        with torch.cuda.device(self.x.device):
            _lib.check(_lib.load().svdq_awq_gemv_w4a16_batched(self._first, self._table.data_ptr(), self.count, _lib.stream_of(self.x)))
        return self.out


def awq_dequantize(
    kernel: torch.Tensor,
    scaling_factors: torch.Tensor,
    zeros: torch.Tensor,
    n: int,
    k: int,
    group_size: int,
    dtype: torch.dtype,
) -> torch.Tensor:
    """
    Unpack a TinyChat-packed AWQ W4 weight to a dense ``(n, k)`` tensor ``q * scaling_factors + zeros`` of ``dtype``
    (reference: nunchaku/ops/triton/awq.py:83-118).
    """
    _lib.require_cuda(kernel, scaling_factors, zeros)
    if kernel.element_size() * kernel.numel() != n * k // 2 or not kernel.is_contiguous():
        raise ValueError(f"unexpected packed AWQ weight shape {tuple(kernel.shape)} for n={n}, k={k}")
    if group_size <= 0 or k % group_size:
        raise ValueError(f"group_size={group_size} does not divide k={k}")
    groups = k // group_size
    if scaling_factors.shape != (groups, n) or zeros.shape != (groups, n):
        raise ValueError(f"scaling_factors / zeros must be ({groups}, {n})")
    if scaling_factors.dtype != dtype or zeros.dtype != dtype:
        raise ValueError("scaling_factors / zeros must have the output dtype")
    if scaling_factors.stride(1) != 1 or zeros.stride() != scaling_factors.stride():
        scaling_factors, zeros = scaling_factors.contiguous(), zeros.contiguous()
    out = torch.empty(n, k, dtype=dtype, device=kernel.device)
    with torch.cuda.device(kernel.device):
        _lib.check(_lib.load().svdq_awq_dequantize(kernel.data_ptr(), scaling_factors.data_ptr(), zeros.data_ptr(),
                                                   out.data_ptr(), n, k, group_size, scaling_factors.stride(0),
                                                   out.stride(0), _lib.dtype_code(dtype), _lib.stream_of(kernel)))  # fmt: skip
    return out


def awq_gemm_w4a16(
    in_feats: torch.Tensor,
    kernel: torch.Tensor,
    scaling_factors: torch.Tensor,
    zeros: torch.Tensor,
    group_size: int = 128,
) -> torch.Tensor:
    """
    AWQ W4A16 GEMM for larger batches (reference: nunchaku/ops/triton/awq.py:232-251): the weight is decoded once by
    :func:`awq_dequantize`, the product is a dense library matmul.
    """
    shape = in_feats.shape
    k = shape[-1]
    x = in_feats.reshape(-1, k)
    n = scaling_factors.shape[-1]
    w = awq_dequantize(kernel, scaling_factors, zeros, n, k, group_size, x.dtype)
    return torch.matmul(x, w.t()).reshape(*shape[:-1], n)


def gemv_awq(in_feats, kernel, scaling_factors, zeros, m: int, n: int, k: int, group_size: int) -> torch.Tensor:
    """The reference's dispatcher name for :func:`awq_gemv_w4a16_cuda` (nunchaku/ops/dispatch.py:19-34)."""
    return awq_gemv_w4a16_cuda(in_feats, kernel, scaling_factors, zeros, m, n, k, group_size)


def gemm_awq(in_feats, kernel, scaling_factors, zeros) -> torch.Tensor:
    """The reference's dispatcher name for :func:`awq_gemm_w4a16` (nunchaku/ops/dispatch.py:37-49)."""
    return awq_gemm_w4a16(in_feats, kernel, scaling_factors, zeros)
