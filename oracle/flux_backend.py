"""Oracle implementation of the four quantized operators and the attention the FLUX.1-shaped harness calls (TEST INFRASTRUCTURE).

Plain torch arithmetic from ``svdq_oracle`` on whatever device the tensors live on, so the same transformer graph can
be evaluated without the HIP library: on the CPU for small configurations, and with ``dense=True`` (one fp32 matmul
of dequantised operands per linear) on a GPU's plain torch kernels for the full-size model.
"""

from __future__ import annotations

import torch

from . import svdq_oracle as O


class OracleBackend:
    def __init__(self, dense: bool = False):
        self.gemm = O.gemm_w4a4_dense if dense else O.gemm_w4a4

    def _lin32(self, x2d, lin, act_unsigned=False):
        qx, sc, la, _ = O.quantize_act(x2d, lin.proj_down, lin.smooth_factor)
        return self.gemm(qx, lin.qweight, sc, lin.wscales, lin.bias, la, lin.proj_up, act_unsigned)

    def linear(self, x, lin):
        B, S, C = x.shape
        return self._lin32(x.reshape(B * S, C), lin).to(x.dtype).view(B, S, -1)

    @staticmethod
    def _mod(x2d, mod):
        return x2d if mod is None else O.layernorm_modulate(x2d, mod[0], mod[1])

    @staticmethod
    def norm_stats(x):
        return None

    @staticmethod
    def gated_residual(x, gate, y, y2=None, want_stats=False, clip=0.0):
        return O.gated_residual(x, gate, y, y2, clip), None

    def gelu_mlp(self, x, fc1, fc2, mod=None):
        B, S, C = x.shape
        h = self._lin32(self._mod(x.reshape(B * S, C), mod), fc1)
        hp, hs, hl, _ = O.gelu_quant(h, fc2.smooth_factor, fc2.proj_down, x.dtype)
        y = self.gemm(hp, fc2.qweight, hs, fc2.wscales, fc2.bias, hl, fc2.proj_up, True)
        return y.to(x.dtype).view(B, S, -1)

    def qkv(self, x, proj, norm_q, norm_k, rot, mod=None):
        B, S, C = x.shape
        lin = self._lin32(self._mod(x.reshape(B * S, C), mod), proj)
        out = O.qk_norm_rope(lin, norm_q.weight, norm_k.weight, rot.reshape(B * S, 128))
        return out.to(x.dtype).view(B, S, -1)

    def awq(self, x, lin):
        N, K = lin.out_features, lin.in_features
        y = O.awq_gemv(x, lin.qweight.view(torch.int16).reshape(N // 4, K), lin.wscales, lin.wzeros).to(x.dtype)
        if lin.bias is not None:
            y = y + lin.bias
        return y

    def attention(self, q, k, v):
        """fp32 softmax(q k^T / sqrt(D)) v on the tensors' device, rounded once to the input type."""
        return torch.nn.functional.scaled_dot_product_attention(q.float(), k.float(), v.float()).to(q.dtype)
