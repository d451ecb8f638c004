"""Operator API of the SVDQuant path: same names and signatures as ``nunchaku.ops`` in the reference."""

from .attention import attention_fp16, scaled_dot_product_attention
from .elementwise import gated_residual
from .fused import fused_gelu_mlp, fused_qkv_norm_rottary, fused_swiglu_mlp, interleave_swiglu_linear_
from .gemm import svdq_gemm_w4a4_cuda
from .gemv import AwqGemvBatch, awq_dequantize, awq_gemm_w4a16, awq_gemv_w4a16_cuda, gemm_awq, gemv_awq
from .quantize import (
    layer_norm_stats,
    quantize_w4a4_act,
    quantize_w4a4_act_fuse_lora,
    quantize_w4a4_wgt,
    svdq_quantize_w4a4_act_fuse_lora_cuda,
)

__all__ = [
    "svdq_quantize_w4a4_act_fuse_lora_cuda",
    "quantize_w4a4_act_fuse_lora",
    "quantize_w4a4_act",
    "quantize_w4a4_wgt",
    "svdq_gemm_w4a4_cuda",
    "awq_gemv_w4a16_cuda",
    "AwqGemvBatch",
    "awq_dequantize",
    "awq_gemm_w4a16",
    "gemv_awq",
    "gemm_awq",
    "fused_gelu_mlp",
    "fused_qkv_norm_rottary",
    "fused_swiglu_mlp",
    "interleave_swiglu_linear_",
    "attention_fp16",
    "layer_norm_stats",
    "gated_residual",
    "scaled_dot_product_attention",
]
