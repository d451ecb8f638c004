"""ctypes binding of ``libsvdq_mi355x.so`` (C ABI: ``include/svdq_mi355x.h``).

torch is here for device memory and streams only: tensors are handed over as raw device pointers and every launch
goes on torch's current HIP stream of the tensor's device, as the reference's native launcher does
(nunchaku/ops/triton/native/hip.py:153-167).
"""

from __future__ import annotations

import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libsvdq_mi355x.so")
ABI_VERSION = 9

BF16, FP16 = 0, 1
EPI_PLAIN, EPI_QK_NORM_ROPE, EPI_GELU_QUANT, EPI_SWIGLU_QUANT = 0, 1, 2, 3
PRE_NONE, PRE_GLU, PRE_GELU = 0, 1, 2
E_INVALID, E_UNSUPPORTED, E_LAUNCH = -1, -2, -3

EXPORTS = (
    "svdq_quantize_act",
    "svdq_row_stats",
    "svdq_gated_residual",
    "svdq_transpose_lora_down",
    "svdq_gemm_w4a4",
    "svdq_gemm_w4a4_set_variant",
    "svdq_block_rotary",
    "svdq_rotary_blocked_bytes",
    "svdq_block_lora_down",
    "svdq_lora_down_blocked_bytes",
    "svdq_gemm_w4a4_scratch_bytes",
    "svdq_gemm_w4a4_static_scratch",
    "svdq_gemm_w4a4_static_scratch_capacity",
    "svdq_gemm_w4a4_static_scratch_prepare",
    "svdq_split_weight_planes",
    "svdq_weight_planes_bytes",
    "svdq_group_acc_i32",
    "svdq_awq_gemv_w4a16",
    "svdq_awq_gemv_w4a16_batched",
    "svdq_awq_dequantize",
    "svdq_attention_fp16",
    "svdq_unpack_mma_weight",
    "svdq_unpack_mma_scale",
    "svdq_unpack_mma_lowrank",
    "svdq_last_error",
    "svdq_abi_version",
)

_vp, _i32, _i64, _f32 = ctypes.c_void_p, ctypes.c_int32, ctypes.c_int64, ctypes.c_float


class QuantizeArgs(ctypes.Structure):
    """``svdq_quantize_args``"""

    _fields_ = (
        [(n, _vp) for n in ("x", "smooth", "lora_down_t", "out", "scales", "lora_act")]
        + [(n, _i32) for n in ("M", "K", "R", "ld_x", "ld_out", "ld_scales", "ld_lora_act", "dtype", "is_unsigned", "prologue")]
        + [("shift", _f32)]
        + [(n, _vp) for n in ("norm_stats", "norm_scale", "norm_shift")]
        + [(n, _i32) for n in ("norm_rows_per_batch", "norm_ld", "norm_stride", "out_blocked", "scales_blocked")]
    )  # fmt: skip


class GemmArgs(ctypes.Structure):
    """``svdq_gemm_args``"""

    _fields_ = (
        [(n, _vp) for n in ("act", "wgt", "wgt_planes", "ascales", "wscales", "bias", "lora_act", "lora_up", "out")]
        + [(n, _i32) for n in ("M", "N", "K", "R", "actual_m", "ld_act", "ld_wgt", "ld_ascales", "ld_wscales",
                               "ld_lora_act", "ld_lora_up", "ld_out", "dtype", "act_unsigned", "epilogue")]
        + [(n, _vp) for n in ("norm_q", "norm_k", "rotary")]
        + [("ld_rotary", _i32), ("eps", _f32)]
        + [(n, _vp) for n in ("qout", "oscales", "smooth_next", "lora_down_t", "lora_act_out", "scratch")]
        + [(n, _i32) for n in ("R2", "ld_qout", "ld_oscales", "ld_lora_act_out")]
        + [("shift", _f32), ("rotary_blocked", _vp), ("lora_down_blocked", _vp), ("act_blocked", _i32), ("qout_blocked", _i32),
           ("ascales_blocked", _i32), ("oscales_blocked", _i32)]
    )  # fmt: skip


class AwqGemvArgs(ctypes.Structure):
    """``svdq_awq_gemv_args``"""

    _fields_ = (
        [(n, _vp) for n in ("x", "qweight", "scales", "zeros", "out")]
        + [(n, _i32) for n in ("M", "N", "K", "ld_x", "ld_scales", "ld_out", "dtype")]
    )  # fmt: skip


class AttentionArgs(ctypes.Structure):
    """``svdq_attention_args``"""

    _fields_ = (
        [(n, _vp) for n in ("q", "k", "v", "o")]
        + [(n, _i64) for n in ("sqb", "sqh", "sqm", "skb", "skh", "skn", "svb", "svh", "svn", "sob", "som")]
        + [(n, _i32) for n in ("B", "H", "Tq", "Tkv", "D", "dtype")]
        + [("scale", _f32)]
    )  # fmt: skip


_lib = None


def load() -> ctypes.CDLL:
    """Load the kernel library (once).  Raises if it is missing: there is no other implementation to fall back to."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `python -m nunchaku_rocm_amd.build` (hipcc, gfx950). "
            "This package has no fallback implementation."
        )
    # torch's own HIP runtime must be the one the kernels launch on: make sure it is mapped before our library
    # resolves its libamdhip64 dependency by SONAME
    if torch.cuda.is_available():
        torch.cuda.init()
    lib = ctypes.CDLL(LIB_PATH, mode=ctypes.RTLD_GLOBAL)
    missing = [s for s in EXPORTS if not hasattr(lib, s)]
    if missing:
        raise RuntimeError(f"{LIB_PATH} does not export {missing}")
    lib.svdq_last_error.restype = ctypes.c_char_p
    lib.svdq_gemm_w4a4_scratch_bytes.restype = ctypes.c_size_t
    lib.svdq_gemm_w4a4_scratch_bytes.argtypes = [_i32, _i32, _i32, _i32]
    lib.svdq_weight_planes_bytes.restype = ctypes.c_size_t
    lib.svdq_weight_planes_bytes.argtypes = [_i32, _i32]
    lib.svdq_split_weight_planes.argtypes = [_vp, _vp, _vp, _i32, _i32, _i32, _i32, _i32, _vp]
    lib.svdq_gated_residual.argtypes = [_vp] * 6 + [_i32] * 9 + [_f32, _f32, _vp]
    lib.svdq_row_stats.argtypes = [_vp, _vp, _i32, _i32, _i32, _i32, _f32, _vp]
    lib.svdq_quantize_act.argtypes = [ctypes.POINTER(QuantizeArgs), _vp]
    lib.svdq_gemm_w4a4.argtypes = [ctypes.POINTER(GemmArgs), _vp]
    lib.svdq_gemm_w4a4_set_variant.argtypes = [_i32]
    lib.svdq_block_rotary.argtypes = [_vp, _vp, _i32, _i32, _vp]
    lib.svdq_rotary_blocked_bytes.restype = ctypes.c_size_t
    lib.svdq_rotary_blocked_bytes.argtypes = [_i32]
    lib.svdq_block_lora_down.argtypes = [_vp, _vp, _i32, _i32, _i32, _vp]
    lib.svdq_lora_down_blocked_bytes.restype = ctypes.c_size_t
    lib.svdq_lora_down_blocked_bytes.argtypes = [_i32, _i32]
    lib.svdq_gemm_w4a4_static_scratch.argtypes = [ctypes.POINTER(GemmArgs), _vp]
    lib.svdq_gemm_w4a4_static_scratch_capacity.restype = ctypes.c_size_t
    lib.svdq_gemm_w4a4_static_scratch_capacity.argtypes = []
    lib.svdq_gemm_w4a4_static_scratch_prepare.argtypes = []
    lib.svdq_awq_gemv_w4a16.argtypes = [ctypes.POINTER(AwqGemvArgs), _vp]
    lib.svdq_awq_gemv_w4a16_batched.argtypes = [ctypes.POINTER(AwqGemvArgs), _vp, _i32, _vp]
    lib.svdq_awq_dequantize.argtypes = [_vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _i32, _i32, _vp]
    lib.svdq_attention_fp16.argtypes = [ctypes.POINTER(AttentionArgs), _vp]
    lib.svdq_unpack_mma_weight.argtypes = [_vp, _vp, _i32, _i32, _i32, _vp]
    lib.svdq_unpack_mma_scale.argtypes = [_vp, _vp, _i32, _i32, _i32, _vp]
    lib.svdq_unpack_mma_lowrank.argtypes = [_vp, _vp, _i32, _i32, _i32, _i32, _vp]
    lib.svdq_transpose_lora_down.argtypes = [_vp, _vp, _i32, _i32, _i32, _vp]
    lib.svdq_group_acc_i32.argtypes = [_vp, _vp, _vp, _i32, _i32, _i32, _i32, _i32, _i32, _i32, _i32, _vp]
    if lib.svdq_abi_version() != ABI_VERSION:
        raise RuntimeError(f"{LIB_PATH} has ABI version {lib.svdq_abi_version()}, expected {ABI_VERSION}: rebuild it")
    _lib = lib
    return lib


def hip_runtimes_mapped() -> list[str]:
    """Paths of the libamdhip64 copies mapped into this process (there must be exactly one once a GPU is in use)."""
    out = set()
    with open("/proc/self/maps") as f:
        for line in f:
            if "libamdhip64" in line:
                out.add(line.split()[-1])
    return sorted(out)


def check(rc: int) -> None:
    """Translate a C return code into the exception the reference's Python layer would raise."""
    if rc == 0:
        return
    msg = load().svdq_last_error().decode()
    if rc == E_INVALID:
        raise ValueError(msg)
    if rc == E_UNSUPPORTED:
        raise NotImplementedError(msg)
    raise RuntimeError(msg)


def dtype_code(dtype: torch.dtype) -> int:
    if dtype == torch.bfloat16:
        return BF16
    if dtype == torch.float16:
        return FP16
    raise ValueError(f"unsupported 16-bit dtype {dtype}")


def ptr(t: torch.Tensor | None):
    return None if t is None else t.data_ptr()


def stream_of(t: torch.Tensor):
    return torch.cuda.current_stream(t.device).cuda_stream


def require_cuda(*tensors: torch.Tensor | None) -> torch.device:
    devs = {t.device for t in tensors if t is not None}
    if len(devs) != 1:
        raise ValueError(f"tensors on different devices: {sorted(map(str, devs))}")
    (dev,) = devs
    if dev.type != "cuda":
        raise RuntimeError(
            f"nunchaku_rocm_amd ops run on an MI355X only (got tensors on {dev}); there is no CPU implementation"
        )
    return dev
