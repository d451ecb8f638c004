"""CPU-only checks of the C-ABI boundary: the library loads, exports every symbol the header declares, matches the
ctypes struct layouts, and rejects bad arguments before any launch."""

import ctypes
import os
import re
import subprocess

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "svdq_mi355x.h")


@pytest.fixture(scope="module")
def lib():
    from nunchaku_rocm_amd import _lib

    return _lib.load()


def test_exports_match_header(lib):
    from nunchaku_rocm_amd import _lib

    text = open(HEADER).read()
    declared = set(re.findall(r"^(?:int|size_t|const char \*)\s*\*?(svdq_\w+)\s*\(", text, flags=re.M))
    assert declared == set(_lib.EXPORTS)
    for name in declared:
        assert hasattr(lib, name), name
    assert lib.svdq_abi_version() == _lib.ABI_VERSION


def test_struct_layouts_match_c(tmp_path):
    from nunchaku_rocm_amd import _lib

    src = tmp_path / "sz.c"
    fields = {
        "svdq_gemm_args": ("GemmArgs", ["act", "M", "actual_m", "epilogue", "norm_q", "eps", "qout", "R2", "shift"]),
        "svdq_quantize_args": ("QuantizeArgs", ["x", "M", "ld_x", "dtype", "shift", "norm_stats", "norm_shift", "norm_rows_per_batch", "norm_stride"]),
        "svdq_awq_gemv_args": ("AwqGemvArgs", ["x", "M", "ld_out", "dtype"]),
        "svdq_attention_args": ("AttentionArgs", ["q", "o", "sqb", "som", "B", "D", "dtype", "scale"]),
    }
    body = "".join(
        f'printf("{c} %zu\\n", sizeof({c}));' + "".join(f'printf("{c}.{f} %zu\\n", offsetof({c}, {f}));' for f in fs)
        for c, (_, fs) in fields.items()
    )
    src.write_text(f'#include <stdio.h>\n#include <stddef.h>\n#include "{HEADER}"\nint main(){{{body}return 0;}}\n')
    exe = tmp_path / "sz"
    subprocess.run(["gcc", str(src), "-o", str(exe)], check=True)
    got = dict(line.split() for line in subprocess.run([str(exe)], capture_output=True, text=True, check=True).stdout.splitlines())
    for c, (py, fs) in fields.items():
        cls = getattr(_lib, py)
        assert int(got[c]) == ctypes.sizeof(cls)
        for f in fs:
            assert int(got[f"{c}.{f}"]) == getattr(cls, f).offset, (c, f)


def test_invalid_arguments_are_rejected_without_launch(lib):
    from nunchaku_rocm_amd import _lib

    q = _lib.QuantizeArgs(x=16, out=16, scales=16, M=4, K=100, ld_x=100, ld_out=50, ld_scales=4)
    assert lib.svdq_quantize_act(q, None) == _lib.E_INVALID
    assert b"multiple of 64" in lib.svdq_last_error()
    with pytest.raises(ValueError):
        _lib.check(_lib.E_INVALID)
    g = _lib.GemmArgs(act=16, wgt=16, ascales=16, wscales=16, out=16, M=8, N=8, K=96, ld_act=48, ld_wgt=48)
    assert lib.svdq_gemm_w4a4(g, None) == _lib.E_INVALID  # K % 64
    assert b"K %% 64".replace(b"%%", b"%") in lib.svdq_last_error()
    g = _lib.GemmArgs(act=16, wgt=16, ascales=16, wscales=16, out=16, M=8, N=8, K=128, ld_act=64, ld_wgt=64,
                      ld_ascales=8, ld_wscales=8, ld_out=8, actual_m=8, epilogue=_lib.EPI_SWIGLU_QUANT,
                      qout=16, oscales=16)  # fmt: skip
    rc = lib.svdq_gemm_w4a4(g, None)
    assert rc in (_lib.E_UNSUPPORTED, _lib.E_INVALID)
    a = _lib.AwqGemvArgs(x=16, qweight=16, scales=16, zeros=16, out=16, M=64, N=64, K=64, ld_x=64, ld_scales=64, ld_out=64)
    assert lib.svdq_awq_gemv_w4a16(a, None) == _lib.E_INVALID  # M > 32
    assert lib.svdq_awq_dequantize(16, 16, 16, 16, 8, 64, 48, 8, 64, 0, None) == _lib.E_INVALID  # group size
    assert lib.svdq_awq_dequantize(16, 16, 16, 16, 6, 64, 64, 8, 64, 0, None) == _lib.E_INVALID  # N % 4
    assert lib.svdq_awq_dequantize(16, 16, 16, 16, 8, 64, 64, 8, 32, 0, None) == _lib.E_INVALID  # ld_out < K
    assert lib.svdq_gemm_w4a4(None, None) == _lib.E_INVALID
    at = _lib.AttentionArgs(q=16, k=16, v=16, o=16, B=1, H=1, Tq=8, Tkv=8, D=32)
    assert lib.svdq_attention_fp16(at, None) == _lib.E_UNSUPPORTED  # head dimension
    at = _lib.AttentionArgs(q=16, k=16, v=0, o=16, B=1, H=1, Tq=8, Tkv=8, D=128)
    assert lib.svdq_attention_fp16(at, None) == _lib.E_INVALID  # null tensor
    at = _lib.AttentionArgs(q=16, k=16, v=16, o=16, B=1, H=1, Tq=8, Tkv=8, D=128, skn=128, svn=64)
    assert lib.svdq_attention_fp16(at, None) == _lib.E_INVALID  # value rows overlap
    assert lib.svdq_gemm_w4a4_scratch_bytes(256, 256, 32, _lib.EPI_GELU_QUANT) == 2 * 256 * 32 * 4
    assert lib.svdq_gemm_w4a4_scratch_bytes(256, 256, 32, _lib.EPI_PLAIN) == 0


def test_ops_refuse_cpu_tensors_loudly():
    from nunchaku_rocm_amd import ops

    x = torch.zeros(4, 64, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="no CPU implementation"):
        ops.svdq_quantize_w4a4_act_fuse_lora_cuda(x, lora_down=torch.zeros(64, 16, dtype=torch.bfloat16))
    with pytest.raises(NotImplementedError):
        ops.svdq_quantize_w4a4_act_fuse_lora_cuda(x, fp4=True)
    with pytest.raises(NotImplementedError):
        ops.svdq_gemm_w4a4_cuda(x, x, out_q=x, ascales=x, wscales=x)
    with pytest.raises(RuntimeError, match="no CPU implementation"):
        ops.awq_gemv_w4a16_cuda(x, x, x, x, 4, 4, 64, group_size=128)
    with pytest.raises(RuntimeError, match="no CPU implementation"):
        ops.awq_dequantize(torch.zeros(1, 32, dtype=torch.int32), x[:1, :4], x[:1, :4], 4, 64, 64, torch.bfloat16)


def test_product_never_imports_the_oracle():
    pkg = os.path.join(ROOT, "nunchaku_rocm_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h")):
                text = open(os.path.join(dirpath, f)).read()
                assert not re.search(r"^\s*(from|import)\s+oracle", text, flags=re.M), f
