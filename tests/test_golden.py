"""The committed fixture tests/golden/svdq_small.npz (written by tests/golden/make_fixtures.py): the CPU oracle still
reproduces it bit for bit (no GPU needed), and the GPU kernels match it through the C ABI (``-m gpu``)."""

import os

import numpy as np
import pytest
import torch

from oracle import mma_packer as P
from oracle import svdq_oracle as O

FIX = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "svdq_small.npz")


@pytest.fixture(scope="module")
def fx():
    z = np.load(FIX)  # allow_pickle stays False
    return {k: torch.from_numpy(z[k]) for k in z.files}


def bf(t):
    return t.view(torch.bfloat16)


def close16(a: torch.Tensor, fixture_bits: torch.Tensor) -> bool:
    """16-bit results of fp32 matrix products: a CPU with another thread count may sum in another order, which can move
    a rounded result by one step; everything elementwise or integer is compared bit for bit instead."""
    ref = bf(fixture_bits).float()
    return bool(((a.float() - ref).abs() <= ref.abs() * 2**-7 + 1e-6).all())


def test_oracle_reproduces_the_fixture(fx):
    x, smooth, pd, pu = bf(fx["x"]), bf(fx["smooth"]), bf(fx["proj_down"]), bf(fx["proj_up"])
    qw = fx["qweight"].view(torch.int8)
    q, s, la, _ = O.quantize_act(x, pd, smooth)
    assert torch.equal(q, fx["q_codes"]) and torch.equal(s.view(torch.int16), fx["q_scales"])
    assert torch.allclose(la, fx["q_lora_act"], rtol=1e-5, atol=1e-6)
    assert torch.equal(O.group_acc_i32(q, qw, False, groups=[1])[0], fx["group1_acc"])
    y = O.gemm_w4a4(q, qw, s, bf(fx["wscales"]), bf(fx["bias"]), la, pu).to(torch.bfloat16)
    assert close16(y, fx["gemm_out"])
    yv = O.awq_gemv(bf(fx["awq_x"]), fx["awq_qweight"].view(torch.int16).reshape(32, 256), bf(fx["awq_wscales"]), bf(fx["awq_wzeros"]))
    assert close16(yv.to(torch.bfloat16), fx["awq_out"])
    ao = O.attention_fp16(bf(fx["attn_q"]), bf(fx["attn_k"])[:, :, :37], bf(fx["attn_v"])[:, :, :37], 128**-0.5)
    assert close16(ao, fx["attn_out"])
    xm = O.layernorm_modulate(x, bf(fx["norm_scale"]), bf(fx["norm_shift"]))
    assert torch.equal(xm.view(torch.int16), fx["norm_out"])
    codes = O.unpack_int4(qw, signed=False).to(torch.int32).numpy()
    assert np.array_equal(P.pack_weight(codes), fx["packed_qweight"].numpy())
    assert np.array_equal(P.pack_scale(bf(fx["wscales"]).t().contiguous().view(torch.int16).numpy()), fx["packed_wscales"].numpy())


@pytest.mark.gpu
def test_kernels_match_the_fixture(fx, dev):
    from nunchaku_rocm_amd import layout, ops
    from nunchaku_rocm_amd.ops.gemm import group_acc_i32

    d = lambda t: t.to(dev)  # noqa: E731
    x, smooth, pd, pu = bf(fx["x"]), bf(fx["smooth"]), bf(fx["proj_down"]), bf(fx["proj_up"])
    qw = fx["qweight"].view(torch.int8)
    M = x.shape[0]
    q, s, la = ops.svdq_quantize_w4a4_act_fuse_lora_cuda(d(x), lora_down=d(pd), smooth=d(smooth))
    assert torch.equal(q[:M].cpu(), fx["q_codes"]) and torch.equal(s[:, :M].cpu().view(torch.int16), fx["q_scales"])
    assert (la[:M].cpu() - fx["q_lora_act"]).abs().max() <= 1e-2 * fx["q_lora_act"].abs().max()
    assert torch.equal(group_acc_i32(q[:M].contiguous(), d(qw), 1).cpu(), fx["group1_acc"])
    out = torch.empty(M, qw.shape[0], dtype=torch.bfloat16, device=dev)
    ops.svdq_gemm_w4a4_cuda(act=q, wgt=d(qw), out=out, ascales=s, wscales=d(bf(fx["wscales"])), lora_act_in=la, lora_up=d(pu), bias=d(bf(fx["bias"])))
    assert O.max_rel_err(out.cpu(), bf(fx["gemm_out"])) <= 1e-2
    yv = ops.awq_gemv_w4a16_cuda(d(bf(fx["awq_x"])), d(fx["awq_qweight"]), d(bf(fx["awq_wscales"])), d(bf(fx["awq_wzeros"])), 2, 128, 256)
    assert O.max_rel_err(yv.cpu(), bf(fx["awq_out"])) <= 1e-2
    ao = torch.empty(1, 40, 256, dtype=torch.bfloat16, device=dev)
    ops.attention_fp16(d(bf(fx["attn_q"])), d(bf(fx["attn_k"]))[:, :, :37], d(bf(fx["attn_v"]))[:, :, :37], ao, 128**-0.5)
    assert O.max_rel_err(ao.cpu(), bf(fx["attn_out"])) <= 1e-2
    qn, sn, _ = ops.svdq_quantize_w4a4_act_fuse_lora_cuda(d(x), lora_down=d(pd), smooth=d(smooth), norm=(d(bf(fx["norm_scale"])), d(bf(fx["norm_shift"]))))
    rq, _, _, _ = O.quantize_act(bf(fx["norm_out"]), pd, smooth)
    assert (O.unpack_int4(qn[:M].cpu(), True) - O.unpack_int4(rq, True)).abs().max() <= 1
    nat = layout.unpack_weight_packed_nibbles(d(fx["packed_qweight"]).view(torch.int8), qw.shape[0], 2 * qw.shape[1])
    assert torch.equal(nat.cpu(), fx["qweight"])
    ws = layout.unpack_scale(d(bf(fx["packed_wscales"])), qw.shape[0], group_size=64)
    assert torch.equal(ws.cpu().view(torch.int16), fx["wscales"])
    torch.cuda.synchronize()
