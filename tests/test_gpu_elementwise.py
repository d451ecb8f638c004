"""GPU parity of the fused gated residual update: bit-exact against the oracle's 16-bit op sequence (no transcendental,
no reordered sum in the values); its row statistics against fp64."""

import pytest
import torch

from oracle import svdq_oracle as O

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,S,C,two", [(1, 7, 64, False), (2, 16, 512, True), (1, 300, 3072, True), (3, 5, 8192, False), (1, 4608, 3072, False)])
def test_gated_residual(dev, B, S, C, two, dtype):
    from nunchaku_rocm_amd import ops

    print(f"case B={B} S={S} C={C} two={two} {dtype}", flush=True)
    g = torch.Generator().manual_seed(B * S + C)
    x, y, y2 = (torch.randn(B, S, C, generator=g).to(dtype) for _ in range(3))
    emb = torch.randn(B, C, 3, generator=g).to(dtype)  # gate as an interleaved slice of a projection output
    gate = emb[:, :, 2]
    out, stats = ops.gated_residual(x.to(dev), emb.to(dev)[:, :, 2], y.to(dev), y2.to(dev) if two else None, want_stats=True)
    torch.cuda.synchronize()
    ref = O.gated_residual(x, gate, y, y2 if two else None)
    assert torch.equal(out.cpu().view(torch.int16), ref.view(torch.int16))
    r64 = ref.double().reshape(B * S, C)
    mean, var = r64.mean(dim=1), r64.var(dim=1, unbiased=False)
    assert (stats[:, 0].cpu().double() - mean).abs().max() <= 1e-5
    assert ((stats[:, 1].cpu().double() - 1 / torch.sqrt(var + 1e-6)).abs() <= 1e-5 / torch.sqrt(var + 1e-6)).all()
    # contiguous gate, in place, no statistics: same bits
    xi = x.to(dev).clone()
    out2, st2 = ops.gated_residual(xi, gate.contiguous().to(dev), y.to(dev), y2.to(dev) if two else None, out=xi)
    assert st2 is None and out2.data_ptr() == xi.data_ptr() and torch.equal(out2, out)


def test_statistics_feed_the_norm_prologue(dev):
    """Statistics written by the residual kernel give the same quantizer output as statistics computed from its result."""
    from nunchaku_rocm_amd import ops

    g = torch.Generator().manual_seed(9)
    x, y = (torch.randn(1, 64, 256, generator=g).to(torch.bfloat16).to(dev) for _ in range(2))
    gate, sc, sh = (torch.randn(1, 256, generator=g).to(torch.bfloat16).to(dev) for _ in range(3))
    out, stats = ops.gated_residual(x, gate, y, want_stats=True)
    st2 = ops.layer_norm_stats(out)
    assert torch.allclose(stats, st2, rtol=1e-5, atol=1e-6)
    q1, s1, _ = ops.svdq_quantize_w4a4_act_fuse_lora_cuda(out[0], norm=(sc, sh, stats))
    q2, s2, _ = ops.svdq_quantize_w4a4_act_fuse_lora_cuda(out[0], norm=(sc, sh, st2))
    assert (q1[:64] != q2[:64]).float().mean() < 1e-3


def test_rejects_bad_arguments(dev):
    from nunchaku_rocm_amd import ops

    x = torch.zeros(1, 4, 16384, dtype=torch.bfloat16, device=dev)
    with pytest.raises(NotImplementedError):
        ops.gated_residual(x, torch.zeros(1, 16384, dtype=torch.bfloat16, device=dev), x)
    with pytest.raises(ValueError):
        ops.gated_residual(x, torch.zeros(2, 16384, dtype=torch.bfloat16, device=dev), x)


@pytest.mark.parametrize("two", [False, True])
def test_fp16_clip_like_the_model(dev, two):
    """fp16 hidden states that overflow are limited to +-65504 as ``.clip(-65504, 65504)`` does in the reference model
    (infinities become the limit, NaN stays), and the statistics are those of the limited values."""
    from nunchaku_rocm_amd import ops

    g = torch.Generator().manual_seed(4)
    B, S, C = 1, 40, 256
    x = (torch.randn(B, S, C, generator=g) * 3e4).to(torch.float16)
    y = (torch.randn(B, S, C, generator=g) * 3e4).to(torch.float16)
    y2 = (torch.randn(B, S, C, generator=g) * 3e4).to(torch.float16)
    gate = (torch.randn(B, C, generator=g) * 2).to(torch.float16)
    x[0, 3, 5] = float("nan")
    free, _ = ops.gated_residual(x.to(dev), gate.to(dev), y.to(dev), y2.to(dev) if two else None)
    assert bool(torch.isinf(free).any())  # the case does overflow
    out, stats = ops.gated_residual(x.to(dev), gate.to(dev), y.to(dev), y2.to(dev) if two else None, want_stats=True, clip=65504.0)
    torch.cuda.synchronize()
    ref = O.gated_residual(x, gate, y, y2 if two else None, clip=65504.0)
    plain = O.gated_residual(x, gate, y, y2 if two else None).clip(-65504, 65504)
    assert torch.equal(ref.nan_to_num(0.0), plain.nan_to_num(0.0))
    got = out.cpu()
    assert bool(torch.isnan(got[0, 3, 5])) and bool(torch.isnan(ref[0, 3, 5]))
    assert torch.equal(got.isnan(), ref.isnan())  # inf - inf where x itself overflowed, and the planted NaN
    assert torch.equal(got.nan_to_num(0.0).view(torch.int16), ref.nan_to_num(0.0).view(torch.int16))
    assert float(got.nan_to_num(0.0).float().abs().max()) == 65504.0
    rows = [r for r in range(S) if not bool(ref[0, r].isnan().any())]
    assert rows
    r64 = ref.double().reshape(S, C)[rows]
    assert ((stats[rows, 0].cpu().double() - r64.mean(dim=1)).abs() <= 1e-5 * r64.abs().amax(dim=1)).all()
