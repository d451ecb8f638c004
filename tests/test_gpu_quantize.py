"""GPU parity of the activation quantizer against the CPU oracle: int4 codes and 16-bit scales bit-exact, LoRA-down
within fp32 accumulation-order noise, pad rows untouched, deterministic."""

import pytest
import torch

from oracle import svdq_oracle as O
from parity_bars import assert_requantized_like_the_reference

pytestmark = pytest.mark.gpu


def _run(x, lin, dev, R, smooth=True, unsigned=False, shift=0.0, pad=0):
    from nunchaku_rocm_amd.ops.quantize import quantize_w4a4_act_fuse_lora

    M, K = x.shape
    ld = lin["proj_down"][:, :R].contiguous() if R else None
    sm = lin["smooth_factor"] if smooth else None
    out = torch.full((M + pad, K // 2), 0xEE, dtype=torch.uint8, device=dev)
    osc = torch.full((K // 64, M + pad), 7.0, dtype=x.dtype, device=dev)
    la = torch.full((M + pad, max(R, 1)), 7.0, dtype=torch.float32, device=dev)[:, :R] if R else None
    quantize_w4a4_act_fuse_lora(
        x.to(dev), out, osc, ld.to(dev) if R else None, la, sm.to(dev) if smooth else None,
        shift_value=shift, unsigned=unsigned,
    )  # fmt: skip
    torch.cuda.synchronize()
    ref = O.quantize_act(x, ld, sm, unsigned=unsigned, shift=shift)
    return (out.cpu(), osc.cpu(), la.cpu() if R else None), ref


@pytest.mark.parametrize("M,K,R", [(1, 128, 16), (16, 256, 32), (130, 384, 48), (257, 3072, 32), (64, 512, 0), (33, 1024, 288),
                                   (40, 640, 64), (18, 3072, 96), (50, 512, 160)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_codes_and_scales_bit_exact(dev, M, K, R, dtype):
    print(f"case M={M} K={K} R={R} {dtype}", flush=True)
    x = O.make_activations(M, K, seed=M + K, dtype=dtype)
    lin = O.make_svdq_linear(K, 64, R=max(R, 16), seed=K, dtype=dtype)
    (out, osc, la), (rp, rs, rl, _) = _run(x, lin, dev, R, pad=5)
    assert torch.equal(out[:M], rp)
    assert torch.equal(osc[:, :M].view(torch.int16), rs.view(torch.int16))
    assert (out[M:] == 0xEE).all() and (osc[:, M:] == 7.0).all()  # pad rows never written
    if R:
        ref64 = x.double() @ lin["proj_down"][:, :R].double()
        assert (la[:M].double() - ref64).abs().max() <= 2e-5 * ref64.abs().max()
        assert (la[M:] == 7.0).all()


@pytest.mark.parametrize("M", [2064, 4112, 4640, 8208])
def test_every_grid_layout_bit_exact(dev, M):
    """The launcher picks 16- or 32-row workgroups and, where CUs would idle, a further workgroup row that only
    quantizes while the others only project (see quantize_grid_y): 2064 rows = 16-row workgroups doing both, 4112 =
    32-row doing both on a 256-CU part, 4640 = 32-row just past the split's limit, 8208 = 16-row again; the small
    shapes of the other tests and M = 4608 take the split layouts."""
    print(f"case M={M}", flush=True)
    K, R = 128, 32
    x = O.make_activations(M, K, seed=M, dtype=torch.bfloat16)
    lin = O.make_svdq_linear(K, 64, R=R, seed=K)
    (out, osc, la), (rp, rs, rl, _) = _run(x, lin, dev, R)
    assert torch.equal(out[:M], rp)
    assert torch.equal(osc[:, :M].view(torch.int16), rs.view(torch.int16))
    ref64 = x.double() @ lin["proj_down"][:, :R].double()
    assert (la[:M].double() - ref64).abs().max() <= 2e-5 * ref64.abs().max()


@pytest.mark.parametrize("M,K", [(512, 3072), (1024, 3072), (96, 320), (48, 704), (2048, 192)])
def test_quantize_only_rows_share_the_groups(dev, M, K):
    """Where CUs are left over the launcher adds up to three workgroup rows that only quantize, each a slice of the
    groups (quantize_grid_y): group counts that do and do not divide by the number of slices, fewer groups than
    wavefronts in a slice, and the largest row count that still takes three slices on a 256-CU part."""
    print(f"case M={M} K={K}", flush=True)
    R = 32
    x = O.make_activations(M, K, seed=M + K, dtype=torch.bfloat16)
    lin = O.make_svdq_linear(K, 64, R=R, seed=K)
    (out, osc, la), (rp, rs, rl, _) = _run(x, lin, dev, R)
    assert torch.equal(out[:M], rp)
    assert torch.equal(osc[:, :M].view(torch.int16), rs.view(torch.int16))
    ref64 = x.double() @ lin["proj_down"][:, :R].double()
    assert (la[:M].double() - ref64).abs().max() <= 2e-5 * ref64.abs().max()


@pytest.mark.parametrize("smooth", [True, False])
def test_unsigned_with_shift_bit_exact(dev, smooth):
    M, K = 96, 512
    g = torch.Generator().manual_seed(3)
    x = (torch.nn.functional.gelu(torch.randn(M, K, generator=g) * 2, approximate="tanh")).to(torch.bfloat16)
    lin = O.make_svdq_linear(K, 64, seed=4)
    (out, osc, la), (rp, rs, rl, _) = _run(x, lin, dev, 32, smooth=smooth, unsigned=True, shift=0.171875)
    assert torch.equal(out, rp)
    assert torch.equal(osc.view(torch.int16), rs.view(torch.int16))


def test_zero_groups_and_ties(dev):
    x = torch.zeros(16, 128, dtype=torch.bfloat16)
    x[1, :64] = torch.arange(64).float().sub(32).mul(0.5).clamp(-7, 7).to(torch.bfloat16)  # exact .5 ties at scale 1
    x[2, 64:] = -3.0
    lin = O.make_svdq_linear(128, 64, seed=5)
    (out, osc, _), (rp, rs, _, _) = _run(x, lin, dev, 0, smooth=False)
    assert torch.equal(out, rp) and torch.equal(osc.view(torch.int16), rs.view(torch.int16))
    (out, osc, _), (rp, rs, _, _) = _run(x, lin, dev, 0, smooth=False, unsigned=True)
    assert torch.equal(out, rp) and torch.equal(osc.view(torch.int16), rs.view(torch.int16))


def test_kernel_multiplies_by_the_reciprocal(dev):
    """Inputs on which ``x * (1 / scale)`` and ``x / scale`` give different codes; the expected codes come from exact
    rational arithmetic (tests/golden/rcp_order_vectors.py)."""
    from nunchaku_rocm_amd import ops
    from test_oracle_pins import _rcp_order_input

    xb, want = _rcp_order_input()
    xp = torch.zeros(16, 64, dtype=torch.bfloat16)
    xp[: xb.shape[0]] = xb
    q, _, _ = ops.svdq_quantize_w4a4_act_fuse_lora_cuda(xp.to(dev))
    codes = O.unpack_int4(q.cpu(), True)
    for i, w in enumerate(want):
        assert int(codes[i, 1 + i]) == w and int(codes[i, 0]) == 7


def test_full_size_qkv_input_bit_exact_and_deterministic(dev):
    """The benchmark configuration: M=4608, K=3072, R=32, outlier channels, smooth U(0.5, 4)."""
    M, K = 4608, 3072
    x = O.make_activations(M, K, seed=1)
    lin = O.make_svdq_linear(K, 64, seed=0)
    (out, osc, la), (rp, rs, rl, _) = _run(x, lin, dev, 32)
    assert torch.equal(out, rp)
    assert torch.equal(osc.view(torch.int16), rs.view(torch.int16))
    assert (la - rl).abs().max() <= 2e-5 * rl.abs().max()
    (out2, osc2, la2), _ = _run(x, lin, dev, 32)
    assert torch.equal(out, out2) and torch.equal(osc.view(torch.int16), osc2.view(torch.int16)) and torch.equal(la, la2)


def test_operator_pads_rows_like_the_reference(dev):
    from nunchaku_rocm_amd import ops

    M, K = 300, 256
    x = O.make_activations(M, K, seed=9).to(dev)
    lin = O.make_svdq_linear(K, 64, seed=9)
    out, osc, la = ops.svdq_quantize_w4a4_act_fuse_lora_cuda(x, lora_down=lin["proj_down"].to(dev), smooth=lin["smooth_factor"].to(dev))
    assert out.shape == (512, K // 2) and osc.shape == (K // 64, 512) and la.shape == (512, 32) and la.dtype == torch.float32
    rp, rs, rl, _ = O.quantize_act(x.cpu(), lin["proj_down"], lin["smooth_factor"])
    assert torch.equal(out[:M].cpu(), rp) and torch.equal(osc[:, :M].cpu().view(torch.int16), rs.view(torch.int16))


def test_fuse_glu_close_to_oracle(dev):
    from nunchaku_rocm_amd.ops.quantize import quantize_w4a4_act_fuse_lora

    M, K = 32, 512
    g = torch.Generator().manual_seed(6)
    x = torch.randn(M, 2 * K, generator=g).to(torch.bfloat16)
    out, osc, _ = quantize_w4a4_act_fuse_lora(x.to(dev), fuse_glu=True)
    rp, rs, _, rc = O.quantize_act(x, fuse_glu=True)
    codes = O.unpack_int4(out.cpu(), True)
    d = (codes - rc).abs()
    assert d.max() <= 1 and ((d > 0).float().mean() < 1e-5 or (d > 0).sum() <= 1)  # exp() differs between libraries
    assert ((osc.cpu().float() - rs.float()).abs() <= rs.float().abs() * 2**-7 + 1e-9).all()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,K,R,batches", [(48, 256, 32, 1), (130, 384, 48, 1), (64, 512, 16, 2), (4608, 3072, 32, 1), (96, 1024, 0, 3),
                                           (64, 512, 128, 2)])
def test_norm_modulate_prologue(dev, M, K, R, batches, dtype):
    """LayerNorm + scale + shift applied inside the quantizer: codes, scales and the LoRA-down product are those of
    the oracle's quantizer fed with the oracle's layernorm_modulate output.  exp-free arithmetic, but the row
    statistics are summed in another order than on the CPU: a 16-bit rounding may flip, so codes may differ by one
    step on a small fraction of entries (the contract of the fused GELU epilogue,
    tests/triton/test_native_epilogues.py:246-253)."""
    from nunchaku_rocm_amd import ops

    print(f"case M={M} K={K} R={R} batches={batches} {dtype}", flush=True)
    g = torch.Generator().manual_seed(M + K)
    x = (torch.randn(M, K, generator=g) * 1.7 + 0.3).to(dtype)
    scale = (1 + 0.3 * torch.randn(batches, K, generator=g)).to(dtype)
    shift = (0.2 * torch.randn(batches, K, generator=g)).to(dtype)
    lin = O.make_svdq_linear(K, 64, R=max(R, 16), seed=K, dtype=dtype)
    ld = lin["proj_down"][:, :R].contiguous() if R else None
    q, s, la = ops.svdq_quantize_w4a4_act_fuse_lora_cuda(x.to(dev), lora_down=None if ld is None else ld.to(dev),
                                                          smooth=lin["smooth_factor"].to(dev), norm=(scale.to(dev), shift.to(dev)))  # fmt: skip
    torch.cuda.synchronize()
    xm = O.layernorm_modulate(x, scale, shift)
    rq, rs, rl, rc = O.quantize_act(xm, ld, lin["smooth_factor"])
    # a group maximum that flipped by one 16-bit step moves the stored scale by up to two of its own steps
    assert_requantized_like_the_reference(O.unpack_int4(q[:M].cpu(), True), rc, s[:, :M].cpu(), rs.to(dtype), dtype, scale_steps=2.01)
    if R:
        assert (la[:M].cpu() - rl).abs().max() <= 1e-2 * rl.abs().max()
    # statistics computed once and passed in give the same bits as computing them inside the call
    st = ops.layer_norm_stats(x.to(dev))
    ref_mean = x.float().mean(dim=1)
    assert (st[:, 0].cpu() - ref_mean).abs().max() <= 1e-5 * (1 + ref_mean.abs().max())
    q2, s2, _ = ops.svdq_quantize_w4a4_act_fuse_lora_cuda(x.to(dev), lora_down=None if ld is None else ld.to(dev),
                                                          smooth=lin["smooth_factor"].to(dev), norm=(scale.to(dev), shift.to(dev), st))  # fmt: skip
    assert torch.equal(q2[:M], q[:M]) and torch.equal(s2[:, :M].view(torch.int16), s[:, :M].view(torch.int16))
    # scale / shift as interleaved slices of one projection output (element stride 6), used where they lie
    emb = torch.zeros(batches, K, 6, dtype=dtype, device=dev)
    emb[:, :, 1], emb[:, :, 0] = scale.to(dev), shift.to(dev)
    q3, s3, _ = ops.svdq_quantize_w4a4_act_fuse_lora_cuda(x.to(dev), lora_down=None if ld is None else ld.to(dev),
                                                          smooth=lin["smooth_factor"].to(dev), norm=(emb[:, :, 1], emb[:, :, 0], st))  # fmt: skip
    assert torch.equal(q3[:M], q[:M]) and torch.equal(s3[:, :M].view(torch.int16), s[:, :M].view(torch.int16))


def test_plain_aliases_and_quantized_product(dev):
    """quantize_w4a4_act / quantize_w4a4_wgt (no smoothing, no LoRA): bit-equal to the oracle, and their outputs are the
    GEMM's natural-layout operands: the int4 product tracks the dense one within the quantization noise."""
    from nunchaku_rocm_amd import ops

    g = torch.Generator().manual_seed(77)
    M, N, K = 96, 160, 512
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = (torch.randn(N, K, generator=g) * 0.05).to(torch.bfloat16)
    qa, sa = ops.quantize_w4a4_act(x.to(dev))
    qw, sw = ops.quantize_w4a4_wgt(w.to(dev))
    torch.cuda.synchronize()
    ra = O.quantize_act(x)
    rw = O.quantize_act(w)
    assert qa.shape == (M, K // 2) and sa.shape == (K // 64, M) and qw.shape == (N, K // 2) and sw.shape == (K // 64, N)
    assert torch.equal(qa.cpu(), ra[0]) and torch.equal(sa.cpu(), ra[1])
    assert torch.equal(qw.cpu(), rw[0]) and torch.equal(sw.cpu(), rw[1])
    out = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
    ops.svdq_gemm_w4a4_cuda(qa, qw, out=out, ascales=sa, wscales=sw)
    torch.cuda.synchronize()
    ref = O.gemm_w4a4(ra[0], rw[0], ra[1], rw[1])
    assert O.max_rel_err(out.cpu(), ref) <= 1e-2
    dense = x.float() @ w.float().t()
    # int4 x int4 with per-group absmax scales: relative error of a dot product of 512 terms is a few percent
    assert O.cosine(out.cpu().float(), dense) >= 0.98
    with pytest.raises(NotImplementedError):
        ops.quantize_w4a4_wgt(w.to(dev), fp4=True)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,K,R", [(48, 256, 32), (130, 384, 0), (257, 1024, 48)])
def test_gelu_prologue(dev, M, K, R, dtype):
    """fuse_gelu: tanh-GELU, LoRA-down on its rounded value, + 0.171875, smoothing, unsigned codes.  exp() differs
    between implementations by an ulp, so codes carry the reference's own bar: off by at most one, rarely."""
    from nunchaku_rocm_amd.ops.quantize import quantize_w4a4_act_fuse_lora

    print(f"case M={M} K={K} R={R} {dtype}", flush=True)
    lin = O.make_svdq_linear(K, 64, R=max(R, 16), seed=K + R, dtype=dtype)
    x = (O.make_activations(M, K, seed=M, dtype=dtype).float() * 0.3).to(dtype)
    ld = lin["proj_down"][:, :R].contiguous() if R else None
    sm = lin["smooth_factor"]
    out, osc, la = quantize_w4a4_act_fuse_lora(x.to(dev), lora_down=ld.to(dev) if R else None, smooth=sm.to(dev),
                                               fuse_gelu=True, shift_value=O.GELU_SHIFT, unsigned=True)  # fmt: skip
    torch.cuda.synchronize()
    rp, rs, rl, rc = O.quantize_act(x, ld, sm, unsigned=True, shift=O.GELU_SHIFT, fuse_gelu=True)
    assert_requantized_like_the_reference(O.unpack_int4(out.cpu(), False), rc, osc.cpu(), rs.to(dtype), dtype)
    if R:
        assert (la.cpu() - rl).abs().max() <= 1e-2 * rl.abs().max()
    with pytest.raises(NotImplementedError):
        quantize_w4a4_act_fuse_lora(torch.zeros(16, 128, dtype=dtype, device=dev), fuse_gelu=True, fuse_glu=True)


def test_full_size_invariants(dev):
    """On the whole (4608, 3072) input, on the GPU: multiplying the input by two leaves the codes alone and doubles the
    scales and the LoRA hidden state exactly; permuting the rows permutes every output."""
    from nunchaku_rocm_amd.ops.quantize import quantize_w4a4_act_fuse_lora

    M, K, R = 4608, 3072, 32
    lin = O.make_svdq_linear(K, 64, R=R, seed=3)
    x = O.make_activations(M, K, seed=4).to(dev)
    ld, sm = lin["proj_down"].to(dev), lin["smooth_factor"].to(dev)
    q0, s0, l0 = quantize_w4a4_act_fuse_lora(x, lora_down=ld, smooth=sm)
    q1, s1, l1 = quantize_w4a4_act_fuse_lora(x * 2, lora_down=ld, smooth=sm)
    assert torch.equal(q0, q1) and torch.equal(s1, s0 * 2) and torch.equal(l1, l0 * 2)
    pm = torch.randperm(M, generator=torch.Generator(device=dev).manual_seed(5), device=dev)
    q2, s2, l2 = quantize_w4a4_act_fuse_lora(x[pm].contiguous(), lora_down=ld, smooth=sm)
    assert torch.equal(q2, q0[pm]) and torch.equal(s2, s0[:, pm]) and torch.equal(l2, l0[pm])
    # every group uses its full range: the largest code magnitude of a group with a non-zero scale is 7 (or -8 never
    # without a 7-magnitude partner: |x| / (absmax / 7) <= 7)
    codes = O.unpack_int4(q0.cpu(), True).view(M, K // 64, 64)
    nz = s0.cpu().t().float() != 0
    assert bool((codes.abs().amax(dim=2)[nz] == 7).all()) and int(codes.min()) >= -7
