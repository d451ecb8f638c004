"""GPU parity of the fused GEMM epilogues (Q/K RMSNorm + RoPE; GELU + next-layer requantization with LoRA-down) and of
the composite operators built on them, against the CPU oracle."""

import pytest
import torch

from oracle import svdq_oracle as O
from parity_bars import assert_requantized_like_the_reference

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True, params=["none", "all"], ids=["int8-loop", "fp8-loop"])
def main_loop(request):
    """Every test runs through both GEMM main loops: packed weights (int8 MFMA) and pre-split weights (fp8 MFMA)."""
    from nunchaku_rocm_amd.ops import gemm as G

    old, G.USE_WEIGHT_PLANES = G.USE_WEIGHT_PLANES, request.param
    yield request.param
    G.USE_WEIGHT_PLANES = old
TOL = 1e-2


def _problem(M, N, K, R, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    return {
        "act": torch.randint(0, 256, (M, K // 2), generator=g, dtype=torch.uint8),
        "wgt": torch.randint(0, 256, (N, K // 2), generator=g, dtype=torch.uint8),
        "asc": (torch.rand(K // 64, M, generator=g) * 0.02 + 0.01).to(dtype),
        "wsc": (torch.rand(K // 64, N, generator=g) * 0.02 + 0.01).to(dtype),
        "bias": torch.randn(N, generator=g).to(dtype),
        "la": torch.randn(M, R, generator=g),
        "lu": (torch.randn(N, R, generator=g) * 0.1).to(dtype),
    }


@pytest.mark.parametrize("unsigned", [False, True])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,H,actual_m", [(136, 1, 130), (256, 2, 256)])
def test_qk_norm_rope(dev, M, H, actual_m, unsigned, dtype):
    from nunchaku_rocm_amd import ops

    print(f"case M={M} H={H} actual_m={actual_m} unsigned={unsigned} {dtype}", flush=True)
    N, K, R = 3 * H * 128, 256, 16
    p = _problem(M, N, K, R, dtype, seed=M + H)
    g = torch.Generator().manual_seed(99)
    nq = (torch.rand(128, generator=g) + 0.5).to(dtype)
    nk = (torch.rand(128, generator=g) + 0.5).to(dtype)
    theta = torch.rand(actual_m, 64, generator=g) * 6.28
    rot = torch.stack([torch.sin(theta), torch.cos(theta)], -1).reshape(actual_m, 64, 1, 2).float()
    d = lambda t: t.to(dev)  # noqa: E731
    buf = torch.full((actual_m + 8, N), float("nan"), dtype=dtype, device=dev)
    kw = dict(act=d(p["act"]), wgt=d(p["wgt"]), ascales=d(p["asc"]), wscales=d(p["wsc"]), bias=d(p["bias"]),
              lora_act_in=d(p["la"]), lora_up=d(p["lu"]), act_unsigned=unsigned)  # fmt: skip
    ops.svdq_gemm_w4a4_cuda(out=buf[:actual_m], norm_q=d(nq), norm_k=d(nk), rotary_emb=d(rot), **kw)
    plain = torch.empty(actual_m, N, dtype=dtype, device=dev)
    ops.svdq_gemm_w4a4_cuda(out=plain, **kw)
    # the same from the (rows, 128) table itself instead of its re-laid-out copy: the same bits
    from nunchaku_rocm_amd.ops import gemm as gemm_mod

    natural = torch.empty(actual_m, N, dtype=dtype, device=dev)
    gemm_mod.USE_BLOCKED_ROTARY = False
    try:
        ops.svdq_gemm_w4a4_cuda(out=natural, norm_q=d(nq), norm_k=d(nk), rotary_emb=d(rot), **kw)
    finally:
        gemm_mod.USE_BLOCKED_ROTARY = True
    torch.cuda.synchronize()
    assert bool(buf[actual_m:].isnan().all())
    assert torch.equal(buf[:actual_m].view(torch.int16), natural.view(torch.int16))
    out = buf[:actual_m].cpu()
    lin = O.gemm_w4a4(p["act"], p["wgt"], p["asc"], p["wsc"], p["bias"], p["la"], p["lu"], unsigned)[:actual_m]
    ref = O.qk_norm_rope(lin, nq, nk, rot.reshape(actual_m, 128))
    assert O.max_rel_err(out[:, : 2 * N // 3], ref[:, : 2 * N // 3]) <= TOL
    # the V third is exactly the plain GEMM's output
    assert torch.equal(out[:, 2 * N // 3 :].view(torch.int16), plain[:, 2 * N // 3 :].cpu().view(torch.int16))


@pytest.mark.parametrize("unsigned", [False, True])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,N,R2,store_out", [(144, 256, 48, True), (64, 512, 32, False), (128, 128, 0, False), (80, 256, 288, False)])
def test_gelu_quant_epilogue(dev, M, N, R2, store_out, unsigned, dtype):
    from nunchaku_rocm_amd import ops

    print(f"case M={M} N={N} R2={R2} store_out={store_out} unsigned={unsigned} {dtype}", flush=True)
    K, R = 256, 16
    p = _problem(M, N, K, R, dtype, seed=N + R2)
    g = torch.Generator().manual_seed(98)
    smooth = (torch.rand(N, generator=g) + 0.5).to(dtype)
    ld = (torch.randn(N, max(R2, 16), generator=g) * 0.1).to(dtype)[:, :R2].contiguous() if R2 else None
    d = lambda t: None if t is None else t.to(dev)  # noqa: E731
    qout = torch.zeros(M + 16, N // 2, dtype=torch.uint8, device=dev)
    osc = torch.empty(N // 64, M, dtype=dtype, device=dev)
    lao = torch.empty(M, R2, dtype=torch.float32, device=dev) if R2 else None
    out = torch.empty(M, N, dtype=dtype, device=dev) if store_out else None
    for _ in range(2):  # run twice: must be deterministic and must not depend on scratch contents
        ops.svdq_gemm_w4a4_cuda(
            act=d(p["act"]), wgt=d(p["wgt"]), out=out, qout=qout, ascales=d(p["asc"]), wscales=d(p["wsc"]), oscales=osc,
            lora_act_in=d(p["la"]), lora_up=d(p["lu"]), lora_down=d(ld), lora_act_out=lao, bias=d(p["bias"]),
            smooth_factor=d(smooth), act_unsigned=unsigned,
        )  # fmt: skip
        torch.cuda.synchronize()
        first = (qout.clone(), osc.clone(), lao.clone() if R2 else None) if _ == 0 else first
    assert torch.equal(first[0], qout) and torch.equal(first[1].view(torch.int16), osc.view(torch.int16))
    assert R2 == 0 or torch.equal(first[2], lao)
    assert (qout[M:] == 0).all()  # rows past M untouched
    if R2:
        # the LoRA-down weight read from its transposed copy instead of the copy in the epilogue's own order: the same bits
        from nunchaku_rocm_amd.ops import gemm as gemm_mod

        gemm_mod.USE_BLOCKED_LORA_DOWN = False
        try:
            lao2 = torch.empty_like(lao)
            ops.svdq_gemm_w4a4_cuda(
                act=d(p["act"]), wgt=d(p["wgt"]), out=out, qout=qout, ascales=d(p["asc"]), wscales=d(p["wsc"]), oscales=osc,
                lora_act_in=d(p["la"]), lora_up=d(p["lu"]), lora_down=d(ld), lora_act_out=lao2, bias=d(p["bias"]),
                smooth_factor=d(smooth), act_unsigned=unsigned,
            )  # fmt: skip
            torch.cuda.synchronize()
        finally:
            gemm_mod.USE_BLOCKED_LORA_DOWN = True
        assert torch.equal(first[0], qout) and torch.equal(first[2], lao2)

    lin = O.gemm_w4a4(p["act"], p["wgt"], p["asc"], p["wsc"], p["bias"], p["la"], p["lu"], unsigned)
    rp, rs, rl, rc = O.gelu_quant(lin, smooth, ld, dtype)
    assert_requantized_like_the_reference(O.unpack_int4(qout[:M].cpu(), False), rc, osc.cpu(), rs, dtype)
    if R2:
        assert (lao.cpu() - rl).abs().max() <= TOL * rl.abs().max()
    if store_out:
        assert O.max_rel_err(out.cpu(), lin) <= TOL


def test_fused_ops_on_flux_block_shapes(dev):
    """fc1 (3072 -> 12288) + GELU + requantization -> fc2 (12288 -> 3072, unsigned activations), and the QKV projection
    (3072 -> 9216) with Q/K RMSNorm + RoPE on the 64x64 image grid + 512 text tokens; oracle on a row sample."""
    from nunchaku_rocm_amd import ops
    from nunchaku_rocm_amd.linear import SVDQW4A4Linear

    M, C, H4 = 4608, 3072, 12288

    def module(K, N, seed, act_unsigned=False):
        lin = O.make_svdq_linear(K, N, seed=seed)
        mod = SVDQW4A4Linear(K, N, rank=32, act_unsigned=act_unsigned, device=dev)
        with torch.no_grad():
            for name in ("qweight", "wscales", "smooth_factor", "proj_down", "proj_up", "bias"):
                getattr(mod, name).copy_(lin[name])
        return mod, lin

    x = O.make_activations(M, C, seed=41)
    rows = torch.randperm(M, generator=torch.Generator().manual_seed(5))[:96].sort().values

    # --- MLP
    fc1, l1 = module(C, H4, 42)
    fc2, l2 = module(H4, C, 43, act_unsigned=True)
    y = ops.fused_gelu_mlp(x.to(dev).view(1, M, C), fc1, fc2).view(M, C)
    torch.cuda.synchronize()
    rp, rs, rl, _ = O.quantize_act(x[rows], l1["proj_down"], l1["smooth_factor"])
    h = O.gemm_w4a4(rp, l1["qweight"], rs, l1["wscales"], l1["bias"], rl, l1["proj_up"])
    hp, hs, hl, _ = O.gelu_quant(h, l2["smooth_factor"], l2["proj_down"], torch.bfloat16)
    ref = O.gemm_w4a4(hp, l2["qweight"], hs, l2["wscales"], l2["bias"], hl, l2["proj_up"], act_unsigned=True)
    err = O.max_rel_err(y[rows].cpu(), ref)
    print(f"fused_gelu_mlp max rel err {err:.3e}", flush=True)
    assert err <= TOL

    # --- QKV with RMSNorm + RoPE
    qkv, lq = module(C, 3 * C, 44)
    nq = torch.nn.RMSNorm(128, eps=1e-6, device=dev, dtype=torch.bfloat16)
    nk = torch.nn.RMSNorm(128, eps=1e-6, device=dev, dtype=torch.bfloat16)
    g = torch.Generator().manual_seed(45)
    with torch.no_grad():
        nq.weight.copy_((torch.rand(128, generator=g) + 0.5).to(torch.bfloat16))
        nk.weight.copy_((torch.rand(128, generator=g) + 0.5).to(torch.bfloat16))
    rot = O.flux_rotary(O.flux_ids(512, 64, 64))
    out = ops.fused_qkv_norm_rottary(x.to(dev).view(1, M, C), qkv, nq, nk, rot.to(dev)).view(M, 3 * C)
    torch.cuda.synchronize()
    rp, rs, rl, _ = O.quantize_act(x[rows], lq["proj_down"], lq["smooth_factor"])
    lin = O.gemm_w4a4(rp, lq["qweight"], rs, lq["wscales"], lq["bias"], rl, lq["proj_up"])
    ref = O.qk_norm_rope(lin, nq.weight.cpu(), nk.weight.cpu(), rot.reshape(M, 128)[rows])
    err = O.max_rel_err(out[rows].cpu(), ref)
    print(f"fused_qkv_norm_rottary max rel err {err:.3e}", flush=True)
    assert err <= TOL


@pytest.mark.parametrize("handover", [0, 2], ids=["matrix", "fp6-codes"])
@pytest.mark.parametrize("zero_mean_weights", [False, True])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_fc1_codes_at_the_flux_size(dev, dtype, zero_mean_weights, main_loop, handover):
    """FLUX.1 fc1 (M = 4608, K = 3072, N = 12288) with GELU + requantization: the int4 codes and scales it hands to fc2,
    as codes, on 192 sampled rows (2.4 M codes, 37 K scales) against the oracle, held to the reference's bar for both
    main loops, both 16-bit types and both weight distributions (codes uniform in [-8, 7], mean -0.5, as the benchmark
    draws them, and codes of zero mean as absmax-quantized checkpoints have).  The fp8 main loop offsets signed
    activations; the offset term it adds per group has no systematic part (a + 8 against the even-k weights, a - 7 against
    the odd-k ones) and is taken out every four stages, so its accumulators stay near the true partial sums.
    ``handover`` 2: activations in and out as fp6 codes in lane order, as the modules pass them (fp8 loop only; there
    is then no offset at all)."""
    from nunchaku_rocm_amd import ops
    from nunchaku_rocm_amd.layout import unblock_activations_f6

    if handover and main_loop != "all":
        return  # the int8 main loop reads the (M, K/2) matrix only (its refusal: test_gpu_gemm.py, test_gpu_blocked.py)

    M, C, H4 = 4608, 3072, 12288
    l1 = O.make_svdq_linear(C, H4, seed=42, dtype=dtype)
    if zero_mean_weights:
        wc = torch.randint(-7, 8, (H4, C), generator=torch.Generator().manual_seed(77), dtype=torch.int32)
        l1["qweight"] = O.pack_int4(wc).view(torch.int8)
    l2 = O.make_svdq_linear(H4, C, seed=43, dtype=dtype)
    x = O.make_activations(M, C, seed=41).to(dtype)
    d1 = {k: v.to(dev) for k, v in l1.items()}
    d2 = {k: v.to(dev) for k, v in l2.items()}
    q1, a1, la1 = ops.svdq_quantize_w4a4_act_fuse_lora_cuda(x.to(dev), lora_down=d1["proj_down"], smooth=d1["smooth_factor"], out_blocked=handover)
    qo = torch.zeros(M, H4 * 3 // 4 if handover else H4 // 2, dtype=torch.uint8, device=dev)
    oo = torch.zeros(H4 // 64, M, dtype=dtype, device=dev)
    lo = torch.zeros(M, 32, dtype=torch.float32, device=dev)
    ops.svdq_gemm_w4a4_cuda(act=q1, wgt=d1["qweight"], qout=qo, ascales=a1, wscales=d1["wscales"], oscales=oo,
                            lora_act_in=la1, lora_up=d1["proj_up"], lora_down=d2["proj_down"], lora_act_out=lo,
                            bias=d1["bias"], smooth_factor=d2["smooth_factor"], act_blocked=handover, qout_blocked=handover)  # fmt: skip
    torch.cuda.synchronize()
    rows = torch.randperm(M, generator=torch.Generator().manual_seed(5))[:192].sort().values
    rp, rs, rl, _ = O.quantize_act(x[rows], l1["proj_down"], l1["smooth_factor"])
    q1m = unblock_activations_f6(q1.cpu()) if handover else q1.cpu()
    qom = unblock_activations_f6(qo.cpu(), True) if handover else qo.cpu()
    assert torch.equal(q1m[rows], rp)
    h = O.gemm_w4a4(rp, l1["qweight"], rs, l1["wscales"], l1["bias"], rl, l1["proj_up"])
    hp, hs, hl, hc = O.gelu_quant(h, l2["smooth_factor"], l2["proj_down"], dtype)
    assert_requantized_like_the_reference(O.unpack_int4(qom[rows], False), hc, oo[:, rows].cpu(), hs, dtype,
                                          what=f"fc1 {main_loop} {dtype} zero-mean={zero_mean_weights} handover={handover}: ")
    assert (lo[rows].cpu() - hl).abs().max() <= TOL * hl.abs().max()


@pytest.mark.parametrize("unsigned", [False, True])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,N,R2", [(144, 256, 48), (64, 512, 32), (128, 128, 0), (80, 256, 160)])
def test_swiglu_quant_epilogue(dev, M, N, R2, unsigned, dtype):
    """``wgt`` rows in the 16-interleaved [gate | up] order; the epilogue quantizes silu(gate) * up (signed int4)."""
    from nunchaku_rocm_amd import ops

    print(f"case M={M} N={N} R2={R2} unsigned={unsigned} {dtype}", flush=True)
    K, R, H = 256, 16, N // 2
    p = _problem(M, N, K, R, dtype, seed=N + R2 + 1)  # natural [gate | up] row order
    g = torch.Generator().manual_seed(97)
    smooth = (torch.rand(H, generator=g) + 0.5).to(dtype)
    ld = (torch.randn(H, max(R2, 16), generator=g) * 0.1).to(dtype)[:, :R2].contiguous() if R2 else None
    idx = O.interleave_swiglu(N)
    d = lambda t: None if t is None else t.to(dev)  # noqa: E731
    qout = torch.zeros(M + 16, H // 2, dtype=torch.uint8, device=dev)
    osc = torch.empty(H // 64, M, dtype=dtype, device=dev)
    lao = torch.empty(M, R2, dtype=torch.float32, device=dev) if R2 else None
    ops.svdq_gemm_w4a4_cuda(
        act=d(p["act"]), wgt=d(p["wgt"][idx].contiguous()), qout=qout, ascales=d(p["asc"]),
        wscales=d(p["wsc"][:, idx].contiguous()), oscales=osc, lora_act_in=d(p["la"]), lora_up=d(p["lu"][idx].contiguous()),
        lora_down=d(ld), lora_act_out=lao, bias=d(p["bias"][idx].contiguous()), smooth_factor=d(smooth),
        act_unsigned=unsigned, fuse_swiglu=True,
    )  # fmt: skip
    torch.cuda.synchronize()
    assert (qout[M:] == 0).all()
    lin = O.gemm_w4a4(p["act"], p["wgt"], p["asc"], p["wsc"], p["bias"], p["la"], p["lu"], unsigned)
    rp, rs, rl, rc = O.swiglu_quant(lin[:, idx], smooth, ld, dtype)
    assert_requantized_like_the_reference(O.unpack_int4(qout[:M].cpu(), True), rc, osc.cpu(), rs, dtype)
    if R2:
        assert (lao.cpu() - rl).abs().max() <= TOL * rl.abs().max()


def test_fused_swiglu_mlp(dev):
    """FLUX.2-style SwiGLU MLP: fc1 (K -> 2H, rows interleaved in place), fused SwiGLU + requantization, fc2 (H -> C)."""
    from nunchaku_rocm_amd import ops
    from nunchaku_rocm_amd.linear import SVDQW4A4Linear

    M, C, H = 320, 512, 1024

    def module(K, N, seed):
        lin = O.make_svdq_linear(K, N, seed=seed)
        mod = SVDQW4A4Linear(K, N, rank=32, device=dev)
        with torch.no_grad():
            for name in ("qweight", "wscales", "smooth_factor", "proj_down", "proj_up", "bias"):
                getattr(mod, name).copy_(lin[name])
        return mod, lin

    fc1, l1 = module(C, 2 * H, 51)
    fc2, l2 = module(H, C, 52)
    ops.interleave_swiglu_linear_(fc1)
    x = O.make_activations(M, C, seed=53)
    y = ops.fused_swiglu_mlp(x.to(dev), fc1, fc2)
    torch.cuda.synchronize()
    assert y.shape == (M, C)
    rp, rs, rl, _ = O.quantize_act(x, l1["proj_down"], l1["smooth_factor"])
    lin = O.gemm_w4a4(rp, l1["qweight"], rs, l1["wscales"], l1["bias"], rl, l1["proj_up"])  # [gate | up]
    hp, hs, hl, _ = O.swiglu_quant(lin[:, O.interleave_swiglu(2 * H)], l2["smooth_factor"], l2["proj_down"], torch.bfloat16)
    ref = O.gemm_w4a4(hp, l2["qweight"], hs, l2["wscales"], l2["bias"], hl, l2["proj_up"])
    err = O.max_rel_err(y.cpu(), ref)
    print(f"fused_swiglu_mlp max rel err {err:.3e}", flush=True)
    assert err <= TOL


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,N,R2,swiglu", [(40, 192, 32, False), (144, 320, 0, False), (40, 256, 16, True)])
def test_requantizing_gemm_on_shapes_the_fused_epilogues_do_not_take(dev, M, N, R2, swiglu, dtype):
    """N not a multiple of 128 or M not a multiple of 16: the 16-bit GEMM output, then the quantizer with its GELU
    prologue (or torch's SiLU product for SwiGLU), as the reference's dispatcher falls back."""
    from nunchaku_rocm_amd import ops

    print(f"case M={M} N={N} R2={R2} swiglu={swiglu} {dtype}", flush=True)
    K, R = 256, 16
    H = N // 2 if swiglu else N
    p = _problem(M, N, K, R, dtype, seed=N + R2 + 7)
    g = torch.Generator().manual_seed(96)
    smooth = (torch.rand(H, generator=g) + 0.5).to(dtype)
    ld = (torch.randn(H, max(R2, 16), generator=g) * 0.1).to(dtype)[:, :R2].contiguous() if R2 else None
    d = lambda t: None if t is None else t.to(dev)  # noqa: E731
    qout = torch.zeros(M + 16, H // 2, dtype=torch.uint8, device=dev)
    osc = torch.empty(H // 64, M, dtype=dtype, device=dev)
    lao = torch.empty(M, R2, dtype=torch.float32, device=dev) if R2 else None
    out = None if swiglu else torch.empty(M, N, dtype=dtype, device=dev)
    ops.svdq_gemm_w4a4_cuda(
        act=d(p["act"]), wgt=d(p["wgt"]), out=out, qout=qout, ascales=d(p["asc"]), wscales=d(p["wsc"]), oscales=osc,
        lora_act_in=d(p["la"]), lora_up=d(p["lu"]), lora_down=d(ld), lora_act_out=lao, bias=d(p["bias"]),
        smooth_factor=d(smooth), fuse_swiglu=swiglu,
    )  # fmt: skip
    torch.cuda.synchronize()
    assert (qout[M:] == 0).all()
    lin = O.gemm_w4a4(p["act"], p["wgt"], p["asc"], p["wsc"], p["bias"], p["la"], p["lu"], False)
    if swiglu:
        x = lin.to(dtype).view(M, N // 32, 2, 16)
        y = (torch.nn.functional.silu(x[:, :, 0]) * x[:, :, 1]).reshape(M, H)
        rp, rs, rl, rc = O.quantize_act(y, ld, smooth)
        tol_rate = 2e-2  # a 16-bit ulp of the GEMM output moves a code now and then
    else:
        assert O.max_rel_err(out.cpu(), lin) <= TOL
        # the quantizer's part is checked on the very output the GPU produced
        rp, rs, rl, rc = O.quantize_act(out.cpu(), ld, smooth, unsigned=True, shift=O.GELU_SHIFT, fuse_gelu=True)
        assert_requantized_like_the_reference(O.unpack_int4(qout[:M].cpu(), False), rc, osc.cpu(), rs.to(dtype), dtype)
        tol_rate = 1e-5
    codes = O.unpack_int4(qout[:M].cpu(), swiglu)
    diff = (codes - rc).abs()
    rate = (diff > 0).float().mean().item()
    print(f"  code mismatch rate {rate:.2e}", flush=True)
    assert diff.max() <= (2 if swiglu else 1) and (rate < tol_rate or (diff > 0).sum() <= 1)
    ulp = 2**-7 if dtype == torch.bfloat16 else 2**-10
    assert ((osc.cpu().float() - rs.float()).abs() <= rs.float().abs() * (4 if swiglu else 1) * ulp + 1e-7).all()
    if R2:
        assert (lao.cpu() - rl).abs().max() <= TOL * rl.abs().max()


def test_rotary_table_in_16_bit(dev):
    """A rotary table that is not fp32 is read as the values it holds (the reference's unfused kernel does the same)."""
    from nunchaku_rocm_amd import ops

    M, H, K, R, dtype = 64, 1, 256, 16, torch.bfloat16
    N = 3 * H * 128
    p = _problem(M, N, K, R, dtype, seed=5)
    g = torch.Generator().manual_seed(95)
    nq = (torch.rand(128, generator=g) + 0.5).to(dtype)
    nk = (torch.rand(128, generator=g) + 0.5).to(dtype)
    theta = torch.rand(M, 64, generator=g) * 6.28
    rot = torch.stack([torch.sin(theta), torch.cos(theta)], -1).reshape(M, 64, 1, 2).to(dtype)
    d = lambda t: t.to(dev)  # noqa: E731
    kw = dict(act=d(p["act"]), wgt=d(p["wgt"]), ascales=d(p["asc"]), wscales=d(p["wsc"]), norm_q=d(nq), norm_k=d(nk))
    a = torch.empty(M, N, dtype=dtype, device=dev)
    b = torch.empty(M, N, dtype=dtype, device=dev)
    ops.svdq_gemm_w4a4_cuda(out=a, rotary_emb=d(rot), **kw)
    ops.svdq_gemm_w4a4_cuda(out=b, rotary_emb=d(rot.float()), **kw)
    torch.cuda.synchronize()
    assert torch.equal(a, b)
