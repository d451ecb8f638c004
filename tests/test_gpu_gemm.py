"""GPU parity of the W4A4 GEMM against the CPU oracle.

Bars: int32 group accumulators bit-exact; with unit scales the output is the exactly rounded integer GEMM
(bit-exact); with real scales the 16-bit output is within max-rel-err 1e-2 of the oracle (relative to max |ref|, the
reference self-test's measure) -- in practice within about one output ulp; rows past ``actual_m`` are never written;
two runs give identical bits.
"""

import pytest
import torch

from oracle import svdq_oracle as O

pytestmark = pytest.mark.gpu

TOL = 1e-2  # max |out - ref| / max |ref| per layer


@pytest.fixture(autouse=True, params=["none", "all"], ids=["int8-loop", "fp8-loop"])
def main_loop(request):
    """Every test runs through both main loops: packed weights (int8 MFMA) and pre-split weights (fp8 MFMA)."""
    from nunchaku_rocm_amd.ops import gemm as G

    old, G.USE_WEIGHT_PLANES = G.USE_WEIGHT_PLANES, request.param
    yield request.param
    G.USE_WEIGHT_PLANES = old


def _rand_problem(M, N, K, R, dtype, seed, scale=0.02):
    g = torch.Generator().manual_seed(seed)
    p = {
        "act": torch.randint(0, 256, (M, K // 2), generator=g, dtype=torch.uint8),
        "wgt": torch.randint(0, 256, (N, K // 2), generator=g, dtype=torch.uint8),
        "asc": (torch.rand(K // 64, M, generator=g) * scale + scale / 2).to(dtype),
        "wsc": (torch.rand(K // 64, N, generator=g) * scale + scale / 2).to(dtype),
        "bias": torch.randn(N, generator=g).to(dtype),
        "la": torch.randn(M, max(R, 16), generator=g)[:, :R].contiguous() if R else None,
        "lu": (torch.randn(N, max(R, 16), generator=g) * 0.1).to(dtype)[:, :R].contiguous() if R else None,
    }
    return p


def _gpu_gemm(p, dev, actual_m=None, unsigned=False, dtype=torch.bfloat16, canary=8, **extra):
    from nunchaku_rocm_amd import ops

    M, N = p["act"].shape[0], p["wgt"].shape[0]
    am = M if actual_m is None else actual_m
    buf = torch.full((am + canary, N), float("nan"), dtype=dtype, device=dev)
    d = lambda t: t.to(dev) if isinstance(t, torch.Tensor) else t  # noqa: E731
    ops.svdq_gemm_w4a4_cuda(
        act=d(p["act"]), wgt=d(p["wgt"]), out=buf[:am], ascales=d(p["asc"]), wscales=d(p["wsc"]), bias=d(p.get("bias")),
        lora_act_in=d(p.get("la")), lora_up=d(p.get("lu")), act_unsigned=unsigned, **{k: d(v) for k, v in extra.items()},
    )  # fmt: skip
    torch.cuda.synchronize()
    assert bool(buf[am:].isnan().all()), "rows past actual_m were written"
    return buf[:am].cpu()


@pytest.mark.parametrize("unsigned", [False, True])
@pytest.mark.parametrize("M,N,K", [(32, 32, 64), (136, 264, 256), (257, 96, 384)])
def test_group_accumulators_bit_exact(dev, M, N, K, unsigned, main_loop):
    from nunchaku_rocm_amd.ops.gemm import group_acc_i32

    print(f"case M={M} N={N} K={K} unsigned={unsigned}", flush=True)
    p = _rand_problem(M, N, K, 0, torch.bfloat16, seed=M + N)
    ref = O.group_acc_i32(p["act"], p["wgt"], unsigned)
    for g in range(K // 64):
        got = group_acc_i32(p["act"].to(dev), p["wgt"].to(dev), g, unsigned, fp8_path=main_loop == "all").cpu()
        assert torch.equal(got, ref[g]), f"group {g}"


@pytest.mark.parametrize("unsigned", [False, True])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("K", [256, 192])
def test_unit_scales_exact_integer_gemm(dev, unsigned, dtype, K):
    """With all scales 1 every fp32 partial sum is an exact integer, so the output must equal the oracle's bit for bit."""
    M, N = 136, 264
    p = _rand_problem(M, N, K, 0, dtype, seed=1)
    p["asc"] = torch.ones_like(p["asc"])
    p["wsc"] = torch.ones_like(p["wsc"])
    p["bias"] = None
    out = _gpu_gemm(p, dev, unsigned=unsigned, dtype=dtype)
    ref = O.gemm_w4a4(p["act"], p["wgt"], p["asc"], p["wsc"], act_unsigned=unsigned).to(dtype)
    assert torch.equal(out.view(torch.int16), ref.view(torch.int16))


@pytest.mark.parametrize("unsigned", [False, True])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("K", [256, 192, 64, 1024])
def test_unit_scales_exact_integer_gemm_from_fp6_codes(dev, unsigned, dtype, K, main_loop):
    """The same through the fp6 x fp6 instruction (activations as fp6 codes in lane order, full range of both operands;
    K = 64 makes the output one group's accumulator, K = 1024 takes the blocked scales too): exact integers, the
    oracle's bits."""
    if main_loop != "all":
        return  # the int8 main loop reads the matrix only
    M, N = 136, 264
    p = _rand_problem(M, N, K, 0, dtype, seed=2)
    p["asc"] = torch.ones_like(p["asc"])
    p["wsc"] = torch.ones_like(p["wsc"])
    p["bias"] = None
    ref = O.gemm_w4a4(p["act"], p["wgt"], p["asc"], p["wsc"], act_unsigned=unsigned).to(dtype)
    q = _as_fp6_codes(p, unsigned)
    out = _gpu_gemm(q, dev, actual_m=M, unsigned=unsigned, dtype=dtype, act_blocked=2)
    assert torch.equal(out.view(torch.int16), ref.view(torch.int16))
    if K % 512 == 0:
        q["asc"] = torch.ones_like(q["asc"])  # all ones, pad rows included: the same bytes in either order
        out = _gpu_gemm(q, dev, actual_m=M, unsigned=unsigned, dtype=dtype, act_blocked=3)
        assert torch.equal(out.view(torch.int16), ref.view(torch.int16))


@pytest.mark.parametrize("unsigned", [False, True])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,N,K,R,actual_m", [(136, 264, 256, 16, 130), (256, 256, 512, 32, 256), (64, 128, 1024, 48, 64), (128, 512, 256, 0, 100),
                                                   (160, 256, 256, 160, 150), (72, 136, 512, 288, 72),  # ranks grown at run time (32 + sum of LoRA ranks)
                                                   (136, 264, 64, 16, 136), (130, 200, 192, 32, 130), (256, 128, 448, 0, 200)])  # K / 64 odd
def test_scaled_gemm_bias_lora(dev, M, N, K, R, actual_m, unsigned, dtype):
    print(f"case M={M} N={N} K={K} R={R} actual_m={actual_m} unsigned={unsigned} {dtype}", flush=True)
    p = _rand_problem(M, N, K, R, dtype, seed=K + R)
    out = _gpu_gemm(p, dev, actual_m=actual_m, unsigned=unsigned, dtype=dtype)
    ref = O.gemm_w4a4(p["act"], p["wgt"], p["asc"], p["wsc"], p["bias"], p["la"], p["lu"], unsigned)[:actual_m]
    assert O.max_rel_err(out, ref) <= TOL
    ulp = 2**-7 if dtype == torch.bfloat16 else 2**-10
    assert ((out.float() - ref).abs() <= ref.abs() * ulp * 1.01 + 1e-3 * ref.abs().max()).all()
    out2 = _gpu_gemm(p, dev, actual_m=actual_m, unsigned=unsigned, dtype=dtype)
    assert torch.equal(out.view(torch.int16), out2.view(torch.int16))


def _as_fp6_codes(p, unsigned):
    """The problem with its activations as fp6 codes in lane order (rows padded with zero codes to a multiple of 32;
    the padded rows' scales and LoRA activations are never used: the output has the original row count)."""
    from nunchaku_rocm_amd.layout import block_activations_f6

    M = p["act"].shape[0]
    Mp = (M + 31) // 32 * 32
    q = dict(p)
    act = torch.zeros(Mp, p["act"].shape[1], dtype=torch.uint8)
    act[:M] = p["act"]
    q["act"] = block_activations_f6(act, unsigned)
    q["asc"] = torch.nn.functional.pad(p["asc"], (0, Mp - M))
    if p.get("la") is not None:
        q["la"] = torch.nn.functional.pad(p["la"], (0, 0, 0, Mp - M))
    return q


@pytest.mark.parametrize("unsigned", [False, True])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,N,K,R,actual_m", [(136, 264, 256, 16, 130), (256, 256, 512, 32, 256), (64, 128, 1024, 48, 64), (128, 512, 256, 0, 100),
                                                   (72, 136, 512, 288, 72), (136, 264, 64, 16, 136), (130, 200, 192, 32, 130), (256, 128, 448, 0, 200)])
def test_scaled_gemm_from_fp6_codes(dev, M, N, K, R, actual_m, unsigned, dtype, main_loop):
    """The same bar with the activations handed over as fp6 codes in lane order (act_blocked = 2; fp8 main loop only)."""
    print(f"case M={M} N={N} K={K} R={R} actual_m={actual_m} unsigned={unsigned} {dtype}", flush=True)
    p = _rand_problem(M, N, K, R, dtype, seed=K + R)
    if main_loop != "all":  # the int8 main loop reads the (M, K/2) matrix only: the operator must refuse
        with pytest.raises(ValueError):
            _gpu_gemm(_as_fp6_codes(p, unsigned), dev, actual_m=actual_m, unsigned=unsigned, dtype=dtype, act_blocked=2)
        return
    out = _gpu_gemm(_as_fp6_codes(p, unsigned), dev, actual_m=actual_m, unsigned=unsigned, dtype=dtype, act_blocked=2)
    ref = O.gemm_w4a4(p["act"], p["wgt"], p["asc"], p["wsc"], p["bias"], p["la"], p["lu"], unsigned)[:actual_m]
    assert O.max_rel_err(out, ref) <= TOL
    ulp = 2**-7 if dtype == torch.bfloat16 else 2**-10
    assert ((out.float() - ref).abs() <= ref.abs() * ulp * 1.01 + 1e-3 * ref.abs().max()).all()


@pytest.mark.parametrize("unsigned", [False, True])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_scale_products_from_fp6_codes_are_exact(dev, dtype, unsigned, main_loop):
    """One group, extreme scales: with fp6 activation codes the signed product has no offset term either, so signed and
    unsigned outputs are the oracle's fp32 product p * (as * ws) rounded once, bit for bit."""
    if main_loop != "all":
        return  # the refusal of the int8 main loop is checked in test_scaled_gemm_from_fp6_codes
    M, N, K = 64, 128, 64
    p = _rand_problem(M, N, K, 0, dtype, seed=5)
    p["bias"] = None
    if dtype == torch.float16:  # weight scales a working copy exists for (its 16-bit offset terms overflow at about 17)
        asc = torch.tensor([2.0**-14, 3 * 2.0**-14, 1023 * 2.0**-14, 2.0**-4, 2.0**-5, 0.0, 2.0**-2, 2.0**-10], dtype=torch.float32)
        wsc = torch.tensor([1.0, 1.5, 2.0, 4.0, 2.5, 16.0, 0.0, 2054.0 / 1024], dtype=torch.float32)
    else:
        asc = torch.tensor([2.0**-60, 1.5 * 2.0**-40, 2.0**-14, 1.0, 2.0**20, 0.0, 255 * 2.0**-30, 2.0**-50], dtype=torch.float32)
        wsc = torch.tensor([1.0, 2.0**30, 2.0**-20, 1.9921875, 2.0**-30, 2.0**40, 0.0, 2.0**-55], dtype=torch.float32)
    p["asc"] = asc.repeat(M // 8).reshape(1, M).to(dtype)
    p["wsc"] = wsc.repeat_interleave(N // 8).reshape(1, N).to(dtype)
    out = _gpu_gemm(_as_fp6_codes(p, unsigned), dev, unsigned=unsigned, dtype=dtype, act_blocked=2)
    ref = O.gemm_w4a4(p["act"], p["wgt"], p["asc"], p["wsc"], act_unsigned=unsigned).to(dtype)
    assert torch.isfinite(ref.float()).all() and (ref != 0).any()
    assert torch.equal(out.view(torch.int16), ref.view(torch.int16))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_scale_products_are_exact_over_the_exponent_range(dev, dtype):
    """as * ws is formed from the 16-bit scales themselves: subnormal fp16 activation scales (|x| < 4e-4 in a group),
    tiny and large bf16 scales and zero scales must give the oracle's fp32 product.  One group: the output is p * as * ws
    with p an exact integer, so a flushed or rounded scale shows as a wrong output.  Unsigned activations: the signed
    fp8 loop adds its offset correction, whose 16-bit pieces are not exact at these magnitudes."""
    M, N, K = 64, 128, 64
    p = _rand_problem(M, N, K, 0, dtype, seed=5)
    p["bias"] = None
    if dtype == torch.float16:  # products from 2^-14 to 2^2: every output is a normal fp16 number or zero
        asc = torch.tensor([2.0**-24, 3 * 2.0**-24, 1023 * 2.0**-24, 2.0**-14, 2.0**-15, 0.0, 2.0**-12, 2.0**-20], dtype=torch.float32)
        wsc = torch.tensor([2.0**10, 1.5 * 2.0**10, 2.0**11, 2.0**12, 1.25 * 2.0**11, 2.0**14, 0.0, 2054.0], dtype=torch.float32)
    else:  # products from 2^-115 to 2^60
        asc = torch.tensor([2.0**-60, 1.5 * 2.0**-40, 2.0**-14, 1.0, 2.0**20, 0.0, 255 * 2.0**-30, 2.0**-50], dtype=torch.float32)
        wsc = torch.tensor([1.0, 2.0**30, 2.0**-20, 1.9921875, 2.0**-30, 2.0**40, 0.0, 2.0**-55], dtype=torch.float32)
    p["asc"] = asc.repeat(M // 8).reshape(1, M).to(dtype)
    p["wsc"] = wsc.repeat_interleave(N // 8).reshape(1, N).to(dtype)
    assert torch.equal(p["asc"].float()[0, :8], asc) and torch.equal(p["wsc"].float()[0, :: N // 8], wsc), "not representable"
    out = _gpu_gemm(p, dev, unsigned=True, dtype=dtype)
    ref = O.gemm_w4a4(p["act"], p["wgt"], p["asc"], p["wsc"], act_unsigned=True).to(dtype)
    assert torch.isfinite(ref.float()).all() and (ref != 0).any()
    assert torch.equal(out.view(torch.int16), ref.view(torch.int16))


def test_strided_row_views(dev):
    """act/wgt/out may be row slices of wider buffers as long as rows stay 16-byte aligned."""
    from nunchaku_rocm_amd import ops

    M, N, K = 64, 128, 256
    p = _rand_problem(M, N, K, 0, torch.bfloat16, seed=77)
    wide_a = torch.zeros(M, K // 2 + 32, dtype=torch.uint8, device=dev)
    wide_a[:, : K // 2] = p["act"].to(dev)
    wide_o = torch.full((M, N + 8), float("nan"), dtype=torch.bfloat16, device=dev)
    ops.svdq_gemm_w4a4_cuda(act=wide_a[:, : K // 2], wgt=p["wgt"].to(dev), out=wide_o[:, :N], ascales=p["asc"].to(dev),
                            wscales=p["wsc"].to(dev), lora_scales=[1.0])  # fmt: skip
    ref = O.gemm_w4a4(p["act"], p["wgt"], p["asc"], p["wsc"])
    assert O.max_rel_err(wide_o[:, :N].cpu(), ref) <= TOL
    assert bool(wide_o[:, N:].isnan().all())


@pytest.mark.parametrize("M", [1024, 4608, 8192])
def test_flux_qkv_shapes_quantizer_then_gemm(dev, M, main_loop):
    """The benchmark linear (K=3072, N=9216, R=32): quantizer -> GEMM on the GPU; oracle on the same seeded inputs.
    The oracle runs on a row sample (rows are independent), all groups of which are also checked bit-exactly."""
    from nunchaku_rocm_amd import ops
    from nunchaku_rocm_amd.ops.gemm import group_acc_i32

    print(f"case M={M}", flush=True)
    K, N = 3072, 9216
    lin = O.make_svdq_linear(K, N, seed=0)
    x = O.make_activations(M, K, seed=1)
    dl = {k: v.to(dev) for k, v in lin.items()}
    qx, asc, la = ops.svdq_quantize_w4a4_act_fuse_lora_cuda(x.to(dev), lora_down=dl["proj_down"], smooth=dl["smooth_factor"])
    out = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
    ops.svdq_gemm_w4a4_cuda(act=qx, wgt=dl["qweight"], out=out, ascales=asc, wscales=dl["wscales"], lora_act_in=la,
                            lora_up=dl["proj_up"], bias=dl["bias"])  # fmt: skip
    torch.cuda.synchronize()
    rows = torch.randperm(M, generator=torch.Generator().manual_seed(M))[:256].sort().values
    rp, rs, rl, _ = O.quantize_act(x[rows], lin["proj_down"], lin["smooth_factor"])
    assert torch.equal(qx[rows].cpu(), rp)
    assert torch.equal(asc[:, rows].cpu().view(torch.int16), rs.view(torch.int16))
    ref = O.gemm_w4a4(rp, lin["qweight"], rs, lin["wscales"], lin["bias"], rl, lin["proj_up"])
    err = O.max_rel_err(out[rows].cpu(), ref)
    print(f"M={M}: max rel err {err:.3e}", flush=True)
    assert err <= TOL
    for g in (0, 17, 47):
        got = group_acc_i32(qx[rows].contiguous(), dl["qweight"], g, fp8_path=main_loop == "all").cpu()
        assert torch.equal(got, O.group_acc_i32(rp, lin["qweight"], False, groups=[g])[0])


def test_full_size_invariants(dev):
    """Properties that hold at any size, checked on the whole QKV problem (M=4608, K=3072, N=9216, R=32) on the GPU:
    doubling the activation scales doubles every output exactly (a power of two commutes with every rounding); a
    permutation of the activation rows permutes the output rows; a permutation of the weight rows permutes the output
    columns -- bit for bit, whatever tile a row or column lands in."""
    from nunchaku_rocm_amd import ops

    M, K, N, R = 4608, 3072, 9216, 32
    g = torch.Generator(device=dev).manual_seed(11)
    act = torch.randint(0, 256, (M, K // 2), generator=g, dtype=torch.uint8, device=dev)
    wgt = torch.randint(0, 256, (N, K // 2), generator=g, dtype=torch.uint8, device=dev)
    asc = (torch.rand(K // 64, M, generator=g, device=dev) * 0.02 + 0.01).to(torch.bfloat16)
    wsc = (torch.rand(K // 64, N, generator=g, device=dev) * 0.02 + 0.01).to(torch.bfloat16)
    bias = torch.randn(N, generator=g, device=dev).to(torch.bfloat16)
    la = torch.randn(M, R, generator=g, device=dev)
    lu = (torch.randn(N, R, generator=g, device=dev) * 0.1).to(torch.bfloat16)

    def run(act, wgt, asc, wsc, bias=None, la=None, lu=None):
        out = torch.empty(act.shape[0], wgt.shape[0], dtype=torch.bfloat16, device=dev)
        ops.svdq_gemm_w4a4_cuda(act=act, wgt=wgt, out=out, ascales=asc, wscales=wsc, bias=bias, lora_act_in=la, lora_up=lu)
        return out

    base = run(act, wgt, asc, wsc)
    assert bool(torch.isfinite(base.float()).all()) and float(base.float().abs().max()) > 0
    assert torch.equal(run(act, wgt, asc * 2, wsc), base * 2)
    assert torch.equal(run(act, wgt, asc, wsc * 0.5), base * 0.5)

    full = run(act, wgt, asc, wsc, bias, la, lu)
    pm = torch.randperm(M, generator=g, device=dev)
    assert torch.equal(run(act[pm].contiguous(), wgt, asc[:, pm].contiguous(), wsc, bias, la[pm].contiguous(), lu), full[pm])
    pn = torch.randperm(N, generator=g, device=dev)
    got = run(act, wgt[pn].contiguous(), asc, wsc[:, pn].contiguous(), bias[pn].contiguous(), la, lu[pn].contiguous())
    assert torch.equal(got, full[:, pn])
    # the low-rank branch and the bias are additive terms of the fp32 accumulator: against the plain output they
    # account for the difference up to the final rounding
    extra = (la.to(torch.bfloat16).float() @ lu.float().t()) + bias.float()
    diff = (full.float() - base.float() - extra).abs()
    assert float(diff.max()) <= 2**-7 * float(full.float().abs().max())


def test_linear_module_matches_dequantised_reference(dev):
    """SVDQW4A4Linear.forward against the SVDQuant formula y = (x / smooth) .q W^T + (x . down) . up^T + bias."""
    from nunchaku_rocm_amd.linear import SVDQW4A4Linear

    K, N, B, S = 512, 384, 2, 75
    lin = O.make_svdq_linear(K, N, seed=5)
    mod = SVDQW4A4Linear(K, N, rank=32, device=dev)
    with torch.no_grad():
        for name in ("qweight", "wscales", "smooth_factor", "proj_down", "proj_up", "bias"):
            getattr(mod, name).copy_(lin[name])
    x = O.make_activations(B * S, K, seed=6).view(B, S, K)
    y = mod(x.to(dev)).cpu()
    assert y.shape == (B, S, N)
    rp, rs, rl, _ = O.quantize_act(x.view(-1, K), lin["proj_down"], lin["smooth_factor"])
    ref = O.gemm_w4a4(rp, lin["qweight"], rs, lin["wscales"], lin["bias"], rl, lin["proj_up"])
    assert O.max_rel_err(y.view(-1, N), ref) <= TOL
    # and against the un-quantized-activation formula within 4-bit quantization noise
    w = O.unpack_int4(lin["qweight"], True).double() * lin["wscales"].double().t().repeat_interleave(64, 1)
    xd = x.view(-1, K).double()
    truth = (xd / lin["smooth_factor"].double()) @ w.t() + (xd @ lin["proj_down"].double()) @ lin["proj_up"].double().t() + lin["bias"].double()
    assert O.cosine(y.view(-1, N), truth) > 0.98


@pytest.mark.parametrize("N,K", [(384, 512), (200, 320)])
def test_release_packed_weight(dev, N, K, main_loop):
    """A module can drop its packed weight and keep only the GEMM's working copy: the forward pass gives the same bits,
    the device holds the packed bytes less, ``state_dict()`` still hands out the packed weight (rebuilt from the copy) and
    ``restore_packed_weight`` puts it back."""
    from nunchaku_rocm_amd.linear import SVDQW4A4Linear
    from nunchaku_rocm_amd.ops import gemm as gemm_mod

    lin = O.make_svdq_linear(K, N, seed=9)
    mod = SVDQW4A4Linear(K, N, rank=32, device=dev)
    with torch.no_grad():
        for name in ("qweight", "wscales", "smooth_factor", "proj_down", "proj_up", "bias"):
            getattr(mod, name).copy_(lin[name])
    x = O.make_activations(150, K, seed=6).view(1, 150, K).to(dev)
    gemm_mod.USE_WEIGHT_PLANES = "all"  # the autouse fixture puts the switch back
    before = mod(x).clone()
    torch.cuda.synchronize()
    held = torch.cuda.memory_allocated(dev)
    assert mod.release_packed_weight()
    torch.cuda.synchronize()
    assert held - torch.cuda.memory_allocated(dev) >= N * K // 2 - 4096
    assert mod.qweight.shape == (N, K // 2) and mod.qweight.untyped_storage().nbytes() <= K // 2
    for switch in ("all", "parameters", "none"):  # the working copy is all there is: the switch no longer matters
        gemm_mod.USE_WEIGHT_PLANES = switch
        assert torch.equal(mod(x).view(torch.int16), before.view(torch.int16))
    sd = mod.state_dict()
    assert torch.equal(sd["qweight"].cpu().view(torch.uint8), lin["qweight"].view(torch.uint8))
    mod.restore_packed_weight()
    assert torch.equal(mod.qweight.cpu().view(torch.uint8), lin["qweight"].view(torch.uint8))
    gemm_mod.USE_WEIGHT_PLANES = main_loop
    ref = mod(x)
    rp, rs, rl, _ = O.quantize_act(x.cpu().view(-1, K), lin["proj_down"], lin["smooth_factor"])
    assert O.max_rel_err(ref.cpu().view(-1, N), O.gemm_w4a4(rp, lin["qweight"], rs, lin["wscales"], lin["bias"], rl, lin["proj_up"])) <= TOL
    # a released module takes a new weight through load_state_dict
    assert mod.release_packed_weight()
    mod.load_state_dict(sd)
    assert torch.equal(mod.qweight.cpu().view(torch.uint8), lin["qweight"].view(torch.uint8))
    assert torch.equal(mod(x).view(torch.int16), before.view(torch.int16)) or main_loop == "none"


def _planes_expected(wgt, wsc, N, K):
    """Host restatement of the pre-split weight layout.  Per (block of 32 rows, stage of two groups) three 1 KB blocks:
    a lane (= parity * 32 + row) holds, per group, 32 six-bit codes sign | magnitude (position p = the nibble of its parity
    of the row's packed byte p of the group; code p in bits 6 p .. 6 p + 5 of 24 little-endian bytes); blocks 0 and 1 = bytes 0-15 of the stage's two groups, block 2 = bytes 16-23 of both.  A group past the end is
    zeros.  Then per (block of rows, stage; one stage of zero padding behind the last) 32 rows of six 16-bit values: for
    each of the stage's two groups the pieces (hi, lo) of -wscale * (8 * sum of the even-k weights - 7 * sum of the odd-k
    weights), then the two weight scales.  Last, a 16-byte status word (0 = usable)."""
    import numpy as np

    nb, G = (N + 31) // 32, K // 64
    nst = (G + 1) // 2
    q = O.unpack_int4(wgt, signed=True).to(torch.int16)  # (N, K) in [-8, 7]
    rows = torch.arange(nb * 32).clamp(max=N - 1)
    qb = q[rows].view(nb, 32, G, 32, 2)  # (nblk, row in block, g, packed byte, even/odd nibble)
    offs = 8 * qb[..., 0].sum(-1) - 7 * qb[..., 1].sum(-1)  # (nblk, row, g)
    code = (qb.abs() | ((qb < 0).to(torch.int16) << 5)).to(torch.uint8)
    code = code.permute(0, 2, 4, 1, 3).reshape(nb, G, 64, 32)  # (nblk, g, lane = parity * 32 + row, position = byte)
    full = torch.zeros(nb, nst * 2, 64, 32, dtype=torch.uint8)
    full[:, :G] = code
    bits = ((full.numpy()[..., None] >> np.arange(6, dtype=np.uint8)) & 1).reshape(nb, nst, 2, 64, 192)
    by = torch.from_numpy(np.packbits(bits, axis=-1, bitorder="little"))  # (nblk, stage, group of the stage, lane, 24)
    planes = torch.zeros(nb, nst, 3, 64, 16, dtype=torch.uint8)
    planes[:, :, 0] = by[:, :, 0, :, :16]
    planes[:, :, 1] = by[:, :, 1, :, :16]
    planes[:, :, 2, :, :8] = by[:, :, 0, :, 16:]
    planes[:, :, 2, :, 8:] = by[:, :, 1, :, 16:]
    ws = wsc.t()[rows].reshape(nb, 32, G)  # (nblk, row, g)
    d = -(ws.float() * offs.float())
    aux = torch.zeros(nb, nst + 1, 32, 6, dtype=wsc.dtype)
    for g in range(G):
        s, gg = divmod(g, 2)
        hi = d[:, :, g].to(wsc.dtype)
        aux[:, s, :, 2 * gg] = hi
        aux[:, s, :, 2 * gg + 1] = (d[:, :, g] - hi.float()).to(wsc.dtype)
        aux[:, s, :, 4 + gg] = ws[:, :, g]
    return planes, aux


@pytest.mark.parametrize("N,K", [(32, 64), (264, 256), (100, 128), (64, 2048), (72, 320)])
def test_weight_planes_layout(dev, N, K):
    from nunchaku_rocm_amd.ops._prep import weight_planes

    g = torch.Generator().manual_seed(N)
    wgt = torch.randint(0, 256, (N, K // 2), generator=g, dtype=torch.uint8)
    wsc = (torch.rand(K // 64, N, generator=g) * 0.02 + 0.005).to(torch.bfloat16)
    got = weight_planes(wgt.to(dev), wsc.to(dev)).cpu()
    planes, aux = _planes_expected(wgt, wsc, N, K)
    assert got.numel() == planes.numel() + aux.numel() * 2 + 16
    assert torch.equal(got[: planes.numel()], planes.view(-1))
    assert torch.equal(got[planes.numel() : -16].view(torch.int16), aux.view(torch.int16).view(-1))
    assert int(got[-16:-12].view(torch.int32)) == 0


@pytest.mark.parametrize("unsigned", [False, True])
@pytest.mark.parametrize("M,N,K,R", [(300, 520, 1152, 32), (129, 136, 320, 16), (2048, 1280, 512, 0)])
def test_fp8_loop_builds_agree_bit_for_bit(dev, M, N, K, R, unsigned):
    """The fp8 main loop is built twice (three workgroups per CU, steps in program order; two per CU, steps software
    pipelined) and the library picks by tile count: both issue the same arithmetic in the same order, so every output bit
    agrees, whichever one a shape gets."""
    from nunchaku_rocm_amd.ops import gemm as gemm_mod

    print(f"case M={M} N={N} K={K} R={R} unsigned={unsigned}", flush=True)
    p = _rand_problem(M, N, K, R, torch.bfloat16, seed=11 + M)
    old = gemm_mod.USE_WEIGHT_PLANES
    try:
        gemm_mod.USE_WEIGHT_PLANES = "all"
        gemm_mod.set_fp8_loop_variant(0)
        three = _gpu_gemm(p, dev, unsigned=unsigned)
        gemm_mod.set_fp8_loop_variant(1)
        two = _gpu_gemm(p, dev, unsigned=unsigned)
    finally:
        gemm_mod.set_fp8_loop_variant(-1)
        gemm_mod.USE_WEIGHT_PLANES = old
    assert torch.equal(three.view(torch.int16), two.view(torch.int16))
    ref = O.gemm_w4a4(p["act"], p["wgt"], p["asc"], p["wsc"], bias=p["bias"], lora_act=p["la"], lora_up=p["lu"], act_unsigned=unsigned)
    assert O.max_rel_err(three.float(), ref) <= TOL


def test_weight_planes_refuse_scales_beyond_fp16(dev):
    """fp16 weight scales so large that -ws * (8 We - 7 Wo) overflows a 16-bit piece: the re-layout raises its status word and
    the operator falls back to the packed weight (int8 main loop) instead of producing NaN."""
    from nunchaku_rocm_amd.ops import gemm as gemm_mod
    from nunchaku_rocm_amd.ops._prep import weight_planes

    p = _rand_problem(64, 128, 256, 0, torch.float16, seed=3)
    p["wsc"] = (p["wsc"].float() * 4000).to(torch.float16)  # about 20 .. 80
    assert weight_planes(p["wgt"].to(dev), p["wsc"].to(dev)) is None
    old = gemm_mod.USE_WEIGHT_PLANES
    try:
        gemm_mod.USE_WEIGHT_PLANES = "all"
        out = _gpu_gemm(p, dev, dtype=torch.float16)
    finally:
        gemm_mod.USE_WEIGHT_PLANES = old
    assert torch.isfinite(out.float()).all()
    ref = O.gemm_w4a4(p["act"], p["wgt"], p["asc"], p["wsc"], bias=p["bias"], lora_act=p["la"], lora_up=p["lu"])
    assert O.max_rel_err(out.float(), ref) <= TOL


@pytest.mark.parametrize("unsigned", [False, True])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,N,K,R", [(136, 264, 256, 16), (256, 512, 1024, 32), (64, 72, 128, 0), (300, 3072, 3072, 32),
                                     (100, 136, 64, 16), (257, 264, 320, 0),  # K / 64 odd
                                     # long K: the offset of signed activations is taken out every four stages (512 of K); these
                                     # end on 1, 0, 0, 3 and 2 stages of a last partial set
                                     (100, 136, 4160, 16), (64, 264, 5120, 0), (64, 128, 6144, 32), (96, 128, 896, 0), (40, 136, 768, 16)])
def test_presplit_weights_against_packed(dev, M, N, K, R, unsigned, dtype):
    """The two main loops (int8 MFMA on packed weights, fp8 MFMA on pre-split weights) compute the same integer group sums
    and differ only in the order of fp32 roundings: outputs agree to one 16-bit ulp of the largest value."""
    print(f"case M={M} N={N} K={K} R={R} unsigned={unsigned} {dtype}", flush=True)
    p = _rand_problem(M, N, K, R, dtype, seed=7 + M)
    from nunchaku_rocm_amd.ops import gemm as gemm_mod

    old = gemm_mod.USE_WEIGHT_PLANES
    try:
        gemm_mod.USE_WEIGHT_PLANES = "none"
        packed = _gpu_gemm(p, dev, unsigned=unsigned, dtype=dtype)
        gemm_mod.USE_WEIGHT_PLANES = "all"
        split = _gpu_gemm(p, dev, unsigned=unsigned, dtype=dtype)
    finally:
        gemm_mod.USE_WEIGHT_PLANES = old
    assert O.max_rel_err(split.float(), packed.float()) <= (2.0**-7 if dtype == torch.bfloat16 else 2.0**-10)
    ref = O.gemm_w4a4(p["act"], p["wgt"], p["asc"], p["wsc"], bias=p["bias"], lora_act=p["la"], lora_up=p["lu"], act_unsigned=unsigned)
    assert O.max_rel_err(split.float(), ref) <= TOL
