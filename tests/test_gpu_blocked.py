"""Quantized activations in the GEMM's own order (``out_blocked`` / ``act_blocked`` / ``qout_blocked``): the same codes
as the (M, K/2) matrix, bit for bit, moved; the same GEMM outputs, bit for bit; and modules / composite operators that
compute the same bits whichever way they pass activations along."""

import pytest
import torch

from oracle import svdq_oracle as O

pytestmark = pytest.mark.gpu


def _module(dev, K, N, seed, dtype=torch.bfloat16, act_unsigned=False):
    from nunchaku_rocm_amd.linear import SVDQW4A4Linear

    lin = O.make_svdq_linear(K, N, seed=seed, dtype=dtype)
    mod = SVDQW4A4Linear(K, N, rank=32, act_unsigned=act_unsigned, torch_dtype=dtype, device=dev)
    with torch.no_grad():
        for name in ("qweight", "wscales", "smooth_factor", "proj_down", "proj_up", "bias"):
            getattr(mod, name).copy_(lin[name])
    return mod


def test_layout_helpers_invert_each_other():
    from nunchaku_rocm_amd.layout import block_activations, unblock_activations

    a = torch.randint(0, 256, (96, 160), dtype=torch.uint8, generator=torch.Generator().manual_seed(0))
    b = block_activations(a)
    assert b.shape == a.shape and not torch.equal(a, b)
    assert torch.equal(unblock_activations(b), a)
    # lane 32 h + r of (row block rb, group g) = bytes 16 h .. of row 32 rb + r
    rb, g, h, r = 2, 3, 1, 7
    piece = b.reshape(-1)[((rb * 5 + g) * 64 + 32 * h + r) * 16 :][:16]
    assert torch.equal(piece, a[32 * rb + r, 32 * g + 16 * h :][:16])


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,K,R,norm", [(300, 256, 16, False), (4608, 3072, 32, False), (272, 320, 32, True), (100, 64, 0, False)])
def test_quantizer_writes_the_same_codes_elsewhere(dev, M, K, R, norm, dtype):
    from nunchaku_rocm_amd import ops
    from nunchaku_rocm_amd.layout import unblock_activations

    print(f"case M={M} K={K} R={R} norm={norm} {dtype}", flush=True)
    g = torch.Generator().manual_seed(M + K)
    x = torch.randn(M, K, generator=g).to(dtype).to(dev)
    smooth = (torch.rand(K, generator=g) + 0.5).to(dtype).to(dev)
    ld = (torch.randn(K, R, generator=g) * 0.1).to(dtype).to(dev) if R else None
    nm = ((torch.randn(K, generator=g) * 0.1 + 1).to(dtype).to(dev), (torch.randn(K, generator=g) * 0.1).to(dtype).to(dev)) if norm else None
    nat = ops.svdq_quantize_w4a4_act_fuse_lora_cuda(x, lora_down=ld, smooth=smooth, norm=nm)
    out_b = torch.full_like(nat[0], 0xEE)
    blk = ops.svdq_quantize_w4a4_act_fuse_lora_cuda(x, output=out_b, lora_down=ld, smooth=smooth, norm=nm, out_blocked=True)
    torch.cuda.synchronize()
    assert torch.equal(unblock_activations(blk[0].cpu())[:M], nat[0].cpu()[:M])
    assert (unblock_activations(blk[0].cpu())[M:] == 0xEE).all()  # pad rows untouched
    assert torch.equal(blk[1].cpu()[:, :M].view(torch.int16), nat[1].cpu()[:, :M].view(torch.int16))
    if R:
        assert torch.equal(blk[2].cpu()[:M], nat[2].cpu()[:M])


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,K,R,norm,unsigned", [(300, 256, 16, False, False), (4608, 3072, 32, False, False), (272, 320, 32, True, False),
                                                 (100, 64, 0, False, False), (1000, 1024, 32, False, True), (4608, 3072, 32, True, False)])
def test_quantizer_writes_fp6_codes(dev, M, K, R, norm, unsigned, dtype):
    """out_blocked=2: the same integers as the (M, K/2) matrix holds, as sign | magnitude codes in lane order; scales and
    LoRA-down product unchanged; rows past M untouched."""
    from nunchaku_rocm_amd import ops
    from nunchaku_rocm_amd.layout import unblock_activations_f6

    print(f"case M={M} K={K} R={R} norm={norm} unsigned={unsigned} {dtype}", flush=True)
    g = torch.Generator().manual_seed(M + K)
    x = torch.randn(M, K, generator=g).to(dtype).to(dev)
    x[3, :64] = 0  # a group of zeros: scale 0, codes 0
    smooth = (torch.rand(K, generator=g) + 0.5).to(dtype).to(dev)
    ld = (torch.randn(K, R, generator=g) * 0.1).to(dtype).to(dev) if R else None
    nm = ((torch.randn(K, generator=g) * 0.1 + 1).to(dtype).to(dev), (torch.randn(K, generator=g) * 0.1).to(dtype).to(dev)) if norm else None
    kw = dict(lora_down=ld, smooth=smooth, norm=nm)
    if unsigned:
        kw.update(shift_value=0.171875, unsigned=True, fuse_gelu=True)
        fn = ops.quantize_w4a4_act_fuse_lora
        nat = fn(x, **kw)
        rows = (M + 31) // 32 * 32
    else:
        fn = ops.svdq_quantize_w4a4_act_fuse_lora_cuda
        nat = fn(x, **kw)
        rows = nat[0].shape[0]
    out_b = torch.full((rows, K * 3 // 4), 0xEE, dtype=torch.uint8, device=dev)
    blk = fn(x, output=out_b, out_blocked=2, **kw)
    torch.cuda.synchronize()
    dec = unblock_activations_f6(blk[0].cpu(), unsigned)
    assert torch.equal(dec[:M], nat[0].cpu()[:M])
    # rows past M of a 32-row block that has rows: untouched bytes decode to whatever 0xEE means; whole untouched blocks stay 0xEE
    full = (M + 31) // 32 * 32
    assert (blk[0].cpu()[full:] == 0xEE).all()
    assert torch.equal(blk[1].cpu()[:, :M].view(torch.int16), nat[1].cpu()[:, :M].view(torch.int16))
    if R:
        assert torch.equal(blk[2].cpu()[:M], nat[2].cpu()[:M])


def test_scale_layout_helpers_invert_each_other():
    from nunchaku_rocm_amd.layout import block_scales, unblock_scales

    a = torch.arange(16 * 96, dtype=torch.float32).reshape(16, 96).to(torch.bfloat16)
    b = block_scales(a)
    assert b.shape == a.shape and torch.equal(unblock_scales(b), a)
    m, g = 70, 11  # element ((m / 32) * (G / 8) + g / 8) * 256 + (m % 32) * 8 + g % 8
    assert b.reshape(-1)[((m // 32) * 2 + g // 8) * 256 + (m % 32) * 8 + g % 8] == a[g, m]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("M,K,N,R,norm", [(300, 512, 264, 16, False), (4608, 3072, 384, 32, False), (1000, 1536, 256, 32, True), (96, 1024, 128, 0, False)])
def test_scales_in_the_gemms_order(dev, M, K, N, R, norm, dtype):
    """out_blocked = act_blocked = 3: fp6 codes as with 2, and the activation scales where the GEMM's lanes read eight
    groups with one load.  The quantizer writes the same scale bits elsewhere; the GEMM computes the same output bits
    as with act_blocked = 2; K that is not a multiple of 512 is refused."""
    from nunchaku_rocm_amd import ops
    from nunchaku_rocm_amd.layout import block_scales, unblock_activations_f6, unblock_scales
    from nunchaku_rocm_amd.ops import gemm as gemm_mod

    print(f"case M={M} K={K} N={N} R={R} norm={norm} {dtype}", flush=True)
    lin = {k: v.to(dev) for k, v in O.make_svdq_linear(K, N, R=max(R, 16), seed=K + N, dtype=dtype).items()}
    g = torch.Generator().manual_seed(M + K)
    x = torch.randn(M, K, generator=g).to(dtype).to(dev)
    ld = lin["proj_down"][:, :R].contiguous() if R else None
    lu = lin["proj_up"][:, :R].contiguous() if R else None
    nm = ((torch.randn(K, generator=g) * 0.1 + 1).to(dtype).to(dev), (torch.randn(K, generator=g) * 0.1).to(dtype).to(dev)) if norm else None
    q2, s2, la2 = ops.svdq_quantize_w4a4_act_fuse_lora_cuda(x, lora_down=ld, smooth=lin["smooth_factor"], norm=nm, out_blocked=2)
    s3 = torch.full_like(s2, 7.0)
    q3, s3, la3 = ops.svdq_quantize_w4a4_act_fuse_lora_cuda(x, oscales=s3, lora_down=ld, smooth=lin["smooth_factor"], norm=nm, out_blocked=3)
    torch.cuda.synchronize()
    full = (M + 31) // 32 * 32
    assert torch.equal(unblock_activations_f6(q2.cpu())[:M], unblock_activations_f6(q3.cpu())[:M])
    assert torch.equal(unblock_scales(s3.cpu())[:, :M].view(torch.int16), s2.cpu()[:, :M].view(torch.int16))
    assert (unblock_scales(s3.cpu())[:, full:] == 7.0).all()  # rows of untouched 32-row blocks keep what the buffer held
    old = gemm_mod.USE_WEIGHT_PLANES
    gemm_mod.USE_WEIGHT_PLANES = "all"
    try:
        outs = []
        for mode, q, s, la in ((2, q2, s2, la2), (3, q3, s3, la3), (3, q2, block_scales(s2), la2)):
            out = torch.full((M, N), float("nan"), dtype=dtype, device=dev)
            ops.svdq_gemm_w4a4_cuda(act=q, wgt=lin["qweight"], out=out, ascales=s, wscales=lin["wscales"], lora_act_in=la if R else None,
                                    lora_up=lu, bias=lin["bias"], act_blocked=mode)  # fmt: skip
            outs.append(out)
        torch.cuda.synchronize()
        assert torch.equal(outs[0].view(torch.int16), outs[1].view(torch.int16))
        assert torch.equal(outs[0].view(torch.int16), outs[2].view(torch.int16))
    finally:
        gemm_mod.USE_WEIGHT_PLANES = old


def test_scales_in_the_gemms_order_need_k_of_512(dev):
    from nunchaku_rocm_amd import ops
    from nunchaku_rocm_amd.ops import gemm as gemm_mod

    M, K, N = 64, 320, 128
    lin = {k: v.to(dev) for k, v in O.make_svdq_linear(K, N, seed=1).items()}
    x = torch.randn(M, K, generator=torch.Generator().manual_seed(2)).to(torch.bfloat16).to(dev)
    with pytest.raises(ValueError):
        ops.svdq_quantize_w4a4_act_fuse_lora_cuda(x, lora_down=lin["proj_down"], smooth=lin["smooth_factor"], out_blocked=3)
    q, s, la = ops.svdq_quantize_w4a4_act_fuse_lora_cuda(x, lora_down=lin["proj_down"], smooth=lin["smooth_factor"], out_blocked=2)
    old = gemm_mod.USE_WEIGHT_PLANES
    gemm_mod.USE_WEIGHT_PLANES = "all"
    try:
        with pytest.raises(ValueError):
            ops.svdq_gemm_w4a4_cuda(act=q, wgt=lin["qweight"], out=torch.empty(M, N, dtype=torch.bfloat16, device=dev), ascales=s,
                                    wscales=lin["wscales"], act_blocked=3)  # fmt: skip
    finally:
        gemm_mod.USE_WEIGHT_PLANES = old


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_quantizer_then_gemm_through_fp6_codes(dev, dtype):
    """The pair as the modules run it: quantizer (out_blocked=2) -> GEMM (act_blocked=2) against the pair through the
    (M, K/2) matrix, at the oracle's bar for the GEMM output."""
    from nunchaku_rocm_amd import ops

    M, K, N, R = 1000, 1024, 768, 32
    lin = {k: v.to(dev) for k, v in O.make_svdq_linear(K, N, seed=5, dtype=dtype).items()}
    x = torch.randn(M, K, generator=torch.Generator().manual_seed(9)).to(dtype).to(dev)
    from nunchaku_rocm_amd.ops import gemm as gemm_mod

    outs = []
    old = gemm_mod.USE_WEIGHT_PLANES
    gemm_mod.USE_WEIGHT_PLANES = "all"
    try:
        for mode in (0, 2):
            q, s, la = ops.svdq_quantize_w4a4_act_fuse_lora_cuda(x, lora_down=lin["proj_down"], smooth=lin["smooth_factor"], out_blocked=mode)
            out = torch.empty(M, N, dtype=dtype, device=dev)
            ops.svdq_gemm_w4a4_cuda(act=q, wgt=lin["qweight"], out=out, ascales=s, wscales=lin["wscales"], lora_act_in=la,
                                    lora_up=lin["proj_up"], bias=lin["bias"], act_blocked=mode)
            outs.append(out.float())
        torch.cuda.synchronize()
    finally:
        gemm_mod.USE_WEIGHT_PLANES = old
    err = (outs[0] - outs[1]).abs().max().item() / outs[0].abs().max().item()
    assert err < (4e-3 if dtype == torch.bfloat16 else 1e-3), err


@pytest.mark.parametrize("unsigned", [False, True])
@pytest.mark.parametrize("M,N,K,R", [(256, 264, 256, 16), (96, 128, 320, 0), (4608, 3072, 3072, 32)])
def test_gemm_reads_either_order(dev, M, N, K, R, unsigned):
    from nunchaku_rocm_amd import ops
    from nunchaku_rocm_amd.layout import block_activations
    from nunchaku_rocm_amd.ops import gemm as gemm_mod

    print(f"case M={M} N={N} K={K} R={R} unsigned={unsigned}", flush=True)
    dtype = torch.bfloat16
    g = torch.Generator().manual_seed(M + N)
    act = torch.randint(0, 256, (M, K // 2), generator=g, dtype=torch.uint8)
    t = dict(wgt=torch.randint(0, 256, (N, K // 2), generator=g, dtype=torch.uint8),
             ascales=(torch.rand(K // 64, M, generator=g) * 0.02 + 0.01).to(dtype),
             wscales=(torch.rand(K // 64, N, generator=g) * 0.02 + 0.01).to(dtype), bias=torch.randn(N, generator=g).to(dtype))  # fmt: skip
    if R:
        t.update(lora_act_in=torch.randn(M, R, generator=g), lora_up=(torch.randn(N, R, generator=g) * 0.1).to(dtype))
    t = {k: v.to(dev) for k, v in t.items()}
    old = gemm_mod.USE_WEIGHT_PLANES
    gemm_mod.USE_WEIGHT_PLANES = "all"
    try:
        nat = torch.empty(M - 5, N, dtype=dtype, device=dev)
        ops.svdq_gemm_w4a4_cuda(act=act.to(dev), out=nat, act_unsigned=unsigned, **t)
        blk = torch.empty(M - 5, N, dtype=dtype, device=dev)
        ops.svdq_gemm_w4a4_cuda(act=block_activations(act).to(dev), out=blk, act_unsigned=unsigned, act_blocked=True, **t)
        torch.cuda.synchronize()
        assert torch.equal(nat.view(torch.int16), blk.view(torch.int16))
        gemm_mod.USE_WEIGHT_PLANES = "none"  # the int8 main loop reads the matrix only
        with pytest.raises(ValueError):
            ops.svdq_gemm_w4a4_cuda(act=block_activations(act).to(dev), out=blk, act_unsigned=unsigned, act_blocked=True, **t)
    finally:
        gemm_mod.USE_WEIGHT_PLANES = old


def test_fp6_layout_helpers_invert_each_other():
    from nunchaku_rocm_amd.layout import block_activations_f6, unblock_activations_f6

    a = torch.randint(0, 256, (96, 160), dtype=torch.uint8, generator=torch.Generator().manual_seed(0))
    for unsigned in (False, True):
        b = block_activations_f6(a, unsigned)
        assert b.shape == (96, 240)
        assert torch.equal(unblock_activations_f6(b, unsigned), a)
    # code p of lane 32 h + r of (row block rb, group g) = value k = 2 p + h of row 32 rb + r's group, sign | magnitude
    b = block_activations_f6(a, False).reshape(-1)
    rb, g, h, r, p = 1, 2, 1, 5, 21  # bit 126: straddles the lane's first 16 bytes and its last 8
    base = (rb * 5 + g) * 1536
    lane = 32 * h + r
    vec = torch.cat([b[base + 16 * lane :][:16], b[base + 1024 + 8 * lane :][:8]]).tolist()
    code = (int.from_bytes(bytes(vec), "little") >> (6 * p)) & 63
    byte = int(a[32 * rb + r, 32 * g + p])  # k = 2 p + 1: the high nibble of byte p of the group
    v = ((byte >> 4) ^ 8) - 8
    assert code == (32 - v if v < 0 else v)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("unsigned", [False, True])
@pytest.mark.parametrize("M,N,K,R", [(256, 264, 256, 16), (96, 128, 320, 0), (4608, 3072, 3072, 32), (1024, 640, 1216, 32)])
def test_gemm_takes_fp6_codes(dev, M, N, K, R, unsigned, dtype):
    """act_blocked=2: the activations as fp6 codes in lane order.  The group sums are the same integers; unsigned
    activations give the same bits as the nibble matrix, signed ones differ by what the nibble path's 16-bit offset
    terms round (so they are compared with the oracle's bar instead, and bit for bit at unit scales)."""
    from nunchaku_rocm_amd import ops
    from nunchaku_rocm_amd.layout import block_activations_f6
    from nunchaku_rocm_amd.ops import gemm as gemm_mod

    print(f"case M={M} N={N} K={K} R={R} unsigned={unsigned} {dtype}", flush=True)
    g = torch.Generator().manual_seed(M + N + K)
    act = torch.randint(0, 256, (M, K // 2), generator=g, dtype=torch.uint8)
    t = dict(wgt=torch.randint(0, 256, (N, K // 2), generator=g, dtype=torch.uint8),
             ascales=(torch.rand(K // 64, M, generator=g) * 0.02 + 0.01).to(dtype),
             wscales=(torch.rand(K // 64, N, generator=g) * 0.02 + 0.01).to(dtype), bias=torch.randn(N, generator=g).to(dtype))  # fmt: skip
    if R:
        t.update(lora_act_in=torch.randn(M, R, generator=g), lora_up=(torch.randn(N, R, generator=g) * 0.1).to(dtype))
    t = {k: v.to(dev) for k, v in t.items()}
    codes = block_activations_f6(act, unsigned).to(dev)
    old = gemm_mod.USE_WEIGHT_PLANES
    gemm_mod.USE_WEIGHT_PLANES = "all"
    try:
        nat = torch.empty(M - 5, N, dtype=dtype, device=dev)
        ops.svdq_gemm_w4a4_cuda(act=act.to(dev), out=nat, act_unsigned=unsigned, **t)
        f6 = torch.full((M - 5, N), float("nan"), dtype=dtype, device=dev)
        ops.svdq_gemm_w4a4_cuda(act=codes, out=f6, act_unsigned=unsigned, act_blocked=2, **t)
        torch.cuda.synchronize()
        if unsigned:
            assert torch.equal(nat.view(torch.int16), f6.view(torch.int16))
        else:
            ref = nat.float()
            err = (f6.float() - ref).abs().max().item() / ref.abs().max().item()
            assert err < (4e-3 if dtype == torch.bfloat16 else 1e-3), err
        # unit scales, no LoRA, no bias: integer results below 2^24, exact either way
        ones = {k: torch.ones_like(t[k]) for k in ("ascales", "wscales")}
        small = torch.randint(0, 256, (M, K // 2), generator=g, dtype=torch.uint8) & 0x11  # values 0 / 1: sums stay exact in T
        o1 = torch.empty(M, N, dtype=dtype, device=dev)
        o2 = torch.empty(M, N, dtype=dtype, device=dev)
        ops.svdq_gemm_w4a4_cuda(act=small.to(dev), wgt=t["wgt"], out=o1, act_unsigned=unsigned, **ones)
        ops.svdq_gemm_w4a4_cuda(act=block_activations_f6(small, unsigned).to(dev), wgt=t["wgt"], out=o2, act_unsigned=unsigned, act_blocked=2, **ones)
        torch.cuda.synchronize()
        assert torch.equal(o1.view(torch.int16), o2.view(torch.int16))
        gemm_mod.USE_WEIGHT_PLANES = "none"  # the int8 main loop reads the matrix only
        with pytest.raises(ValueError):
            ops.svdq_gemm_w4a4_cuda(act=codes, out=f6, act_unsigned=unsigned, act_blocked=2, **t)
    finally:
        gemm_mod.USE_WEIGHT_PLANES = old


@pytest.mark.parametrize("swiglu", [False, True])
def test_requantizing_epilogues_write_either_order(dev, swiglu):
    from nunchaku_rocm_amd import ops
    from nunchaku_rocm_amd.layout import unblock_activations
    from nunchaku_rocm_amd.ops import gemm as gemm_mod

    M, N, K, R2, dtype = 288, 1024, 256, 32, torch.bfloat16  # 1024 / 512 requantized columns: eight groups of scales
    NQ = N // 2 if swiglu else N
    g = torch.Generator().manual_seed(11)
    t = dict(act=torch.randint(0, 256, (M, K // 2), generator=g, dtype=torch.uint8), wgt=torch.randint(0, 256, (N, K // 2), generator=g, dtype=torch.uint8),
             ascales=(torch.rand(K // 64, M, generator=g) * 0.2 + 0.05).to(dtype), wscales=(torch.rand(K // 64, N, generator=g) * 0.02 + 0.01).to(dtype),
             bias=torch.randn(N, generator=g).to(dtype), smooth_factor=(torch.rand(NQ, generator=g) + 0.5).to(dtype),
             lora_down=(torch.randn(NQ, R2, generator=g) * 0.1).to(dtype))  # fmt: skip
    t = {k: v.to(dev) for k, v in t.items()}
    from nunchaku_rocm_amd.layout import unblock_activations_f6

    from nunchaku_rocm_amd.layout import unblock_scales

    res = []
    for blocked in (False, True, 2, 3):
        qout = torch.full((M, NQ * 3 // 4 if blocked >= 2 else NQ // 2), 0xEE, dtype=torch.uint8, device=dev)
        osc = torch.zeros(NQ // 64, M, dtype=dtype, device=dev)
        lao = torch.zeros(M, R2, dtype=torch.float32, device=dev)
        ops.svdq_gemm_w4a4_cuda(qout=qout, oscales=osc, lora_act_out=lao, fuse_swiglu=swiglu, qout_blocked=blocked, **t)
        torch.cuda.synchronize()
        # the GELU epilogue's codes are unsigned, the SwiGLU epilogue's signed
        codes = unblock_activations_f6(qout.cpu(), not swiglu) if blocked >= 2 else unblock_activations(qout.cpu()) if blocked else qout.cpu()
        res.append((codes, (unblock_scales(osc.cpu()) if blocked == 3 else osc.cpu()).view(torch.int16), lao.cpu()))
    for other in res[1:]:
        for a, b in zip(res[0], other):
            assert torch.equal(a, b)
    assert (res[0][0] != 0xEE).any()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_modules_compute_the_same_bits_either_way(dev, dtype):
    """SVDQW4A4Linear.forward, fused_gelu_mlp, fused_qkv_norm_rottary and fused_swiglu_mlp with the hand-over switched
    off, as the matrix's bytes in lane order (the same bits) and as the default, fp6 codes from the quantizer (the same
    group sums without the nibble path's 16-bit offset terms: compared at the GEMM's bar); row counts that are and are
    not multiples of 256."""
    from nunchaku_rocm_amd import ops
    from nunchaku_rocm_amd.ops import gemm as gemm_mod

    C, H4 = 256, 1024
    fc1, fc2 = _module(dev, C, H4, 1, dtype), _module(dev, H4, C, 2, dtype, act_unsigned=True)
    qkv = _module(dev, C, 3 * 128, 3, dtype)
    g1, g2 = _module(dev, C, 2 * 512, 4, dtype), _module(dev, 512, C, 5, dtype)
    ops.interleave_swiglu_linear_(g1)
    nq = torch.nn.RMSNorm(128, eps=1e-6, device=dev, dtype=dtype)
    nk = torch.nn.RMSNorm(128, eps=1e-6, device=dev, dtype=dtype)
    for S in (512, 300):
        x = torch.randn(1, S, C, generator=torch.Generator().manual_seed(S)).to(dtype).to(dev)
        rot = O.flux_rotary(O.flux_ids(S - 64, 8, 8)).to(dev)
        outs = []
        for flag in (True, 1, False):
            gemm_mod.USE_BLOCKED_ACTIVATIONS = flag
            try:
                assert fc1.takes_blocked(S) == (2 if flag is True else int(flag))  # K = 256
                assert fc2.takes_blocked(S) == (3 if flag is True else int(flag))  # K = 1024: scales in the GEMM's order too
                outs.append([fc1(x).clone(), ops.fused_gelu_mlp(x, fc1, fc2).clone(), ops.fused_qkv_norm_rottary(x, qkv, nq, nk, rot).clone(),
                             ops.fused_swiglu_mlp(x, g1, g2).clone()])  # fmt: skip
            finally:
                gemm_mod.USE_BLOCKED_ACTIVATIONS = True
        torch.cuda.synchronize()
        for f6, lanes, matrix in zip(*outs):
            assert torch.equal(lanes.view(torch.int16), matrix.view(torch.int16))
            err = (f6.float() - matrix.float()).abs().max().item() / matrix.float().abs().max().item()
            assert err < (1.5e-2 if dtype == torch.bfloat16 else 4e-3), err
