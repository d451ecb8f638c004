"""Seeded sweeps over odd shapes (ragged M, N not a multiple of the tile, odd group counts, ranks 0..64, rows past
``actual_m``) of the quantizer, the GEMM and attention against the CPU oracle: the bars of the fixed-shape tests, on shapes
nobody picked by hand."""

import random

import pytest
import torch

from oracle import svdq_oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True, params=["none", "all"], ids=["int8-loop", "fp8-loop"])
def main_loop(request):
    """Every test runs through both GEMM main loops: packed weights (int8 MFMA) and pre-split weights (fp8 MFMA)."""
    from nunchaku_rocm_amd.ops import gemm as G

    old, G.USE_WEIGHT_PLANES = G.USE_WEIGHT_PLANES, request.param
    yield request.param
    G.USE_WEIGHT_PLANES = old


def test_gemm_random_shapes(dev):
    from nunchaku_rocm_amd import ops

    rnd = random.Random(1234)
    for case in range(40):
        M = rnd.choice([1, 7, 31, 32, 33, 100, 127, 128, 129, 200, 257, 300])
        N = 8 * rnd.randint(1, 50)
        K = 64 * rnd.randint(1, 9)
        R = rnd.choice([0, 16, 32, 48, 64])
        am = rnd.randint(1, M)
        unsigned = rnd.random() < 0.5
        dtype = rnd.choice([torch.bfloat16, torch.float16])
        bias = rnd.random() < 0.7
        print(f"case {case}: M={M} N={N} K={K} R={R} actual_m={am} unsigned={unsigned} {dtype} bias={bias}", flush=True)
        g = torch.Generator().manual_seed(case)
        act = torch.randint(0, 256, (M, K // 2), generator=g, dtype=torch.uint8)
        wgt = torch.randint(0, 256, (N, K // 2), generator=g, dtype=torch.uint8)
        asc = (torch.rand(K // 64, M, generator=g) * 0.02 + 0.01).to(dtype)
        wsc = (torch.rand(K // 64, N, generator=g) * 0.02 + 0.01).to(dtype)
        b = torch.randn(N, generator=g).to(dtype) if bias else None
        la = torch.randn(M, R, generator=g) if R else None
        lu = (torch.randn(N, R, generator=g) * 0.1).to(dtype) if R else None
        d = lambda t: None if t is None else t.to(dev)  # noqa: E731
        buf = torch.full((am + 3, N), float("nan"), dtype=dtype, device=dev)
        ops.svdq_gemm_w4a4_cuda(act=d(act), wgt=d(wgt), out=buf[:am], ascales=d(asc), wscales=d(wsc), bias=d(b),
                                lora_act_in=d(la), lora_up=d(lu), act_unsigned=unsigned)  # fmt: skip
        torch.cuda.synchronize()
        assert bool(buf[am:].isnan().all()), "rows past actual_m were written"
        ref = O.gemm_w4a4(act, wgt, asc, wsc, b, la, lu, unsigned)[:am]
        assert O.max_rel_err(buf[:am].cpu(), ref) <= 1e-2


def test_hand_over_random_shapes(dev, main_loop):
    """Quantizer -> GEMM as the modules chain them, on random shapes and every hand-over the shape allows (the matrix,
    its bytes in lane order, fp6 codes, fp6 codes with the scales in the GEMM's order): codes and scales decoded from
    the quantizer's output bit-equal to the oracle's, GEMM output at the oracle's bar."""
    from nunchaku_rocm_amd import ops
    from nunchaku_rocm_amd.layout import unblock_activations, unblock_activations_f6, unblock_scales

    if main_loop != "all":
        return  # the int8 main loop reads the matrix only (its refusal of the other forms: test_gpu_blocked.py)
    rnd = random.Random(777)
    for case in range(24):
        M = rnd.choice([1, 31, 32, 33, 100, 257, 300, 512, 1000])
        K = 64 * rnd.choice([1, 2, 3, 5, 8, 8, 16, 16, 24])
        N = 8 * rnd.randint(1, 48)
        R = rnd.choice([0, 16, 32, 48])
        dtype = rnd.choice([torch.bfloat16, torch.float16])
        mode = rnd.choice([0, 1, 2, 3] if K % 512 == 0 else [0, 1, 2])
        print(f"case {case}: M={M} K={K} N={N} R={R} mode={mode} {dtype}", flush=True)
        lin = O.make_svdq_linear(K, N, R=max(R, 16), seed=case, dtype=dtype)
        x = O.make_activations(M, K, seed=200 + case, dtype=dtype)
        ld = lin["proj_down"][:, :R].contiguous() if R else None
        lu = lin["proj_up"][:, :R].contiguous() if R else None
        d = lambda t: None if t is None else t.to(dev)  # noqa: E731
        q, s, la = ops.svdq_quantize_w4a4_act_fuse_lora_cuda(x.to(dev), lora_down=d(ld), smooth=lin["smooth_factor"].to(dev), out_blocked=mode)
        out = torch.full((M + 2, N), float("nan"), dtype=dtype, device=dev)
        ops.svdq_gemm_w4a4_cuda(act=q, wgt=lin["qweight"].to(dev), out=out[:M], ascales=s, wscales=lin["wscales"].to(dev),
                                lora_act_in=la if R else None, lora_up=d(lu), bias=lin["bias"].to(dev), act_blocked=mode)  # fmt: skip
        torch.cuda.synchronize()
        rp, rs, rl, _ = O.quantize_act(x, ld, lin["smooth_factor"])
        codes = unblock_activations_f6(q.cpu()) if mode >= 2 else unblock_activations(q.cpu()) if mode else q.cpu()
        assert torch.equal(codes[:M], rp), "codes"
        scales = unblock_scales(s.cpu()) if mode == 3 else s.cpu()
        assert torch.equal(scales[:, :M].view(torch.int16), rs.view(torch.int16)), "scales"
        assert bool(out[M:].isnan().all()), "rows past actual_m were written"
        ref = O.gemm_w4a4(rp, lin["qweight"], rs, lin["wscales"], lin["bias"], rl if R else None, lu)
        assert O.max_rel_err(out[:M].cpu(), ref) <= 1e-2


def test_quantizer_random_shapes(dev):
    from nunchaku_rocm_amd.ops.quantize import quantize_w4a4_act_fuse_lora

    rnd = random.Random(4321)
    for case in range(30):
        M = rnd.choice([1, 5, 15, 16, 17, 63, 64, 65, 130, 255, 300])
        K = 64 * rnd.randint(1, 20)
        R = rnd.choice([0, 16, 32, 48, 144])
        smooth = rnd.random() < 0.7
        unsigned = rnd.random() < 0.3
        dtype = rnd.choice([torch.bfloat16, torch.float16])
        print(f"case {case}: M={M} K={K} R={R} smooth={smooth} unsigned={unsigned} {dtype}", flush=True)
        lin = O.make_svdq_linear(K, 64, R=max(R, 16), seed=case, dtype=dtype)
        x = O.make_activations(M, K, seed=100 + case, dtype=dtype)
        ld = lin["proj_down"][:, :R].contiguous() if R else None
        sm = lin["smooth_factor"] if smooth else None
        shift = 0.171875 if unsigned else 0.0
        out, osc, la = quantize_w4a4_act_fuse_lora(x.to(dev), lora_down=ld.to(dev) if R else None,
                                                   smooth=sm.to(dev) if smooth else None, shift_value=shift, unsigned=unsigned)  # fmt: skip
        torch.cuda.synchronize()
        rp, rs, rl, _ = O.quantize_act(x, ld, sm, unsigned=unsigned, shift=shift)
        assert torch.equal(out.cpu(), rp), "codes"
        assert torch.equal(osc.cpu().view(torch.int16), rs.view(torch.int16)), "scales"
        if R:
            assert (la.cpu() - rl).abs().max() <= 1e-3 * rl.abs().max() + 1e-6


def test_attention_random_shapes(dev):
    from nunchaku_rocm_amd import ops

    rnd = random.Random(99)
    for case in range(24):
        B, H = rnd.randint(1, 2), rnd.randint(1, 3)
        D = rnd.choice([128, 64])
        Tq = rnd.choice([1, 3, 31, 64, 65, 127, 128, 129, 200, 333])
        Tkv = rnd.choice([1, 2, 15, 16, 17, 63, 64, 65, 100, 128, 191, 400])
        dtype = rnd.choice([torch.bfloat16, torch.float16])
        print(f"case {case}: B={B} H={H} Tq={Tq} Tkv={Tkv} D={D} {dtype}", flush=True)
        g = torch.Generator().manual_seed(case)
        q = torch.randn(B, H, Tq, D, generator=g).to(dtype)
        k = torch.randn(B, H, Tkv, D, generator=g).to(dtype)
        v = torch.randn(B, H, Tkv, D, generator=g).to(dtype)
        o = torch.full((B, Tq, H * D), float("nan"), dtype=dtype, device=dev)
        ops.attention_fp16(q.to(dev), k.to(dev), v.to(dev), o, D**-0.5)
        torch.cuda.synchronize()
        ref = O.attention_fp16(q, k, v, D**-0.5)
        assert bool(torch.isfinite(o.float()).all())
        assert O.max_rel_err(o.cpu(), ref) <= 1e-2


def test_epilogue_random_shapes(dev):
    from nunchaku_rocm_amd import ops

    rnd = random.Random(77)
    for case in range(16):
        M = 16 * rnd.randint(1, 18)
        N = 128 * rnd.randint(1, 4)
        K = 64 * rnd.randint(1, 6)
        R, R2 = rnd.choice([0, 16, 32]), rnd.choice([0, 16, 32, 48])
        smooth_on, store_out = rnd.random() < 0.7, rnd.random() < 0.5
        dtype = rnd.choice([torch.bfloat16, torch.float16])
        print(f"case {case}: gelu M={M} N={N} K={K} R={R} R2={R2} smooth={smooth_on} out={store_out} {dtype}", flush=True)
        g = torch.Generator().manual_seed(1000 + case)
        act = torch.randint(0, 256, (M, K // 2), generator=g, dtype=torch.uint8)
        wgt = torch.randint(0, 256, (N, K // 2), generator=g, dtype=torch.uint8)
        asc = (torch.rand(K // 64, M, generator=g) * 0.02 + 0.01).to(dtype)
        wsc = (torch.rand(K // 64, N, generator=g) * 0.02 + 0.01).to(dtype)
        b = torch.randn(N, generator=g).to(dtype)
        la = torch.randn(M, R, generator=g) if R else None
        lu = (torch.randn(N, R, generator=g) * 0.1).to(dtype) if R else None
        sm = (torch.rand(N, generator=g) + 0.5).to(dtype) if smooth_on else None
        ld = (torch.randn(N, R2, generator=g) * 0.1).to(dtype) if R2 else None
        d = lambda t: None if t is None else t.to(dev)  # noqa: E731
        qout = torch.zeros(M + 16, N // 2, dtype=torch.uint8, device=dev)
        osc = torch.empty(N // 64, M, dtype=dtype, device=dev)
        lao = torch.empty(M, R2, dtype=torch.float32, device=dev) if R2 else None
        out = torch.empty(M, N, dtype=dtype, device=dev) if store_out else None
        ops.svdq_gemm_w4a4_cuda(act=d(act), wgt=d(wgt), out=out, qout=qout, ascales=d(asc), wscales=d(wsc), oscales=osc,
                                lora_act_in=d(la), lora_up=d(lu), lora_down=d(ld), lora_act_out=lao, bias=d(b),
                                smooth_factor=d(sm))  # fmt: skip
        torch.cuda.synchronize()
        assert (qout[M:] == 0).all()
        lin = O.gemm_w4a4(act, wgt, asc, wsc, b, la, lu, False)
        rp, rs, rl, rc = O.gelu_quant(lin, sm, ld, dtype)
        diff = (O.unpack_int4(qout[:M].cpu(), False) - rc).abs()
        assert diff.max() <= 1 and (diff > 0).float().mean() < 2e-3
        ulp = 2**-7 if dtype == torch.bfloat16 else 2**-10
        assert ((osc.cpu().float() - rs.float()).abs() <= rs.float().abs() * ulp + 1e-7).all()
        if R2:
            assert (lao.cpu() - rl).abs().max() <= 1e-2 * rl.abs().max()
        if store_out:
            assert O.max_rel_err(out.cpu(), lin) <= 1e-2

    for case in range(10):
        H = rnd.randint(1, 3)
        M = rnd.choice([8, 64, 100, 136, 256, 300])
        am = rnd.randint(1, M)
        K, N = 64 * rnd.randint(1, 5), 3 * H * 128
        dtype = rnd.choice([torch.bfloat16, torch.float16])
        print(f"case {case}: rope M={M} H={H} K={K} actual_m={am} {dtype}", flush=True)
        g = torch.Generator().manual_seed(2000 + case)
        act = torch.randint(0, 256, (M, K // 2), generator=g, dtype=torch.uint8)
        wgt = torch.randint(0, 256, (N, K // 2), generator=g, dtype=torch.uint8)
        asc = (torch.rand(K // 64, M, generator=g) * 0.02 + 0.01).to(dtype)
        wsc = (torch.rand(K // 64, N, generator=g) * 0.02 + 0.01).to(dtype)
        b = torch.randn(N, generator=g).to(dtype)
        nq = (torch.rand(128, generator=g) + 0.5).to(dtype)
        nk = (torch.rand(128, generator=g) + 0.5).to(dtype)
        theta = torch.rand(am, 64, generator=g) * 6.28
        rot = torch.stack([torch.sin(theta), torch.cos(theta)], -1).reshape(am, 64, 1, 2).float()
        d = lambda t: t.to(dev)  # noqa: E731
        buf = torch.full((am + 2, N), float("nan"), dtype=dtype, device=dev)
        ops.svdq_gemm_w4a4_cuda(act=d(act), wgt=d(wgt), out=buf[:am], ascales=d(asc), wscales=d(wsc), bias=d(b),
                                norm_q=d(nq), norm_k=d(nk), rotary_emb=d(rot))  # fmt: skip
        torch.cuda.synchronize()
        assert bool(buf[am:].isnan().all())
        lin = O.gemm_w4a4(act, wgt, asc, wsc, b)[:am]
        ref = O.qk_norm_rope(lin, nq, nk, rot.reshape(am, 128))
        assert O.max_rel_err(buf[:am].cpu(), ref) <= 1e-2


def test_awq_random_shapes(dev):
    from nunchaku_rocm_amd import ops

    rnd = random.Random(5)
    for case in range(16):
        m = rnd.choice([1, 2, 3, 8, 9, 17, 32, 33, 40])
        N, K = 32 * rnd.randint(1, 12), 64 * rnd.randint(1, 10)
        dtype = rnd.choice([torch.bfloat16, torch.float16])
        print(f"case {case}: m={m} N={N} K={K} {dtype}", flush=True)
        lin = O.make_awq_linear(K, N, seed=case, dtype=dtype)
        x = torch.randn(m, K, generator=torch.Generator().manual_seed(300 + case)).to(dtype)
        out = ops.awq_gemv_w4a16_cuda(x.to(dev), lin["qweight"].to(dev), lin["wscales"].to(dev), lin["wzeros"].to(dev), m, N, K)
        torch.cuda.synchronize()
        ref = O.awq_gemv(x, lin["qweight"].view(torch.int16).reshape(N // 4, K), lin["wscales"], lin["wzeros"])
        assert O.max_rel_err(out.cpu(), ref) <= 1e-2
