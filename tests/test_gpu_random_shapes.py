"""Seeded sweeps over odd shapes (ragged M, N not a multiple of the tile, odd group counts, ranks 0..64, rows past
``actual_m``) of the quantizer, the GEMM and attention against the CPU oracle: the bars of the fixed-shape tests, on shapes
nobody picked by hand."""

import random

import pytest
import torch

from oracle import svdq_oracle as O

pytestmark = pytest.mark.gpu


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
