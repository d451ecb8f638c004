#!/usr/bin/env python3
"""Benchmark of the SVDQuant kernel path on one MI355X.

A step is one pass of the hot path over one batch of synthetic input: the FLUX.1 QKV linear
(M=4608 tokens, K=3072, N=9216, group 64, LoRA rank 32) as activation quantizer + W4A4 GEMM, inputs resident in HBM.
``value`` is 2*M*N*K / step time in TOP/s (the reference's GEMM convention, tests/triton/bench_kernels.py:61, charged
with the quantizer's time as well).  The step's two launches are recorded once into a HIP graph and the timed region
replays it, so the figure is what the kernels take and not what Python needs to marshal two calls (about 15 us each,
more than the quantizer runs); ``--eager`` times the eager calls instead.  Every timed region follows at least 0.12 s
of the same work without a pause (the W warm-up steps and as many more as that takes): the GPU's clocks need about
50 ms of continuous work to settle, and the settled rate is the one a denoising loop sees.  The JSON line also carries the roofline of
the dominant kernel (the GEMM: HIP events on the launch stream around back-to-back launches of it, the figure the
rocprofv3 kernel trace under profiles/ reproduces), a per-kernel table (quantizer GB/s, AWQ GEMV GB/s, GEMM M-sweep and fused
epilogue shapes), and the CPU baseline (the oracle's pure-PyTorch restatement of the reference's CPU path).

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu-baseline] [--no-extras] [--eager]
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

INT8_MFMA_PEAK_TOPS = 5000.0  # MI355X dense int8 MFMA, published
FP6_MFMA_PEAK_TOPS = 10100.0  # MI355X dense fp6 / fp4 MFMA, published
BF16_MFMA_PEAK_TFLOPS = 2500.0  # MI355X dense bf16 / fp16 MFMA, published
HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published
# HBM bytes of one QKV GEMM launch: 2.00 x FETCH_SIZE + 1.00 x WRITE_SIZE (KiB per dispatch) of the grid-663552 launches
# in profiles/bench_all_kernels_hbm_traffic.txt, the factors being what the same counters read on plain copy kernels of
# known size in the same run (FETCH_SIZE reads half the bytes of 16-byte-per-lane loads); counters cannot be read from
# inside this process
GEMM_QKV_HBM_BYTES = (2.0 * 103184.3 + 82944.0) * 1024


def _events(n):
    import torch

    return [torch.cuda.Event(enable_timing=True) for _ in range(n)]


STEADY_S = 0.12  # continuous work before a timed region: the GPU's clocks take about 50 ms of it to settle


def _steady(run, seconds=STEADY_S):
    """Repeat ``run`` (a batch of launches) until ``seconds`` of wall time have passed without the GPU going idle for
    longer than a host round trip.  After an idle period the QKV GEMM takes 240 us per launch and settles at 194 us
    within 50 ms of continuous launches (measured in batches of 20 launches: 240, 229, 219, 213, 210, 206, 201, 198,
    196, 194, then 193-195 for the next 1000 launches).  Every figure of this benchmark is the settled one."""
    import torch

    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        run()
        torch.cuda.synchronize()


def _time_kernel(fn, iters=50, warmup=10, graph=False):
    """Average launch duration in ms at settled clocks: HIP events on the launch stream around ``iters`` back-to-back
    launches.  ``graph=True`` records the launches into one HIP graph first, which takes the host's launch cost (about
    15 us per call through ctypes, more than the small kernels run) out of the figure."""
    import torch

    for _ in range(warmup):
        fn()
    a, b = _events(2)
    torch.cuda.synchronize()
    if graph:
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for _ in range(iters):
                fn()
        _steady(g.replay)
        a.record()
        g.replay()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) / iters

    def batch():
        for _ in range(iters):
            fn()

    _steady(batch)
    a.record()
    batch()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / iters


def cpu_baseline(M, K, N):
    """The oracle (a pure-PyTorch port of the reference's CPU-runnable path: quantizer restatement + per-group fp32
    GEMM + LoRA-up + bias, nunchaku/ops/triton/native/w4a4.py:713-726) timed on this host's cores."""
    import torch

    from oracle import svdq_oracle as O

    cores = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "0") or (os.cpu_count() or 1)))
    torch.set_num_threads(cores)
    lin = O.make_svdq_linear(K, N, seed=0)
    x = O.make_activations(M, K, seed=1)

    def run(rows):
        rp, rs, rl, _ = O.quantize_act(x[:rows], lin["proj_down"], lin["smooth_factor"])
        return O.gemm_w4a4(rp, lin["qweight"], rs, lin["wscales"], lin["bias"], rl, lin["proj_up"])

    run(M)  # warm-up
    times = []
    for _ in range(3):
        t0 = time.perf_counter()
        run(M)
        times.append(time.perf_counter() - t0)
    t = sorted(times)[1]  # median of three
    return {
        "value": round(2.0 * M * N * K / t / 1e12, 4),
        "unit": "TOP/s",
        "cores": cores,
        "kind": "port",
        "sample": f"full config 0 (M={M}, K={K}, N={N}, R=32): quantizer + GEMM, one warm-up then the median of {len(times)} runs ({t:.2f} s), torch {torch.__version__} CPU fp32",
        "seconds": round(t, 3),
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extras", action="store_true")
    ap.add_argument("--eager", action="store_true", help="time the small kernels eagerly too (no HIP graph): for counter runs")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs on one GPU only (the path would shard over tokens with no exchange between "
              "GPUs, and no multi-GPU figure is produced); run with --gpus 1", file=sys.stderr)  # fmt: skip
        sys.exit(2)

    import torch

    from nunchaku_rocm_amd import _lib, ops
    from oracle import svdq_oracle as O  # input generators only; nothing from the oracle is timed on the GPU side

    _lib.load()
    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    # torch loads a kernel's code object at that kernel's first launch.  Under rocprofv3's counter collection such a first
    # launch late in the run (the small index and table kernels of the model set-up, 12 GB already allocated) has crashed
    # the profiler on some boxes; launched once here, while the device is empty, it does not.
    if not args.no_extras:
        from nunchaku_rocm_amd.flux_shaped import FluxShapedConfig, flux_ids, rope_table

        torch.arange(4, device=dev).sum().item()
        rope_table(flux_ids(8, 2, 2, device=dev), FluxShapedConfig().axes_dim, FluxShapedConfig().theta).sum().item()
    M, K, N, R = 4608, 3072, 9216, 32
    # weights as module parameters, which is what the operators see in a model (the GEMM keeps its re-laid-out working
    # copy per parameter)
    lin = {k: torch.nn.Parameter(v.to(dev), requires_grad=False) for k, v in O.make_svdq_linear(K, N, R, seed=0).items()}
    x = O.make_activations(M, K, seed=1).to(dev)
    qx = torch.empty(M, K * 3 // 4, dtype=torch.uint8, device=dev)  # fp6 codes in the GEMM's lane order
    asc = torch.empty(K // 64, M, dtype=torch.bfloat16, device=dev)
    la = torch.empty(M, R, dtype=torch.float32, device=dev)
    out = torch.empty(M, N, dtype=torch.bfloat16, device=dev)

    # The two operator calls of SVDQW4A4Linear.forward, with the hand-over it uses: the quantizer writes the codes as fp6
    # (sign | magnitude) in the order the GEMM's lanes read them, and the scales so that one load brings eight groups'
    # (out_blocked = act_blocked = 3: the same integers and scales, the codes taken by the matrix instruction as they are).  The GEMM on the reference's (M, K/2) matrix is
    # timed next to it in the per-kernel table.
    def quant():
        ops.svdq_quantize_w4a4_act_fuse_lora_cuda(x, qx, asc, lin["proj_down"], la, lin["smooth_factor"], out_blocked=3)

    def gemm():
        ops.svdq_gemm_w4a4_cuda(act=qx, wgt=lin["qweight"], out=out, ascales=asc, wscales=lin["wscales"],
                                lora_act_in=la, lora_up=lin["proj_up"], bias=lin["bias"], act_blocked=3)  # fmt: skip

    def step():
        quant()
        gemm()

    for _ in range(max(args.warmup, 3)):  # also builds the cached weight re-layouts before anything is recorded
        step()
    torch.cuda.synchronize()
    if args.eager:
        run_step = step
    else:
        step_graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(step_graph):
            step()
        run_step = step_graph.replay
        for _ in range(args.warmup):
            run_step()
    torch.cuda.synchronize()

    def steps_back_to_back():
        for _ in range(args.steps):
            run_step()

    _steady(steps_back_to_back)  # more untimed steps, until the clocks have settled (see _steady)
    t0 = time.perf_counter()
    for _ in range(args.steps):
        run_step()
    torch.cuda.synchronize()
    step_ms = (time.perf_counter() - t0) * 1e3 / args.steps
    # the GEMM kernel by itself: events on the launch stream around back-to-back eager launches (the host queues them
    # faster than they run; a graph of identical launches lets one launch's workgroups fill the emptying slots of the
    # one before and reads 10 % low)
    gemm_ms = _time_kernel(gemm, iters=max(args.steps, 20), warmup=5)
    quant_ms = _time_kernel(quant, iters=max(args.steps, 20), warmup=5, graph=not args.eager)
    ops_per_gemm = 2.0 * M * N * K
    achieved = ops_per_gemm / (gemm_ms * 1e-3) / 1e12

    kernels = {}
    if not args.no_extras:
        q_ms = _time_kernel(quant, graph=not args.eager)
        q_bytes = 2 * M * K + M * K // 2 + 2 * (K // 64) * M + 4 * M * R + 2 * K * R + 2 * K
        kernels["quantize_act M4608 K3072 R32"] = {
            "ms": round(q_ms, 5), "GB/s": round(q_bytes / q_ms / 1e6, 1), "frac_hbm": round(q_bytes / q_ms / 1e6 / HBM_PEAK_GBS, 4),
            "bytes": q_bytes, "GB/s_ref_convention": round((2 * M * K + M * K // 2) / q_ms / 1e6, 1),
        }  # fmt: skip
        # the same quantizer with LayerNorm + adaLN modulate applied on the way in, and the row statistics it needs
        nsc = (1 + 0.3 * torch.randn(K, device=dev)).to(torch.bfloat16)
        nsh = (0.2 * torch.randn(K, device=dev)).to(torch.bfloat16)
        st = ops.layer_norm_stats(x)
        ms = _time_kernel(lambda: ops.svdq_quantize_w4a4_act_fuse_lora_cuda(x, qx, asc, lin["proj_down"], la, lin["smooth_factor"], norm=(nsc, nsh, st)), graph=not args.eager)
        nb = q_bytes + 8 * M + 4 * K
        kernels["quantize_act + layernorm + modulate M4608 K3072 R32"] = {"ms": round(ms, 5), "GB/s": round(nb / ms / 1e6, 1), "frac_hbm": round(nb / ms / 1e6 / HBM_PEAK_GBS, 4), "bytes": nb}  # fmt: skip
        ms = _time_kernel(lambda: ops.layer_norm_stats(x), graph=not args.eager)
        nb = 2 * M * K + 8 * M
        kernels["row_stats M4608 K3072"] = {"ms": round(ms, 5), "GB/s": round(nb / ms / 1e6, 1), "frac_hbm": round(nb / ms / 1e6 / HBM_PEAK_GBS, 4), "bytes": nb}  # fmt: skip
        # gated residual update (x + gate * y) with the row statistics of the result
        xr = x.view(1, M, K)
        yr = torch.randn(1, M, K, device=dev).to(torch.bfloat16)
        gt = torch.randn(1, K, device=dev).to(torch.bfloat16)
        orr = torch.empty_like(xr)
        ms = _time_kernel(lambda: ops.gated_residual(xr, gt, yr, out=orr, want_stats=True), graph=not args.eager)
        nb = 3 * 2 * M * K + 2 * K + 8 * M
        kernels["gated_residual + row_stats M4608 K3072"] = {"ms": round(ms, 5), "GB/s": round(nb / ms / 1e6, 1), "frac_hbm": round(nb / ms / 1e6 / HBM_PEAK_GBS, 4), "bytes": nb}  # fmt: skip
        del yr, orr
        g_ms = _time_kernel(gemm)
        qn = ops.svdq_quantize_w4a4_act_fuse_lora_cuda(x, lora_down=lin["proj_down"], smooth=lin["smooth_factor"])[0]  # the matrix
        n_ms = _time_kernel(lambda: ops.svdq_gemm_w4a4_cuda(act=qn, wgt=lin["qweight"], out=out, ascales=asc, wscales=lin["wscales"],
                                                            lora_act_in=la, lora_up=lin["proj_up"], bias=lin["bias"]))  # fmt: skip
        del qn
        kernels["gemm_w4a4 M4608 K3072 N9216"] = {"ms": round(g_ms, 5), "TOP/s": round(ops_per_gemm / g_ms / 1e9, 1),
                                                  "frac_int8_mfma": round(ops_per_gemm / g_ms / 1e9 / INT8_MFMA_PEAK_TOPS, 4),
                                                  "ms_act_as_matrix": round(n_ms, 5)}  # fmt: skip
        for Ms in (1024, 8192):
            xs = O.make_activations(Ms, K, seed=1).to(dev)
            q2, a2, l2 = ops.svdq_quantize_w4a4_act_fuse_lora_cuda(xs, lora_down=lin["proj_down"], smooth=lin["smooth_factor"], out_blocked=3)
            o2 = torch.empty(Ms, N, dtype=torch.bfloat16, device=dev)
            ms = _time_kernel(lambda: ops.svdq_gemm_w4a4_cuda(act=q2, wgt=lin["qweight"], out=o2, ascales=a2, wscales=lin["wscales"],
                                                              lora_act_in=l2, lora_up=lin["proj_up"], bias=lin["bias"], act_blocked=3))  # fmt: skip
            kernels[f"gemm_w4a4 M{Ms} K3072 N9216"] = {"ms": round(ms, 5), "TOP/s": round(2.0 * Ms * N * K / ms / 1e9, 1),
                                                       "frac_int8_mfma": round(2.0 * Ms * N * K / ms / 1e9 / INT8_MFMA_PEAK_TOPS, 4)}  # fmt: skip
            del xs, q2, a2, l2, o2
        # fused epilogues at the FLUX MLP / attention shapes
        from nunchaku_rocm_amd.linear import SVDQW4A4Linear

        def module(k, n, seed, act_unsigned=False):
            p = O.make_svdq_linear(k, n, seed=seed)
            m = SVDQW4A4Linear(k, n, rank=32, act_unsigned=act_unsigned, device=dev)
            with torch.no_grad():
                for name in ("qweight", "wscales", "smooth_factor", "proj_down", "proj_up", "bias"):
                    getattr(m, name).copy_(p[name])
            return m

        fc1, fc2 = module(3072, 12288, 42), module(12288, 3072, 43, True)
        q1, a1, l1 = fc1.quantize(x, blocked=3)
        qo = torch.empty(M, 12288 * 3 // 4, dtype=torch.uint8, device=dev)  # fp6 codes in fc2's lane order
        oo = torch.empty(192, M, dtype=torch.bfloat16, device=dev)
        lo = torch.empty(M, 32, dtype=torch.float32, device=dev)
        y2 = torch.empty(M, 3072, dtype=torch.bfloat16, device=dev)

        def fc1_fused():
            ops.svdq_gemm_w4a4_cuda(act=q1, wgt=fc1.qweight, qout=qo, ascales=a1, wscales=fc1.wscales, oscales=oo, lora_act_in=l1,
                                    lora_up=fc1.proj_up, lora_down=fc2.proj_down, lora_act_out=lo, bias=fc1.bias,
                                    smooth_factor=fc2.smooth_factor, act_blocked=3, qout_blocked=3)  # fmt: skip

        ms = _time_kernel(fc1_fused)
        f = 2.0 * M * 12288 * 3072
        kernels["gemm_w4a4+gelu+requant fc1 M4608 K3072 N12288"] = {"ms": round(ms, 5), "TOP/s": round(f / ms / 1e9, 1), "frac_int8_mfma": round(f / ms / 1e9 / INT8_MFMA_PEAK_TOPS, 4)}  # fmt: skip
        ms = _time_kernel(lambda: fc2.forward_quant(qo, oo, lo, y2, act_blocked=3))
        kernels["gemm_w4a4 fc2 (unsigned act) M4608 K12288 N3072"] = {"ms": round(ms, 5), "TOP/s": round(f / ms / 1e9, 1), "frac_int8_mfma": round(f / ms / 1e9 / INT8_MFMA_PEAK_TOPS, 4)}  # fmt: skip
        nq = (torch.rand(128, device=dev) + 0.5).to(torch.bfloat16)
        rot = O.flux_rotary(O.flux_ids(512, 64, 64)).to(dev)
        ms = _time_kernel(lambda: ops.svdq_gemm_w4a4_cuda(act=qx, wgt=lin["qweight"], out=out, ascales=asc, wscales=lin["wscales"],
                                                          lora_act_in=la, lora_up=lin["proj_up"], bias=lin["bias"], norm_q=nq, norm_k=nq, rotary_emb=rot,
                                                          act_blocked=3))  # fmt: skip
        kernels["gemm_w4a4+qknorm+rope M4608 K3072 N9216"] = {"ms": round(ms, 5), "TOP/s": round(ops_per_gemm / ms / 1e9, 1), "frac_int8_mfma": round(ops_per_gemm / ms / 1e9 / INT8_MFMA_PEAK_TOPS, 4)}  # fmt: skip
        # AWQ GEMV, adaLN shape.  In the model every adaLN layer has its own weight, so a launch finds its 32 MB in HBM, not in
        # the 256 MB memory-side cache: the launches of the timed graph walk over 12 weight sets (384 MB) in turn ("cold",
        # the figure reported as frac_hbm); the same weight launch after launch ("warm") is listed beside it.
        import itertools

        aw = {k: v.to(dev) for k, v in O.make_awq_linear(3072, 18432, seed=2).items() if k != "codes"}
        aw_sets = [aw] + [{"qweight": torch.randint(-(2**31), 2**31 - 1, aw["qweight"].shape, dtype=torch.int32, device=dev),
                           "wscales": aw["wscales"].clone(), "wzeros": aw["wzeros"].clone()} for _ in range(11)]  # fmt: skip
        for m in (1, 2, 8):
            xv = torch.randn(m, 3072, device=dev).to(torch.bfloat16)
            turn = itertools.count()

            def gemv_cold():
                w = aw_sets[next(turn) % len(aw_sets)]
                ops.awq_gemv_w4a16_cuda(xv, w["qweight"], w["wscales"], w["wzeros"], m, 18432, 3072)

            ms = _time_kernel(gemv_cold, iters=204, warmup=24, graph=not args.eager)
            warm = _time_kernel(lambda: ops.awq_gemv_w4a16_cuda(xv, aw["qweight"], aw["wscales"], aw["wzeros"], m, 18432, 3072), iters=200, warmup=20, graph=not args.eager)
            nbytes = 18432 * 3072 // 2 + 2 * 2 * 48 * 18432 + 2 * m * 3072 + 2 * m * 18432
            kernels[f"awq_gemv_w4a16 M{m} K3072 N18432"] = {"ms": round(ms, 5), "GB/s": round(nbytes / ms / 1e6, 1),
                                                           "frac_hbm": round(nbytes / ms / 1e6 / HBM_PEAK_GBS, 4), "bytes": nbytes,
                                                           "weights": "12 sets in turn (384 MB): read from HBM",
                                                           "ms_same_weight": round(warm, 5), "frac_hbm_same_weight": round(nbytes / warm / 1e6 / HBM_PEAK_GBS, 4)}  # fmt: skip
            # the twelve weights in ONE launch, as a model can run its adaLN projections (all take the same vector)
            batch = ops.AwqGemvBatch([w["qweight"] for w in aw_sets], [w["wscales"] for w in aw_sets], [w["wzeros"] for w in aw_sets], m, 18432, 3072)
            ms = _time_kernel(lambda: batch(xv), iters=20, warmup=3, graph=not args.eager) / len(aw_sets)
            kernels[f"awq_gemv_w4a16 M{m} K3072 N18432, 12 layers per launch"] = {
                "ms_per_layer": round(ms, 5), "GB/s": round(nbytes / ms / 1e6, 1), "frac_hbm": round(nbytes / ms / 1e6 / HBM_PEAK_GBS, 4),
                "bytes_per_layer": nbytes, "note": "svdq_awq_gemv_w4a16_batched; includes the copy of x into the batch's buffer"}  # fmt: skip
            del batch
        del aw_sets

        # joint attention of one FLUX.1 block: 24 heads, 512 + 4096 tokens, q / k / v strided views of the fused projection
        qkv_t = torch.randn(1, M, 3 * 3072, device=dev).to(torch.bfloat16)
        aq, ak, av = (qkv_t[..., i * 3072 : (i + 1) * 3072].view(1, M, 24, 128).transpose(1, 2) for i in range(3))
        ao = torch.empty(1, M, 3072, dtype=torch.bfloat16, device=dev)
        ms = _time_kernel(lambda: ops.attention_fp16(aq, ak, av, ao, 128**-0.5))
        fl = 4.0 * M * M * 128 * 24
        kernels["attention bf16 H24 T4608 D128"] = {"ms": round(ms, 5), "TFLOP/s": round(fl / ms / 1e9, 1),
                                                     "frac_bf16_mfma": round(fl / ms / 1e9 / BF16_MFMA_PEAK_TFLOPS, 4)}  # fmt: skip
        del qkv_t, aq, ak, av, ao

        # FLUX.1-schnell-shaped transformer, 4 denoising steps at 1024^2 (4096 image + 512 text tokens)
        from nunchaku_rocm_amd.flux_shaped import FluxShapedConfig, FluxShapedTransformer, flux_ids, rope_table

        del fc1, fc2, q1, a1, l1, qo, oo, lo, y2, aw
        cfg = FluxShapedConfig()
        model = FluxShapedTransformer(cfg, device=dev, seed=0)
        lat = torch.randn(1, 4096, 64, device=dev).to(torch.bfloat16)
        txt = torch.randn(1, 512, 4096, device=dev).to(torch.bfloat16)
        pooled = torch.randn(1, 768, device=dev).to(torch.bfloat16)
        rot = rope_table(flux_ids(512, 64, 64, device=dev), cfg.axes_dim, cfg.theta)
        model.denoise(lat, txt, pooled, rot, steps=1)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        model.denoise(lat, txt, pooled, rot, steps=4)
        torch.cuda.synchronize()
        kernels["flux1_schnell_shaped 19+38 blocks 4608 tokens"] = {"s_per_step": round((time.perf_counter() - t1) / 4, 4), "steps": 4}
        if not args.eager:
            # the same steps with each forward pass replayed from one recorded HIP graph (both streams' launches)
            step_fn = model.capture(lat, txt, pooled, rot)
            model.denoise(lat, txt, pooled, rot, steps=1, step_fn=step_fn)
            torch.cuda.synchronize()
            t1 = time.perf_counter()
            model.denoise(lat, txt, pooled, rot, steps=4, step_fn=step_fn)
            torch.cuda.synchronize()
            kernels["flux1_schnell_shaped 19+38 blocks 4608 tokens, HIP graph"] = {
                "s_per_step": round((time.perf_counter() - t1) / 4, 4), "steps": 4}  # fmt: skip
            del step_fn
        del model
        # plain elementwise kernel of known size: the scale reference for the FETCH_SIZE / WRITE_SIZE counters
        # (random data, and a second buffer written in between so that the read comes from HBM, not from cache)
        src = torch.randn(64 << 20, dtype=torch.float32, device=dev)
        dst = torch.empty_like(src)
        flush = torch.randn(128 << 20, dtype=torch.float32, device=dev)
        torch.cuda.synchronize()
        torch.add(src, 1.0, out=dst)  # one elementwise kernel: reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()
        del flush
        del src, dst

    result = {
        "metric": "W4A4 GEMM TOPS at the FLUX.1 QKV shape (quantizer + GEMM per step)",
        "value": round(ops_per_gemm / (step_ms * 1e-3) / 1e12, 2),
        "unit": "TOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(step_ms, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "i8",
        "data": "synthetic",
        "config": {"workload": "FLUX.1 QKV SVDQuant linear: activation quantizer + W4A4 GEMM, M=4608 K=3072 N=9216 group 64 LoRA rank 32 (the reference's FLUX.1 QKV benchmark shape); the two operator calls of SVDQW4A4Linear.forward, codes handed over as fp6, and their scales, in the GEMM's lane order",
                   "M": M, "K": K, "N": N, "rank": R, "group": 64},  # fmt: skip
        "roofline": {
            "bound": "mfma",
            "kernel": "gemm_w4a4_f8_kernel<BF16, fp6 activation codes with their scales in the loop's order, plain epilogue, three workgroups per CU>",
            "achieved": round(achieved, 2),
            "peak": INT8_MFMA_PEAK_TOPS,
            "unit": "TOP/s",
            "frac": round(achieved / INT8_MFMA_PEAK_TOPS, 4),
            "traffic": GEMM_QKV_HBM_BYTES,
            "traffic_unit": "bytes per launch (rocprofv3 2.00 x FETCH_SIZE + 1.00 x WRITE_SIZE, the factors from copy kernels of known size; see profiles/)",
            "ops_per_launch": ops_per_gemm,
            "avg_launch_ms": round(gemm_ms, 5),
            "quantizer_launch_ms": round(quant_ms, 5),
            "step_over_kernels": round(step_ms / (gemm_ms + quant_ms), 4),
            "frac_of_fp6_mfma_peak": round(achieved / FP6_MFMA_PEAK_TOPS, 4),
            "note": "2*M*N*K integer ops per launch against the int8 MFMA peak the target is stated in (5.0 POP/s); the group "
                    "products run on the fp6 x fp6 form of v_mfma_scale_f32_32x32x64_f8f6f4 on int4-valued codes (exact integer "
                    "sums), whose own published dense peak is 10.1 POP/s (frac_of_fp6_mfma_peak), next to one 16-bit MFMA "
                    "and 16 fp32 FMAs per 32x32 block and group for the scales; avg_launch_ms = back-to-back launches "
                    "between HIP events on the launch stream",
        },
        "kernels": kernels,
    }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(M, K, N)
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
