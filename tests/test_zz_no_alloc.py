"""The GEMM entry point that allocates nothing (``svdq_gemm_w4a4_static_scratch``: LoRA-down partial sums in a buffer
built into the library) against ``svdq_gemm_w4a4`` with a caller-provided buffer: bit-identical codes, scales, LoRA
hidden state and 16-bit output, on two calls in a row, the second with a smaller input (the buffer keeps the first
call's contents), and a clear refusal beyond the buffer's size."""

import pytest
import torch

from oracle import svdq_oracle as O

pytestmark = pytest.mark.gpu


def _run(dev, M, N, K, R2, swiglu, static, seed):
    from nunchaku_rocm_amd import ops
    from nunchaku_rocm_amd.ops import gemm as G

    dtype = torch.bfloat16
    lin = O.make_svdq_linear(K, N, seed=seed, dtype=dtype)
    g = torch.Generator().manual_seed(seed + 1)
    act = torch.randint(0, 256, (M, K // 2), generator=g, dtype=torch.uint8)
    asc = (torch.rand(K // 64, M, generator=g) * 0.2 + 0.05).to(dtype)
    NQ = N // 2 if swiglu else N
    smooth = (torch.rand(NQ, generator=g) + 0.5).to(dtype)
    ld = (torch.randn(NQ, R2, generator=g) * 0.1).to(dtype)
    d = lambda t: t.to(dev)  # noqa: E731
    qout = torch.zeros(M, NQ // 2, dtype=torch.uint8, device=dev)
    osc = torch.zeros(NQ // 64, M, dtype=dtype, device=dev)
    lao = torch.zeros(M, R2, dtype=torch.float32, device=dev)
    out = None if swiglu else torch.zeros(M, N, dtype=dtype, device=dev)
    G.STATIC_SCRATCH = static
    try:
        ops.svdq_gemm_w4a4_cuda(
            act=d(act), wgt=d(lin["qweight"]), out=out, qout=qout, ascales=d(asc), wscales=d(lin["wscales"]), oscales=osc,
            lora_down=d(ld), lora_act_out=lao, bias=d(lin["bias"]), smooth_factor=d(smooth), fuse_swiglu=swiglu,
        )  # fmt: skip
        torch.cuda.synchronize()
    finally:
        G.STATIC_SCRATCH = False
    return qout.cpu(), osc.cpu().view(torch.int16), lao.cpu(), None if out is None else out.cpu().view(torch.int16)


@pytest.mark.parametrize("swiglu", [False, True])
def test_static_scratch_matches_caller_scratch_twice(dev, swiglu):
    # first a larger problem, then a smaller one: the second call finds the first call's partial sums in the buffer
    for M, N, K, R2, seed in ((272, 512, 256, 48, 5), (80, 256, 128, 16, 6)):
        print(f"case swiglu={swiglu} M={M} N={N} K={K} R2={R2}", flush=True)
        ref = _run(dev, M, N, K, R2, swiglu, False, seed)
        got = _run(dev, M, N, K, R2, swiglu, True, seed)
        for r, g_ in zip(ref, got):
            assert (r is None and g_ is None) or torch.equal(r, g_)
        assert ref[2].abs().max() > 0  # the LoRA-down branch did run


def test_static_scratch_under_graph_capture(dev):
    """The use the entry point is for: a GELU-epilogue GEMM captured into a HIP graph (the buffer's address looked up
    beforehand, as the header asks) and replayed, the program's own eager work between the replays; every replay gives
    the eager call's bits."""
    from nunchaku_rocm_amd import ops
    from nunchaku_rocm_amd.ops import gemm as G

    M, N, K, R2, dtype = 272, 512, 256, 48, torch.bfloat16
    lin = O.make_svdq_linear(K, N, seed=7, dtype=dtype)
    g = torch.Generator().manual_seed(8)
    t = {"act": torch.randint(0, 256, (M, K // 2), generator=g, dtype=torch.uint8), "asc": (torch.rand(K // 64, M, generator=g) * 0.2 + 0.05).to(dtype),
         "smooth": (torch.rand(N, generator=g) + 0.5).to(dtype), "ld": (torch.randn(N, R2, generator=g) * 0.1).to(dtype)}  # fmt: skip
    t = {k: v.to(dev) for k, v in t.items()}
    w = {k: v.to(dev) for k, v in lin.items()}
    qout = torch.zeros(M, N // 2, dtype=torch.uint8, device=dev)
    osc = torch.zeros(N // 64, M, dtype=dtype, device=dev)
    lao = torch.zeros(M, R2, dtype=torch.float32, device=dev)
    out = torch.zeros(M, N, dtype=dtype, device=dev)

    def call():
        ops.svdq_gemm_w4a4_cuda(act=t["act"], wgt=w["qweight"], out=out, qout=qout, ascales=t["asc"], wscales=w["wscales"],
                                oscales=osc, lora_down=t["ld"], lora_act_out=lao, bias=w["bias"], smooth_factor=t["smooth"])  # fmt: skip

    call()  # eager, caller-provided scratch; also makes the cached re-layouts of the weights
    torch.cuda.synchronize()
    want = [x.clone() for x in (qout, osc, lao, out)]
    G.prepare_static_scratch(dev)
    G.STATIC_SCRATCH = True
    try:
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            call()
        for rep in range(3):
            for x in (qout, osc, lao, out):
                x.fill_(0)  # a fill kernel, eager, between the replays
            graph.replay()
            torch.cuda.synchronize()
            for got, ref in zip((qout, osc, lao, out), want):
                assert torch.equal(got.view(torch.uint8), ref.view(torch.uint8)), f"replay {rep}"
    finally:
        G.STATIC_SCRATCH = False


def test_static_scratch_refuses_what_does_not_fit(dev):
    from nunchaku_rocm_amd import _lib

    lib = _lib.load()
    cap = lib.svdq_gemm_w4a4_static_scratch_capacity()
    assert cap == 16 << 20
    M, N, R2 = 4608, 12288, 32  # 96 tiles x 4608 rows x 32 ranks x 4 bytes = 56.6 MB
    assert lib.svdq_gemm_w4a4_scratch_bytes(M, N, R2, _lib.EPI_GELU_QUANT) > cap
    g = _lib.GemmArgs(act=16, wgt=16, ascales=16, wscales=16, M=M, N=N, K=128, R2=R2, ld_act=64, ld_wgt=64, ld_ascales=M,
                      ld_wscales=N, actual_m=M, epilogue=_lib.EPI_GELU_QUANT, qout=16, oscales=16, lora_down_t=16,
                      lora_act_out=16, ld_qout=N // 2, ld_oscales=M, ld_lora_act_out=R2)  # fmt: skip
    assert lib.svdq_gemm_w4a4_static_scratch(g, None) == _lib.E_UNSUPPORTED
    assert b"caller-provided scratch" in lib.svdq_last_error()
