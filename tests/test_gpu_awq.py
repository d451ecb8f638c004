"""GPU parity of the AWQ W4A16 GEMV against the CPU oracle (fp32 result, then one rounding to the 16-bit type)."""

import pytest
import torch

from oracle import svdq_oracle as O

pytestmark = pytest.mark.gpu


def _case(dev, m, N, K, dtype, seed):
    from nunchaku_rocm_amd import ops

    lin = O.make_awq_linear(K, N, seed=seed, dtype=dtype)
    g = torch.Generator().manual_seed(seed + 1)
    x = torch.randn(m, K, generator=g).to(dtype)
    out = ops.awq_gemv_w4a16_cuda(x.to(dev), lin["qweight"].to(dev), lin["wscales"].to(dev), lin["wzeros"].to(dev), m, N, K)
    torch.cuda.synchronize()
    ref = O.awq_gemv(x, lin["qweight"].view(torch.int16).reshape(N // 4, K), lin["wscales"], lin["wzeros"])
    return out.cpu(), ref


@pytest.mark.parametrize("m", [1, 2, 8, 5, 32, 40])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_small_shapes(dev, m, dtype):
    print(f"case m={m} {dtype}", flush=True)
    out, ref = _case(dev, m, 128, 256, dtype, seed=m)
    assert out.shape == (m, 128) and out.dtype == dtype
    # fp32 accumulation then one rounding: within one 16-bit ulp of the oracle's rounded value
    tol = ref.abs() * (2**-7 if dtype == torch.bfloat16 else 2**-10) + 1e-3
    assert ((out.float() - ref).abs() <= tol).all()
    assert O.max_rel_err(out, ref) <= 1e-2


@pytest.mark.parametrize("m", [1, 2, 8])
def test_flux_adaln_shape(dev, m):
    """K=3072, N=18432: the double-stream adaLN modulation linear."""
    print(f"case m={m}", flush=True)
    out, ref = _case(dev, m, 18432, 3072, torch.bfloat16, seed=20 + m)
    assert O.max_rel_err(out, ref) <= 1e-2
    assert ((out.float() - ref).abs() <= ref.abs() * 2**-7 + 2e-2).all()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("m,N,K,count", [(1, 18432, 3072, 3), (2, 96, 576, 5), (8, 256, 1088, 2), (3, 64, 64, 7), (5, 9216, 3072, 1),
                                         (8, 4096, 1088, 8), (5, 18432, 3072, 2), (7, 2048, 192, 16), (6, 1056, 640, 16)])
def test_batched_launch_matches_single_launches(dev, m, N, K, count, dtype):
    """``count`` weights of one shape on the same input in one launch (the adaLN projections of a model): every output
    bit as from the single launches, and the oracle's result.  The last four cases have more than four rows and 512
    and more workgroups of 64 channels, where the launch gives a workgroup 64 channels (N = 1056 is no multiple of 64
    and keeps 32)."""
    from nunchaku_rocm_amd import ops

    print(f"case m={m} N={N} K={K} count={count} {dtype}", flush=True)
    lins = [O.make_awq_linear(K, N, seed=40 + i, dtype=dtype) for i in range(count)]
    d = [{k: v.to(dev) for k, v in lin.items() if k != "codes"} for lin in lins]
    x = torch.randn(m, K, generator=torch.Generator().manual_seed(3)).to(dtype)
    batch = ops.AwqGemvBatch([t["qweight"] for t in d], [t["wscales"] for t in d], [t["wzeros"] for t in d], m, N, K)
    for rep in range(2):  # the batch object is reused: its output buffer is overwritten
        xr = (x * (rep + 1)).to(dtype)
        got = batch(xr.to(dev)).cpu()
        assert got.shape == (count, m, N)
        for i, (lin, t) in enumerate(zip(lins, d)):
            single = ops.awq_gemv_w4a16_cuda(xr.to(dev), t["qweight"], t["wscales"], t["wzeros"], m, N, K).cpu()
            assert torch.equal(got[i].view(torch.int16), single.view(torch.int16)), f"problem {i}"
            ref = O.awq_gemv(xr, lin["qweight"].view(torch.int16).reshape(N // 4, K), lin["wscales"], lin["wzeros"])
            assert O.max_rel_err(got[i], ref) <= 1e-2


@pytest.mark.parametrize("m", [1, 3, 4, 7, 12])
@pytest.mark.parametrize("K", [64, 192, 576, 1088, 3136, 3520, 6208])
def test_ragged_k(dev, m, K):
    """Group counts that leave wavefronts without work (K = 64: one group for eight wavefronts), batches that are not
    full (1088 = 17 groups: three wavefronts get three, the others two), and a partial batch after full ones (3136 = 49
    groups, 6208 = 97); every row-count variant of the kernel (1, 2, 4, 8 padded rows, and the one for more than 8)."""
    print(f"case m={m} K={K}", flush=True)
    out, ref = _case(dev, m, 96, K, torch.bfloat16, seed=K + m)
    assert O.max_rel_err(out, ref) <= 1e-2
    assert ((out.float() - ref).abs() <= ref.abs() * 2**-7 + 2e-2).all()


@pytest.mark.parametrize("m", [2, 8, 32])
@pytest.mark.parametrize("K", [3584, 4096, 12288])
def test_long_k(dev, m, K):
    """Long rows for every kernel variant: up to eight rows the kernel's LDS use does not depend on K; K = 12288 with
    32 rows, where the per-group tables of the kernel for more than eight rows do not fit LDS, goes to the operator's
    decode-and-multiply route."""
    print(f"case m={m} K={K}", flush=True)
    out, ref = _case(dev, m, 256, K, torch.bfloat16, seed=K + m)
    assert O.max_rel_err(out, ref) <= 1e-2


def test_linear_module_adds_bias_after_kernel(dev):
    from nunchaku_rocm_amd.linear import AWQW4A16Linear

    K, N = 256, 128
    lin = O.make_awq_linear(K, N, seed=31)
    mod = AWQW4A16Linear(K, N, bias=True, device=dev)
    with torch.no_grad():
        mod.qweight.copy_(lin["qweight"])
        mod.wscales.copy_(lin["wscales"])
        mod.wzeros.copy_(lin["wzeros"])
        mod.bias.copy_(torch.arange(N).to(torch.bfloat16) * 0.01)
    x = torch.randn(2, K, generator=torch.Generator().manual_seed(32)).to(torch.bfloat16)
    y = mod(x.to(dev)).cpu()
    ref = O.awq_gemv(x, lin["qweight"].view(torch.int16).reshape(N // 4, K), lin["wscales"], lin["wzeros"])
    ref = ref.to(torch.bfloat16) + (torch.arange(N).to(torch.bfloat16) * 0.01)
    assert O.max_rel_err(y, ref) <= 1e-2


def test_model_side_batching_follows_the_layers_tensors(dev):
    """The harness batches its adaLN layers through a cached plan of device addresses; a layer whose tensors were replaced
    or whose bias changed in place must not be served from the old plan."""
    from nunchaku_rocm_amd.flux_shaped import HipBackend
    from nunchaku_rocm_amd.linear import AWQW4A16Linear

    K, N = 256, 128
    mods = []
    for i in range(3):
        lin = O.make_awq_linear(K, N, seed=50 + i)
        mod = AWQW4A16Linear(K, N, bias=True, device=dev)
        with torch.no_grad():
            mod.qweight.copy_(lin["qweight"])
            mod.wscales.copy_(lin["wscales"])
            mod.wzeros.copy_(lin["wzeros"])
            mod.bias.copy_(torch.full((N,), 0.25 * i).to(torch.bfloat16))
        mods.append(mod)
    x = torch.randn(1, K, generator=torch.Generator().manual_seed(7)).to(torch.bfloat16).to(dev)
    be = HipBackend(two_streams=False)

    def check():
        got = be.awq_many(x, mods)
        for g, mod in zip(got, mods):
            assert torch.equal(g.cpu().view(torch.int16), mod(x).cpu().view(torch.int16))

    check()
    check()  # from the cached plan
    other = O.make_awq_linear(K, N, seed=99)
    mods[1].qweight.data = other["qweight"].to(dev)  # new storage
    mods[1].wscales.data = other["wscales"].to(dev)
    check()
    with torch.no_grad():
        mods[2].bias.add_(1.0)  # same storage, new values
    check()


@pytest.mark.parametrize("group_size", [32, 64, 128])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_dequantize_bit_exact(dev, group_size, dtype):
    """out = T(q * s + z): q * s is exact in fp32, so kernel and oracle perform the same single rounding."""
    from nunchaku_rocm_amd import ops

    print(f"case group_size={group_size} {dtype}", flush=True)
    K, N = 384, 44
    g = torch.Generator().manual_seed(40 + group_size)
    q = torch.randint(0, 16, (N, K), generator=g, dtype=torch.int32)
    s = (torch.rand(K // group_size, N, generator=g) * 0.015 + 0.005).to(dtype)
    z = (-torch.randint(0, 16, (K // group_size, N), generator=g).float() * s.float()).to(dtype)
    packed = O.awq_pack(q)
    w = ops.awq_dequantize(packed.view(torch.int32).to(dev), s.to(dev), z.to(dev), N, K, group_size, dtype)
    torch.cuda.synchronize()
    assert w.shape == (N, K) and w.dtype == dtype
    assert torch.equal(w.cpu(), O.awq_dequantize(packed, s, z, group_size))


def test_dequantize_flux_adaln_weight(dev):
    from nunchaku_rocm_amd import ops

    K, N = 3072, 18432
    lin = O.make_awq_linear(K, N, seed=41)
    w = ops.awq_dequantize(lin["qweight"].to(dev), lin["wscales"].to(dev), lin["wzeros"].to(dev), N, K, 64, torch.bfloat16)
    torch.cuda.synchronize()
    ref = O.awq_dequantize(lin["qweight"].view(torch.int16).reshape(N // 4, K), lin["wscales"], lin["wzeros"], 64)
    assert torch.equal(w.cpu(), ref)


@pytest.mark.parametrize("m,group_size", [(48, 128), (3, 32), (300, 64)])
def test_gemm_and_gemv_fallback_decode_then_matmul(dev, m, group_size):
    """awq_gemm_w4a16 and the group_size != 64 branch of the GEMV: dense decode, then a library matmul."""
    from nunchaku_rocm_amd import ops

    print(f"case m={m} group_size={group_size}", flush=True)
    K, N = 256, 96
    g = torch.Generator().manual_seed(50 + m)
    q = torch.randint(0, 16, (N, K), generator=g, dtype=torch.int32)
    s = (torch.rand(K // group_size, N, generator=g) * 0.015 + 0.005).to(torch.bfloat16)
    z = (-torch.randint(0, 16, (K // group_size, N), generator=g).float() * s.float()).to(torch.bfloat16)
    x = torch.randn(2, m, K, generator=g).to(torch.bfloat16)
    packed = O.awq_pack(q)
    kern = packed.view(torch.int32).to(dev)
    wref = O.awq_dequantize(packed, s, z, group_size)
    ref = x.float() @ wref.float().t()
    out = ops.awq_gemm_w4a16(x.to(dev), kern, s.to(dev), z.to(dev), group_size=group_size)
    assert out.shape == (2, m, N) and out.dtype == torch.bfloat16
    assert O.max_rel_err(out.cpu(), ref) <= 1e-2
    out2 = ops.gemv_awq(x.to(dev), kern, s.to(dev), z.to(dev), 2 * m, N, K, group_size)
    assert out2.shape == (2, m, N)
    assert O.max_rel_err(out2.cpu(), ref) <= 1e-2
    if group_size == 128:
        assert torch.equal(ops.gemm_awq(x.to(dev), kern, s.to(dev), z.to(dev)), out)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("N,K,group_size", [(256, 512, 128), (128, 256, 64)])
def test_dequantize_inverts_the_packing(dev, dtype, N, K, group_size):
    """Unit scales and zero zero-points: the decoder returns the packed codes exactly (the reference's own round-trip
    test, tests/triton/test_gemm.py:98-110), from the int16 view of the packed tensor as well as the int32 one."""
    from nunchaku_rocm_amd import ops

    q = torch.randint(0, 16, (N, K), generator=torch.Generator().manual_seed(N), dtype=torch.int32)
    packed = O.awq_pack(q).to(dev)
    ones = torch.ones(K // group_size, N, dtype=dtype, device=dev)
    out = ops.awq_dequantize(packed, ones, torch.zeros_like(ones), N, K, group_size, dtype)
    assert torch.equal(out.float().cpu(), q.float())
    out32 = ops.awq_dequantize(packed.view(torch.int32), ones, torch.zeros_like(ones), N, K, group_size, dtype)
    assert torch.equal(out32, out)
