"""GPU parity of the unmasked attention kernel against the CPU oracle (floating point: max |err| / max |ref| <= 1e-2
per call, and the reference's own bound of rtol = atol = 3e-2 against fp32 attention,
tests/triton/test_w4a4.py:241-254, tests/triton/test_backend.py:75-106)."""

import pytest
import torch

from oracle import svdq_oracle as O

pytestmark = pytest.mark.gpu

TOL = 1e-2


def _inputs(B, H, Tq, Tkv, dtype, seed, spread=1.0, D=128):
    g = torch.Generator().manual_seed(seed)
    q = (torch.randn(B, H, Tq, D, generator=g) * spread).to(dtype)
    k = (torch.randn(B, H, Tkv, D, generator=g) * spread).to(dtype)
    v = torch.randn(B, H, Tkv, D, generator=g).to(dtype)
    return q, k, v


def _run(dev, q, k, v, scale):
    from nunchaku_rocm_amd import ops

    B, H, Tq, D = q.shape
    o = torch.full((B, Tq, H * D), float("nan"), dtype=q.dtype, device=dev)
    ops.attention_fp16(q.to(dev), k.to(dev), v.to(dev), o, scale)
    torch.cuda.synchronize()
    return o.cpu()


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize(
    "B,H,Tq,Tkv",
    [(1, 4, 128, 512), (2, 2, 100, 77), (2, 4, 300, 300), (1, 1, 1, 1), (1, 2, 129, 63), (1, 2, 7, 64), (1, 3, 257, 65), (3, 1, 64, 1000)],
)
def test_against_oracle(dev, dtype, B, H, Tq, Tkv):
    print(f"case {B}x{H}x{Tq}x{Tkv} {dtype}", flush=True)
    q, k, v = _inputs(B, H, Tq, Tkv, dtype, seed=Tq * 7 + Tkv)
    scale = 128**-0.5
    out = _run(dev, q, k, v, scale)
    ref = O.attention_fp16(q, k, v, scale)
    assert out.shape == ref.shape and out.dtype == dtype
    assert torch.isfinite(out.float()).all()
    assert O.max_rel_err(out, ref) <= TOL
    exact = torch.softmax(q.float() @ k.float().transpose(-1, -2) * scale, dim=-1) @ v.float()
    torch.testing.assert_close(out.float(), exact.transpose(1, 2).reshape(B, Tq, -1), rtol=3e-2, atol=3e-2)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("B,H,Tq,Tkv", [(2, 8, 256, 256), (2, 2, 100, 77), (1, 3, 129, 65), (1, 1, 1, 1), (1, 16, 333, 1000)])
def test_head_dimension_64(dev, dtype, B, H, Tq, Tkv):
    """The reference's own test shapes with 64-dimensional heads (tests/triton/test_w4a4.py:242) and ragged ones."""
    print(f"case D=64 {B}x{H}x{Tq}x{Tkv} {dtype}", flush=True)
    q, k, v = _inputs(B, H, Tq, Tkv, dtype, seed=Tq + 3 * Tkv, D=64)
    scale = 64**-0.5
    out = _run(dev, q, k, v, scale)
    ref = O.attention_fp16(q, k, v, scale)
    assert out.shape == (B, Tq, H * 64) and torch.isfinite(out.float()).all()
    assert O.max_rel_err(out, ref) <= TOL
    exact = torch.softmax(q.float() @ k.float().transpose(-1, -2) * scale, dim=-1) @ v.float()
    torch.testing.assert_close(out.float(), exact.transpose(1, 2).reshape(B, Tq, -1), rtol=3e-2, atol=3e-2)
    # a sharp softmax moves the reference every tile
    q2 = (q.float() * 6).to(dtype)
    assert O.max_rel_err(_run(dev, q2, k, v, scale), O.attention_fp16(q2, k, v, scale)) <= TOL


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_moving_maximum_and_other_scale(dev, dtype):
    """Scores that grow along the keys make every block move the running maximum; a non-default scale is honoured."""
    q, k, v = _inputs(1, 2, 96, 640, dtype, seed=3, spread=1.0)
    k = (k.float() * torch.linspace(0.2, 4.0, 640)[None, None, :, None]).to(dtype)
    for scale in (128**-0.5, 0.2):
        print(f"case scale={scale} {dtype}", flush=True)
        out = _run(dev, q, k, v, scale)
        assert O.max_rel_err(out, O.attention_fp16(q, k, v, scale)) <= TOL


def test_dominant_key_selects_its_value_row(dev):
    """One key dominates each query (a different one per query and head): the output row is that key's v."""
    H, Tq, Tkv = 2, 40, 200
    q = torch.zeros(1, H, Tq, 128)
    k = torch.zeros(1, H, Tkv, 128)
    v = torch.randn(1, H, Tkv, 128, generator=torch.Generator().manual_seed(1)).half()
    pick = torch.zeros(H, Tq, dtype=torch.long)
    for t in range(Tq):
        q[0, :, t, t] = 60.0
        pick[0, t], pick[1, t] = 3 * t + 1, Tkv - 1 - 4 * t
        k[0, 0, pick[0, t], t] = 60.0
        k[0, 1, pick[1, t], t] = 60.0
    out = _run(dev, q.half(), k.half(), v, 128**-0.5).float()
    for h in range(H):
        assert torch.allclose(out[0, :, 128 * h : 128 * (h + 1)], v[0, h, pick[h]].float(), atol=1e-3)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("layout", ["bhtd", "bthd_view"])
def test_sdpa_wrapper(dev, dtype, layout):
    """The drop-in for F.scaled_dot_product_attention: both layouts; a mask goes to torch instead of being ignored."""
    from nunchaku_rocm_amd import ops

    print(f"case {layout} {dtype}", flush=True)
    B, H, T, D = 2, 4, 300, 128
    g = torch.Generator().manual_seed(11)
    if layout == "bhtd":
        q, k, v = (torch.randn(B, H, T, D, generator=g).to(dtype).to(dev) for _ in range(3))
    else:
        q, k, v = (torch.randn(B, T, H, D, generator=g).to(dtype).to(dev).transpose(1, 2) for _ in range(3))
    out = ops.scaled_dot_product_attention(q, k, v)
    ref = torch.nn.functional.scaled_dot_product_attention(q.float(), k.float(), v.float())
    assert out.shape == ref.shape
    torch.testing.assert_close(out.float(), ref, rtol=3e-2, atol=3e-2)
    assert O.max_rel_err(out.transpose(1, 2).reshape(B, T, H * D).cpu(), O.attention_fp16(q.cpu(), k.cpu(), v.cpu(), D**-0.5)) <= TOL
    mask = torch.rand(B, 1, T, T, device=dev) > 0.5
    mask[..., 0] = True
    out = ops.scaled_dot_product_attention(q, k, v, attn_mask=mask)
    ref = torch.nn.functional.scaled_dot_product_attention(q.float(), k.float(), v.float(), attn_mask=mask)
    torch.testing.assert_close(out.float(), ref, rtol=3e-2, atol=3e-2)
    # head dimension 64 runs on the kernel too (here on strided slices of the 128-wide tensors)
    out = ops.scaled_dot_product_attention(q[..., :64], k[..., :64], v[..., :64])
    ref = torch.nn.functional.scaled_dot_product_attention(q[..., :64].float(), k[..., :64].float(), v[..., :64].float())
    torch.testing.assert_close(out.float(), ref, rtol=3e-2, atol=3e-2)
    # head dimension 32 is outside the kernel: the wrapper goes to torch, the bare operator says so
    q32, k32, v32 = (t[..., :32].contiguous() for t in (q, k, v))
    out = ops.scaled_dot_product_attention(q32, k32, v32)
    ref = torch.nn.functional.scaled_dot_product_attention(q32.float(), k32.float(), v32.float())
    torch.testing.assert_close(out.float(), ref, rtol=3e-2, atol=3e-2)
    with pytest.raises(NotImplementedError):
        ops.attention_fp16(q32, k32, v32, torch.empty(B, T, H * 32, dtype=dtype, device=dev), 0.125)


def test_flux_shape_sampled_queries(dev):
    """The FLUX.1 joint-attention shape (24 heads, 512 + 4096 tokens), q / k / v as strided views of one fused
    (tokens, 3 * 3072) projection as the model holds them; every 41st query row is checked against the oracle."""
    from nunchaku_rocm_amd import ops

    T, H = 4608, 24
    g = torch.Generator().manual_seed(23)
    qkv = torch.randn(1, T, 3 * H * 128, generator=g).to(torch.bfloat16)
    q, k, v = (qkv[..., i * H * 128 : (i + 1) * H * 128].view(1, T, H, 128).transpose(1, 2) for i in range(3))
    qkv_d = qkv.to(dev)
    qd, kd, vd = (qkv_d[..., i * H * 128 : (i + 1) * H * 128].view(1, T, H, 128).transpose(1, 2) for i in range(3))
    o = torch.empty(1, T, H * 128, dtype=torch.bfloat16, device=dev)
    ops.attention_fp16(qd, kd, vd, o, 128**-0.5)
    torch.cuda.synchronize()
    rows = torch.arange(0, T, 41)
    ref = O.attention_fp16(q[:, :, rows], k, v, 128**-0.5)
    assert O.max_rel_err(o.cpu()[:, rows], ref) <= TOL
    # linearity in v (holds for any weights): attention(q, k, 2 v) = 2 attention(q, k, v), exactly in binary fp
    o2 = torch.empty_like(o)
    ops.attention_fp16(qd, kd, (vd * 2).contiguous(), o2, 128**-0.5)
    assert torch.equal(o2.float(), o.float() * 2)


def test_full_size_invariants(dev):
    """Properties that hold at any size, on the FLUX shape (24 heads, 4608 tokens, D = 128) entirely on the GPU:
    doubling v doubles the output exactly; a permutation of the queries permutes the output rows bit for bit; a
    permutation of the keys (with their values) changes only the order of the fp32 sums."""
    from nunchaku_rocm_amd import ops

    B, H, T, D = 1, 24, 4608, 128
    g = torch.Generator(device=dev).manual_seed(21)
    q = torch.randn(B, H, T, D, generator=g, device=dev).to(torch.bfloat16)
    k = torch.randn(B, H, T, D, generator=g, device=dev).to(torch.bfloat16)
    v = torch.randn(B, H, T, D, generator=g, device=dev).to(torch.bfloat16)
    scale = D**-0.5

    def run(q, k, v):
        o = torch.empty(B, q.shape[2], H * D, dtype=q.dtype, device=dev)
        ops.attention_fp16(q, k, v, o, scale)
        return o

    base = run(q, k, v)
    assert bool(torch.isfinite(base.float()).all())
    assert torch.equal(run(q, k, v * 2), base * 2)
    pq = torch.randperm(T, generator=g, device=dev)
    moved = run(q[:, :, pq].contiguous(), k, v)
    err_q = float((moved.float() - base[:, pq].float()).abs().max()) / float(base.float().abs().max())
    pk = torch.randperm(T, generator=g, device=dev)
    shuffled = run(q, k[:, :, pk].contiguous(), v[:, :, pk].contiguous())
    err_k = float((shuffled.float() - base.float()).abs().max()) / float(base.float().abs().max())
    print(f"query permutation: max rel diff {err_q:.2e}; key permutation: {err_k:.2e}", flush=True)
    assert err_q == 0.0 and err_k <= TOL  # query rows are computed independently of each other
    # each output row is a convex combination of value rows
    vmax = v.float().abs().amax(dim=2)  # (B, H, D)
    assert bool((base.view(B, T, H, D).float().abs() <= vmax[:, None] * (1 + 2**-6)).all())
