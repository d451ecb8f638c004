"""End-to-end: the FLUX.1-shaped transformer on the HIP operators against the same graph on the oracle operators.

Bar: cosine of the final latents >= 0.999 after the 4-step denoise (the two paths differ by 16-bit output rounding
and, after GELU, by codes that may be one step apart; every quantizer in between is a discontinuity, so this is a
statement about error growth through 57 blocks, not bit parity).
"""

import copy
import time

import pytest
import torch

from oracle import svdq_oracle as O
from oracle.flux_backend import OracleBackend

pytestmark = pytest.mark.gpu


def _inputs(cfg, t_txt, gh, gw, dev, seed=7, dtype=torch.bfloat16):
    from nunchaku_rocm_amd.flux_shaped import flux_ids, rope_table

    g = torch.Generator().manual_seed(seed)
    lat = torch.randn(1, gh * gw, cfg.in_channels, generator=g).to(dtype).to(dev)
    txt = torch.randn(1, t_txt, cfg.text_dim, generator=g).to(dtype).to(dev)
    pooled = torch.randn(1, cfg.pooled_dim, generator=g).to(dtype).to(dev)
    rot = rope_table(flux_ids(t_txt, gh, gw, device=dev), cfg.axes_dim, cfg.theta)
    return lat, txt, pooled, rot


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_small_config_against_cpu_oracle(dev, dtype):
    from nunchaku_rocm_amd.flux_shaped import FluxShapedConfig, FluxShapedTransformer

    cfg = FluxShapedConfig(hidden=512, heads=4, mlp=2048, text_dim=256, pooled_dim=64, n_double=2, n_single=3)
    model = FluxShapedTransformer(cfg, device=dev, dtype=dtype, seed=3)
    lat, txt, pooled, rot = _inputs(cfg, 32, 16, 16, dev, dtype=dtype)
    out = model.denoise(lat, txt, pooled, rot, steps=4).cpu()
    cpu_model = copy.deepcopy(model).to("cpu")
    ref = cpu_model.denoise(lat.cpu(), txt.cpu(), pooled.cpu(), rot.cpu(), steps=4, backend=OracleBackend())
    cos = O.cosine(out, ref)
    print(f"small config latent cosine {cos:.6f}", flush=True)
    assert torch.isfinite(out.float()).all()
    assert cos >= 0.999


def test_two_streams_give_the_same_bits(dev):
    """The text stream of the dual-stream blocks on a second HIP stream: every kernel is deterministic, so the result
    must be bit-equal to the single-stream run, on repeated runs too (a missed dependency would show up here)."""
    from nunchaku_rocm_amd.flux_shaped import FluxShapedConfig, FluxShapedTransformer, HipBackend

    cfg = FluxShapedConfig(hidden=1024, heads=8, mlp=4096, text_dim=256, pooled_dim=64, n_double=4, n_single=2)
    model = FluxShapedTransformer(cfg, device=dev, seed=5)
    lat, txt, pooled, rot = _inputs(cfg, 512, 32, 32, dev)
    one = model.denoise(lat, txt, pooled, rot, steps=2, backend=HipBackend(two_streams=False))
    torch.cuda.synchronize()
    two = HipBackend(two_streams=True)
    for _ in range(3):
        out = model.denoise(lat, txt, pooled, rot, steps=2, backend=two)
        torch.cuda.synchronize()
        assert torch.equal(out, one)


def test_flux1_schnell_shape_four_steps(dev):
    """19 double + 38 single blocks, hidden 3072, 4096 image + 512 text tokens, 4 steps; the reference path is the
    oracle's dense-dequantised fp32 formulation evaluated with plain torch kernels on the same GPU."""
    from nunchaku_rocm_amd.flux_shaped import FluxShapedConfig, FluxShapedTransformer

    cfg = FluxShapedConfig()
    print("building the random-init FLUX.1-shaped model", flush=True)
    model = FluxShapedTransformer(cfg, device=dev, seed=0)
    lat, txt, pooled, rot = _inputs(cfg, 512, 64, 64, dev)
    model.denoise(lat, txt, pooled, rot, steps=1)  # warm-up (weight re-layout caches, allocator)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    out = model.denoise(lat, txt, pooled, rot, steps=4)
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / 4
    print(f"HIP path: {dt:.4f} s/step", flush=True)
    assert torch.isfinite(out.float()).all()
    prev = torch.backends.cuda.matmul.allow_tf32
    torch.backends.cuda.matmul.allow_tf32 = False
    try:
        t0 = time.perf_counter()
        ref = model.denoise(lat, txt, pooled, rot, steps=4, backend=OracleBackend(dense=True))
        torch.cuda.synchronize()
        print(f"oracle (dense fp32 torch on GPU): {(time.perf_counter() - t0) / 4:.3f} s/step", flush=True)
    finally:
        torch.backends.cuda.matmul.allow_tf32 = prev
    cos = O.cosine(out, ref)
    print(f"FLUX.1-shaped 4-step latent cosine {cos:.6f}", flush=True)
    assert cos >= 0.999


def test_relayout_made_on_one_stream_is_ordered_before_its_use_on_another(dev):
    """The cached weight re-layouts are launched on the stream of their first use; a first use elsewhere right after
    must wait for them (same bits as a run where everything happens on one stream)."""
    from nunchaku_rocm_amd.linear import SVDQW4A4Linear

    K, N, M = 3072, 3072, 512
    lin = O.make_svdq_linear(K, N, seed=9)
    x = O.make_activations(M, K, seed=10).view(1, M, K).to(dev)

    def fresh():
        mod = SVDQW4A4Linear(K, N, rank=32, device=dev)
        with torch.no_grad():
            for name in ("qweight", "wscales", "smooth_factor", "proj_down", "proj_up", "bias"):
                getattr(mod, name).copy_(lin[name])
        return mod

    ref = fresh()(x)
    torch.cuda.synchronize()
    mod = fresh()
    side = torch.cuda.Stream()
    busy = torch.empty(64 << 20, device=dev)
    torch.cuda.synchronize()
    for _ in range(8):
        busy.normal_()  # keeps the main stream busy, so the re-layouts queued behind it are still pending below
    y_main = mod(x)  # first use: re-layouts and this call on the main stream
    with torch.cuda.stream(side):
        y_side = mod(x)  # cache hits on another stream
    torch.cuda.synchronize()
    assert torch.equal(y_main, ref) and torch.equal(y_side, ref)
