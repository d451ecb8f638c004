"""A forward pass recorded into a HIP graph: every replay gives the bits of the eager pass."""

import time

import pytest
import torch

pytestmark = pytest.mark.gpu


def _inputs(cfg, t_txt, gh, gw, dev, seed=0):
    from nunchaku_rocm_amd.flux_shaped import flux_ids, rope_table

    g = torch.Generator(device=dev).manual_seed(seed)
    lat = torch.randn(1, gh * gw, cfg.in_channels, device=dev, generator=g).to(torch.bfloat16)
    txt = torch.randn(1, t_txt, cfg.text_dim, device=dev, generator=g).to(torch.bfloat16)
    pooled = torch.randn(1, cfg.pooled_dim, device=dev, generator=g).to(torch.bfloat16)
    rot = rope_table(flux_ids(t_txt, gh, gw, device=dev), cfg.axes_dim, cfg.theta)
    return lat, txt, pooled, rot


def test_graph_replays_equal_eager(dev):
    from nunchaku_rocm_amd.flux_shaped import FluxShapedConfig, FluxShapedTransformer

    cfg = FluxShapedConfig(hidden=1024, heads=8, mlp=4096, text_dim=256, pooled_dim=64, n_double=3, n_single=3)
    model = FluxShapedTransformer(cfg, device=dev, seed=5)
    lat, txt, pooled, rot = _inputs(cfg, 512, 32, 32, dev)
    print("capturing", flush=True)
    step = model.capture(lat, txt, pooled, rot)
    print("captured", flush=True)
    g = torch.Generator(device=dev).manual_seed(1)
    for i, tval in enumerate((1.0, 0.75, 0.3, 0.05)):
        x = torch.randn(lat.shape, device=dev, generator=g).to(torch.bfloat16)
        t = torch.full((1,), tval, device=dev)
        eager = model.forward(x, txt, pooled, t, rot)
        torch.cuda.synchronize()
        got = step(x, t).clone()
        torch.cuda.synchronize()
        assert torch.equal(got, eager), f"replay {i}"
        print(f"replay {i} ok", flush=True)
    a = model.denoise(lat, txt, pooled, rot, steps=3)
    b = model.denoise(lat, txt, pooled, rot, steps=3, step_fn=step)
    torch.cuda.synchronize()
    assert torch.equal(a, b)
