"""Run-time LoRA on single layers: the widened low-rank branch of an SVDQuant linear (ranks 32 + sum r, padded to a
multiple of 16) against the oracle on the concatenated factors, the base layer's bits restored on detach, and the
forward hook of layers without a low-rank branch."""

import pytest
import torch

from oracle import svdq_oracle as O

pytestmark = pytest.mark.gpu


def _module(dev, K, N):
    from nunchaku_rocm_amd.linear import SVDQW4A4Linear

    lin = O.make_svdq_linear(K, N, seed=5)
    mod = SVDQW4A4Linear(K, N, rank=32, device=dev)
    with torch.no_grad():
        for name in ("qweight", "wscales", "smooth_factor", "proj_down", "proj_up", "bias"):
            getattr(mod, name).copy_(lin[name])
    return mod, lin


@pytest.mark.parametrize("ranks", [(16,), (8, 20), (64, 64, 128)])
def test_attach_widens_the_low_rank_branch(dev, ranks):
    from nunchaku_rocm_amd.lora import attach_lora, detach_lora

    print(f"case ranks={ranks}", flush=True)
    K, N, M = 512, 384, 150
    mod, lin = _module(dev, K, N)
    x = O.make_activations(M, K, seed=6).view(1, M, K)
    base = mod(x.to(dev)).cpu()
    g = torch.Generator().manual_seed(sum(ranks))
    pairs = [((torch.randn(r, K, generator=g) * 0.05).to(torch.bfloat16), (torch.randn(N, r, generator=g) * 0.2).to(torch.bfloat16))
             for r in ranks]  # fmt: skip
    attach_lora(mod, pairs)
    R = 32 + sum(ranks)
    Rp = (R + 15) // 16 * 16
    assert mod.proj_down.shape == (K, Rp) and mod.proj_up.shape == (N, Rp) and mod.rank == Rp
    assert bool((mod.proj_down[:, R:] == 0).all()) and bool((mod.proj_up[:, R:] == 0).all())
    y = mod(x.to(dev)).cpu()
    down = torch.cat([lin["proj_down"]] + [d.t() for d, _ in pairs], 1)
    up = torch.cat([lin["proj_up"]] + [u for _, u in pairs], 1)
    rp, rs, rl, _ = O.quantize_act(x.view(-1, K), down, lin["smooth_factor"])
    ref = O.gemm_w4a4(rp, lin["qweight"], rs, lin["wscales"], lin["bias"], rl, up)
    assert O.max_rel_err(y.view(-1, N), ref) <= 1e-2
    # the added term is what the LoRAs compute on the unquantized activation (16-bit rounding of the hidden state aside)
    xd = x.view(-1, K).double()
    extra = sum((xd @ d.double().t()) @ u.double().t() for d, u in pairs)
    assert O.cosine((y.view(-1, N).double() - base.view(-1, N).double()), extra) > 0.99
    detach_lora(mod)
    assert mod.proj_down.shape == (K, 32) and mod.rank == 32
    assert torch.equal(mod(x.to(dev)).cpu(), base)
    detach_lora(mod)  # nothing attached: no-op


def test_hook_on_a_layer_without_low_rank_branch(dev):
    from nunchaku_rocm_amd.linear import AWQW4A16Linear
    from nunchaku_rocm_amd.lora import attach_lora, detach_lora

    K, N = 256, 128
    lin = O.make_awq_linear(K, N, seed=31)
    mod = AWQW4A16Linear(K, N, bias=False, device=dev)
    with torch.no_grad():
        mod.qweight.copy_(lin["qweight"])
        mod.wscales.copy_(lin["wscales"])
        mod.wzeros.copy_(lin["wzeros"])
    g = torch.Generator().manual_seed(3)
    x = torch.randn(2, K, generator=g).to(torch.bfloat16)
    d = (torch.randn(8, K, generator=g) * 0.05).to(torch.bfloat16)
    u = (torch.randn(N, 8, generator=g) * 0.2).to(torch.bfloat16)
    base = mod(x.to(dev)).cpu()
    attach_lora(mod, [(d, u)])
    y = mod(x.to(dev)).cpu()
    extra = (x.double() @ d.double().t()) @ u.double().t()
    assert O.max_rel_err((y.double() - base.double()).float(), extra.float()) <= 3e-2
    detach_lora(mod)
    assert torch.equal(mod(x.to(dev)).cpu(), base)
    with pytest.raises(NotImplementedError):
        attach_lora(mod, [((d, (3, 3)), u)])
