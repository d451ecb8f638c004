"""Low-rank branch widened at run time: ranks 32 + sum r (padded to a multiple of 16) through the same two kernels,
against the oracle on the concatenated factors; swapping one set of factors for another of the same rank (the
re-laid-out copy of ``proj_down`` must follow); the base layer's bits restored when the original tensors come back.
The reference's own ``attach_lora`` (nunchaku/lora/runtime.py:476-525) does exactly this to the two parameters."""

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


def _factors(K, N, ranks, seed):
    g = torch.Generator().manual_seed(seed)
    return [((torch.randn(r, K, generator=g) * 0.05).to(torch.bfloat16), (torch.randn(N, r, generator=g) * 0.2).to(torch.bfloat16))
            for r in ranks]  # fmt: skip


def _widen(mod, lin, pairs, dev):
    """What a run-time LoRA loader does to the layer: append the factors to the two low-rank parameters, zero-padded
    to a multiple of 16, by assigning ``.data``."""
    down = torch.cat([lin["proj_down"]] + [d.t() for d, _ in pairs], 1)
    up = torch.cat([lin["proj_up"]] + [u for _, u in pairs], 1)
    R = down.shape[1]
    pad = -R % 16
    if pad:
        down = torch.cat([down, down.new_zeros(down.shape[0], pad)], 1)
        up = torch.cat([up, up.new_zeros(up.shape[0], pad)], 1)
    mod.proj_down.data = down.to(dev).contiguous()
    mod.proj_up.data = up.to(dev).contiguous()
    mod.rank = R + pad
    return down, up


@pytest.mark.parametrize("ranks", [(16,), (8, 20), (64, 64, 128)])
def test_widened_low_rank_branch(dev, ranks):
    print(f"case ranks={ranks}", flush=True)
    K, N, M = 512, 384, 150
    mod, lin = _module(dev, K, N)
    x = O.make_activations(M, K, seed=6).view(1, M, K)
    base = mod(x.to(dev)).cpu()
    pairs = _factors(K, N, ranks, seed=sum(ranks))
    down, up = _widen(mod, lin, pairs, dev)
    y = mod(x.to(dev)).cpu()
    rp, rs, rl, _ = O.quantize_act(x.view(-1, K), down, lin["smooth_factor"])
    ref = O.gemm_w4a4(rp, lin["qweight"], rs, lin["wscales"], lin["bias"], rl, up)
    assert O.max_rel_err(y.view(-1, N), ref) <= 1e-2
    # the added term is what the LoRAs compute on the unquantized activation (16-bit rounding of the hidden state aside)
    xd = x.view(-1, K).double()
    extra = sum((xd @ d.double().t()) @ u.double().t() for d, u in pairs)
    assert O.cosine((y.view(-1, N).double() - base.view(-1, N).double()), extra) > 0.99
    # back to the base tensors: the base layer's bits
    mod.proj_down.data = lin["proj_down"].to(dev)
    mod.proj_up.data = lin["proj_up"].to(dev)
    mod.rank = 32
    assert torch.equal(mod(x.to(dev)).cpu(), base)


def test_swapping_factors_of_the_same_rank(dev):
    """Assigning ``.data`` changes neither the parameter object nor its version counter, and the allocator likes to hand
    the block just freed to the next tensor of the same size: the cached transposed ``proj_down`` must not survive it."""
    K, N, M = 512, 384, 150
    mod, lin = _module(dev, K, N)
    x = O.make_activations(M, K, seed=7).view(1, M, K)
    for round_, seed in enumerate((11, 12, 13)):
        pairs = _factors(K, N, (16,), seed=seed)
        down, up = _widen(mod, lin, pairs, dev)
        y = mod(x.to(dev)).cpu()
        rp, rs, rl, _ = O.quantize_act(x.view(-1, K), down, lin["smooth_factor"])
        ref = O.gemm_w4a4(rp, lin["qweight"], rs, lin["wscales"], lin["bias"], rl, up)
        assert O.max_rel_err(y.view(-1, N), ref) <= 1e-2, f"round {round_}: stale low-rank factors"
        # the quantizer's LoRA hidden state itself, not just the output
        from nunchaku_rocm_amd import ops

        _, _, la = ops.svdq_quantize_w4a4_act_fuse_lora_cuda(x.view(-1, K).to(dev), lora_down=mod.proj_down,
                                                             smooth=mod.smooth_factor)  # fmt: skip
        assert O.max_rel_err(la[:M].cpu(), rl) <= 1e-2, f"round {round_}: LoRA-down read a stale transposed copy"
