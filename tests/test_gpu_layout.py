"""GPU parity of checkpoint ingestion (bit-exact permutations): the device unpackers invert the CPU restatement of the
checkpoint packer, and a module loaded in checkpoint layout computes what its logical tensors say
(reference tests: tests/triton/test_layout.py:19-60, :80-153)."""

import numpy as np
import pytest
import torch

from oracle import mma_packer as P
from oracle import svdq_oracle as O

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("n,k", [(128, 128), (256, 256), (128, 512), (384, 128), (3072, 3072)])
def test_unpack_weight_int4(dev, n, k):
    from nunchaku_rocm_amd import layout

    print(f"case n={n} k={k}", flush=True)
    w = torch.randint(0, 16, (n, k), dtype=torch.int32, generator=torch.Generator().manual_seed(n + k))
    packed = torch.from_numpy(P.pack_weight(w.numpy())).view(torch.int8).to(dev)
    assert torch.equal(layout.unpack_weight(packed, n, k).cpu(), w)
    nib = layout.unpack_weight_packed_nibbles(packed, n, k).cpu()
    assert nib.dtype == torch.uint8 and torch.equal(nib, O.pack_int4(w))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("n", [128, 256, 9216])
def test_unpack_scale_per_channel(dev, n, dtype):
    from nunchaku_rocm_amd import layout

    s = torch.randn(n, generator=torch.Generator().manual_seed(n)).to(dtype)
    packed = torch.from_numpy(P.pack_scale(s.view(torch.int16).numpy())).view(dtype).to(dev)
    got = layout.unpack_scale(packed, n, group_size=-1)
    assert got.shape == (n,) and torch.equal(got.cpu().view(torch.int16), s.view(torch.int16))


@pytest.mark.parametrize("n,k", [(128, 256), (256, 512), (9216, 3072)])
def test_unpack_scale_grouped(dev, n, k):
    from nunchaku_rocm_amd import layout

    s = torch.randn(n, k // 64, generator=torch.Generator().manual_seed(k)).to(torch.bfloat16)
    packed = torch.from_numpy(P.pack_scale(s.view(torch.int16).numpy())).view(torch.bfloat16).reshape(-1, n).to(dev)
    got = layout.unpack_scale(packed, n, group_size=64)
    assert got.shape == (k // 64, n) and torch.equal(got.cpu().view(torch.int16), s.t().contiguous().view(torch.int16))


@pytest.mark.parametrize("c,r", [(128, 32), (3072, 32), (256, 160), (48, 16)])
def test_unpack_lowrank(dev, c, r):
    from nunchaku_rocm_amd import layout

    g = torch.Generator().manual_seed(c + r)
    up = torch.randn(c, r, generator=g).to(torch.bfloat16)
    packed = torch.from_numpy(P.pack_lowrank_weight(up.view(torch.int16).numpy(), down=False)).view(torch.bfloat16).to(dev)
    assert torch.equal(layout.unpack_lowrank_weight(packed, down=False).cpu().view(torch.int16), up.view(torch.int16))
    down = torch.randn(c, r, generator=g).to(torch.bfloat16)  # logical proj_down (in_features, rank)
    packed = torch.from_numpy(P.pack_lowrank_weight(down.t().contiguous().view(torch.int16).numpy(), down=True)).view(torch.bfloat16).to(dev)
    assert packed.shape == (c, r)
    assert torch.equal(layout.unpack_lowrank_weight(packed, down=True).cpu().view(torch.int16), down.view(torch.int16))


def test_convert_linear_and_forward(dev):
    """A module filled in checkpoint layout, converted in place, then run: tensors decode to the logical values and the
    forward pass matches the oracle on those logical values."""
    from nunchaku_rocm_amd import layout
    from nunchaku_rocm_amd.linear import SVDQW4A4Linear

    K, N, R = 256, 128, 32
    lin = O.make_svdq_linear(K, N, R=R, seed=5)
    mod = SVDQW4A4Linear(K, N, rank=R, device=dev)
    codes = O.unpack_int4(lin["qweight"], signed=False).to(torch.int32)
    as16 = lambda t: t.contiguous().view(torch.int16).numpy()  # noqa: E731
    bf = lambda a: torch.from_numpy(a).view(torch.bfloat16)  # noqa: E731
    with torch.no_grad():
        mod.qweight.data = torch.from_numpy(P.pack_weight(codes.numpy())).view(torch.int8).to(dev)
        mod.wscales.data = bf(P.pack_scale(as16(lin["wscales"].t()))).reshape(-1, N).to(dev)
        mod.bias.data = bf(P.pack_scale(as16(lin["bias"]))).to(dev)
        mod.smooth_factor.data = bf(P.pack_scale(as16(lin["smooth_factor"]))).to(dev)
        mod.proj_down.data = bf(P.pack_lowrank_weight(as16(lin["proj_down"].t()), down=True)).to(dev)
        mod.proj_up.data = bf(P.pack_lowrank_weight(as16(lin["proj_up"]), down=False)).to(dev)
    assert not torch.equal(mod.qweight.data.cpu().view(torch.uint8), lin["qweight"].view(torch.uint8))
    layout.convert_svdq_linear_to_natural_layout(mod)
    for name in ("wscales", "bias", "smooth_factor", "proj_down", "proj_up"):
        assert torch.equal(getattr(mod, name).data.cpu().view(torch.int16), lin[name].view(torch.int16)), name
    assert torch.equal(mod.qweight.data.cpu().view(torch.uint8), lin["qweight"].view(torch.uint8))
    x = O.make_activations(40, K, seed=6)
    y = mod(x.to(dev)[None])[0].cpu()
    qx, sc, la, _ = O.quantize_act(x, lin["proj_down"], lin["smooth_factor"])
    ref = O.gemm_w4a4(qx, lin["qweight"], sc, lin["wscales"], lin["bias"], la, lin["proj_up"])[:40]
    assert O.max_rel_err(y, ref) <= 1e-2


def test_bad_shapes_are_rejected(dev):
    from nunchaku_rocm_amd import layout

    with pytest.raises(ValueError):
        layout.unpack_weight_packed_nibbles(torch.zeros(64, 64, dtype=torch.int8, device=dev), 64, 128)  # n % 128
    with pytest.raises(ValueError):
        layout.unpack_scale(torch.zeros(100, dtype=torch.bfloat16, device=dev), 100, group_size=-1)
    with pytest.raises(ValueError):
        layout.unpack_lowrank_weight(torch.zeros(24, 16, dtype=torch.bfloat16, device=dev), down=False)
