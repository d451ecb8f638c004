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


# harness names -> nunchaku model names -> legacy checkpoint names: the inverse of what the loader applies
_TO_MODEL = (
    ("double_blocks.", "transformer_blocks."), ("single_blocks.", "single_transformer_blocks."),
    (".norm1_context.", ".norm1_context.linear."), (".norm1.", ".norm1.linear."), (".norm.", ".norm.linear."),
    (".ffc_fc1.", ".ff_context.net.0.proj."), (".ffc_fc2.", ".ff_context.net.2."),
    (".ff_fc1.", ".ff.net.0.proj."), (".ff_fc2.", ".ff.net.2."),
    ("time_in.0.", "time_text_embed.timestep_embedder.linear_1."), ("time_in.2.", "time_text_embed.timestep_embedder.linear_2."),
    ("pooled_in.0.", "time_text_embed.text_embedder.linear_1."), ("pooled_in.2.", "time_text_embed.text_embedder.linear_2."),
    ("norm_out_linear.", "norm_out.linear."),
)  # fmt: skip
_TO_LEGACY_DOUBLE = (
    (".ff_context.net.0.proj.", ".mlp_context_fc1."), (".ff_context.net.2.", ".mlp_context_fc2."),
    (".ff.net.0.proj.", ".mlp_fc1."), (".ff.net.2.", ".mlp_fc2."),
    (".attn.add_qkv_proj.", ".qkv_proj_context."), (".attn.to_qkv.", ".qkv_proj."),
    (".attn.to_add_out.", ".out_proj_context."), (".attn.to_out.", ".out_proj."),
    (".attn.norm_added_q.", ".norm_added_q."), (".attn.norm_added_k.", ".norm_added_k."),
    (".attn.norm_q.", ".norm_q."), (".attn.norm_k.", ".norm_k."),
)  # fmt: skip
_TO_LEGACY_SINGLE = (
    (".attn.to_qkv.", ".qkv_proj."), (".attn.to_out.", ".out_proj."), (".attn.norm_q.", ".norm_q."), (".attn.norm_k.", ".norm_k."),
)  # fmt: skip


def _legacy_key(name: str) -> str:
    for old, new in _TO_MODEL:
        name = name.replace(old, new)
    if name.startswith("transformer_blocks."):
        for old, new in _TO_LEGACY_DOUBLE:
            if old in name:
                name = name.replace(old, new)
                break
    elif name.startswith("single_transformer_blocks."):
        for old, new in _TO_LEGACY_SINGLE:
            if old in name:
                name = name.replace(old, new)
                break
    name = name.replace(".proj_down", ".lora_down").replace(".proj_up", ".lora_up")
    if name.endswith(".smooth_factor"):
        name = name[: -len(".smooth_factor")] + ".smooth"
    return name


def test_converted_checkpoint_runs(dev, tmp_path):
    """A model written out the way the published int4 checkpoints are stored -- legacy module names, every SVDQuant tensor
    shuffled into the mma fragment order by the packer restatement, one ``.safetensors`` file -- read back through
    ``layout.load_checkpoint``, ``convert_flux_state_dict`` and ``FluxShapedTransformer.load_converted`` computes the
    same bits as the model it was written from (reference: transformer_flux_v2.py:375-435)."""
    from safetensors.torch import save_file

    from nunchaku_rocm_amd import layout
    from nunchaku_rocm_amd.flux_shaped import FluxShapedConfig, FluxShapedTransformer
    from nunchaku_rocm_amd.linear import SVDQW4A4Linear
    from oracle import mma_packer as P

    cfg = FluxShapedConfig(hidden=256, heads=2, mlp=512, text_dim=128, pooled_dim=64, n_double=2, n_single=2)
    src = FluxShapedTransformer(cfg, device=dev, seed=11)
    svdq = {n for n, m in src.named_modules() if isinstance(m, SVDQW4A4Linear)}
    as16 = lambda t: t.detach().cpu().contiguous().view(torch.int16).numpy()  # noqa: E731
    bf = lambda a: torch.from_numpy(a).view(torch.bfloat16)  # noqa: E731
    ckpt = {}
    for name, t in src.state_dict().items():
        mod, leaf = name.rsplit(".", 1) if "." in name else ("", name)
        t = t.detach().cpu()
        if mod in svdq:
            if leaf == "smooth_factor_orig":
                continue
            if leaf == "qweight":
                codes = O.unpack_int4(t, signed=False).to(torch.int32)
                t = torch.from_numpy(P.pack_weight(codes.numpy())).view(torch.int8)
            elif leaf == "wscales":
                t = bf(P.pack_scale(as16(t.t()))).reshape(t.shape)
            elif leaf in ("bias", "smooth_factor"):
                t = bf(P.pack_scale(as16(t)))
            elif leaf == "proj_down":
                t = bf(P.pack_lowrank_weight(as16(t.t()), down=True))
            elif leaf == "proj_up":
                t = bf(P.pack_lowrank_weight(as16(t), down=False))
        ckpt[_legacy_key(name)] = t.contiguous()
    assert any(".qkv_proj_context.lora_down" in k for k in ckpt) and any(k.endswith(".mlp_fc2.smooth") for k in ckpt)
    path = tmp_path / "svdq-int4-flux-shaped.safetensors"
    save_file(ckpt, str(path), metadata={"config": "{\"num_layers\": 2}", "quantization_config": "{\"rank\": 32}"})

    state, meta, config = layout.load_checkpoint(path)
    assert config == {"num_layers": 2} and "quantization_config" in meta
    dst = FluxShapedTransformer(cfg, device=dev, seed=99)  # other weights: everything must come from the file
    dst.load_converted(layout.convert_flux_state_dict(state))
    for (n1, t1), (n2, t2) in zip(src.state_dict().items(), dst.state_dict().items()):
        if n1.endswith("smooth_factor_orig"):
            continue
        assert n1 == n2 and torch.equal(t1.view(torch.uint8), t2.view(torch.uint8)), n1
    lat, txt, pooled, rot = _inputs(cfg, 32, 16, 16, dev)
    a = src.denoise(lat, txt, pooled, rot, steps=2)
    b = dst.denoise(lat, txt, pooled, rot, steps=2)
    torch.cuda.synchronize()
    assert torch.equal(a, b)
    # a file that lacks a tensor, or brings one with no place, is refused
    broken = dict(layout.convert_flux_state_dict(state))
    broken.pop("transformer_blocks.0.attn.to_qkv.qweight")
    with pytest.raises(KeyError):
        dst.load_converted(broken)
