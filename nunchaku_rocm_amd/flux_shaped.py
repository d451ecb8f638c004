"""FLUX.1-shaped transformer (diffusers-free) wired to the SVDQuant operators.

Same dataflow as the reference's ``NunchakuFluxTransformer2DModelV2`` (nunchaku/models/transformers/
transformer_flux_v2.py:144-343 blocks, :437-576 forward; nunchaku/models/normalization.py:85-98,155-165 adaLN with
the interleaved 6-/3-way split and ``scale_shift = 0``; nunchaku/models/attention_processors/flux.py:62-109 attention;
nunchaku/models/embeddings.py:11-97 rotary table): 19 double-stream + 38 single-stream blocks, hidden 3072, 24 heads
x 128, MLP 12288, all block linears ``SVDQW4A4Linear`` (fused QKV + RMSNorm + RoPE, fused GELU MLP with unsigned fc2
activations, plain out-projections) and all modulation linears ``AWQW4A16Linear``.  The sub-modules the reference
inherits from diffusers (embedders, timestep/pooled-text MLPs, final AdaLayerNormContinuous + projection) are plain
bf16 torch layers here.  Weights are random-init in the natural layout: there is no checkpoint to load offline.

The quantized operators are reached through a small backend object (default: the HIP operators of this package), so a
test can run the identical graph on another implementation of the same four operators.
"""

from __future__ import annotations

import math
from dataclasses import dataclass

import torch
import torch.nn.functional as F
from torch import nn

from . import ops as _ops
from .linear import AWQW4A16Linear, SVDQW4A4Linear


@dataclass
class FluxShapedConfig:
    hidden: int = 3072
    heads: int = 24
    head_dim: int = 128
    mlp: int = 12288
    in_channels: int = 64
    text_dim: int = 4096
    pooled_dim: int = 768
    n_double: int = 19
    n_single: int = 38
    axes_dim: tuple = (16, 56, 56)
    theta: float = 10000.0
    rank: int = 32


class HipBackend:
    """The product path: every call lands in ``libsvdq_mi355x.so``."""

    @staticmethod
    def linear(x, lin: SVDQW4A4Linear):
        return lin(x)

    # mod = (scale, shift[, stats]): the block's LayerNorm + adaLN modulate of x, applied inside the quantizer
    @staticmethod
    def gelu_mlp(x, fc1, fc2, mod=None):
        return _ops.fused_gelu_mlp(x, fc1, fc2, norm=mod)

    writes_in_place = True  # qkv(out=...) stores straight into a caller's (tokens, 3 C) buffer

    def __init__(self, two_streams: bool = True):
        # The text stream of a dual-stream block is 512 tokens: its GEMMs cover a fraction of the 256 CUs (96 to 288
        # tiles for 512 workgroup slots).  Run on a second HIP stream (default priority) they fill the slots the image
        # stream's launches leave empty instead of queueing behind them.
        self.two_streams = two_streams
        self._side = {}
        self._awq_plans = {}

    def __deepcopy__(self, memo):
        return HipBackend(self.two_streams)  # streams are per process, not part of a model copy

    def side_stream(self, device):
        if not self.two_streams:
            return None
        key = torch.device(device).index
        if key not in self._side:
            self._side[key] = torch.cuda.Stream(device)
        return self._side[key]

    def join(self, device):
        """Make the current stream wait for everything queued on the side stream."""
        side = self._side.get(torch.device(device).index)
        if side is not None:
            torch.cuda.current_stream(device).wait_stream(side)

    @staticmethod
    def qkv(x, proj, norm_q, norm_k, rot, mod=None, out=None):
        return _ops.fused_qkv_norm_rottary(x, proj, norm_q, norm_k, rot, output=out, norm=mod)

    @staticmethod
    def gated_residual(x, gate, y, y2=None, want_stats=False, clip=0.0):
        """``(x + gate[:, None] * (y [+ y2]), row statistics of the result or None)``; ``clip``: limit of the result"""
        return _ops.gated_residual(x, gate, y, y2, want_stats=want_stats, clip=clip)

    @staticmethod
    def norm_stats(x):
        """Row statistics of x, to share between several ``mod=`` consumers of the same rows."""
        return _ops.layer_norm_stats(x)

    @staticmethod
    def awq(x, lin: AWQW4A16Linear):
        return lin(x)

    def awq_many(self, x, lins):
        """``[lin(x) for lin in lins]`` with the layers of equal width in one launch each (``ops.AwqGemvBatch``): the
        adaLN projections of all blocks take the same vector and nothing else, so a forward pass runs them first, all
        together; a 32 MB weight by itself is too short a read for the HBM rate.  The results live in buffers the next
        call overwrites."""
        if x.shape[0] > 8 or any(lin.group_size != 64 or lin.out_features % 32 for lin in lins):
            return [lin(x) for lin in lins]
        # the plan holds device addresses and a stacked copy of the biases: it is only good while the layers' tensors stay
        # where they are (a model moved, reloaded or given other parameters gets a new plan)
        key = tuple((lin.qweight.data_ptr(), lin.wscales.data_ptr(), lin.wzeros.data_ptr(),
                     None if lin.bias is None else (lin.bias.data_ptr(), lin.bias._version)) for lin in lins) + (x.shape[0], x.dtype)  # fmt: skip
        plan = self._awq_plans.get(key)
        if plan is None:
            plan = []
            for n in sorted({lin.out_features for lin in lins}):
                idx = [i for i, lin in enumerate(lins) if lin.out_features == n]
                batch = _ops.AwqGemvBatch([lins[i].qweight for i in idx], [lins[i].wscales for i in idx],
                                          [lins[i].wzeros for i in idx], x.shape[0], n, lins[0].in_features)  # fmt: skip
                bias = torch.stack([lins[i].bias for i in idx])[:, None] if all(lins[i].bias is not None for i in idx) else None
                assert bias is not None or all(lins[i].bias is None for i in idx)
                plan.append((idx, batch, bias))
            self._awq_plans = {key: plan}  # one model at a time: a new set of layers replaces the old plan
        out = [None] * len(lins)
        for idx, batch, bias in plan:
            y = batch(x)
            if bias is not None:
                y += bias
            for j, i in enumerate(idx):
                out[i] = y[j]
        return out

    @staticmethod
    def attention(q, k, v):
        return _ops.scaled_dot_product_attention(q, k, v)


def _fp16_clip(x: torch.Tensor) -> float:
    """The reference limits fp16 hidden states to the finite range at the end of the text stream of a dual-stream block
    and at the end of a single-stream block (nunchaku/models/transformers/transformer_flux_v2.py:255-256, :340-341)."""
    return 65504.0 if x.dtype == torch.float16 else 0.0


def rope_table(ids: torch.Tensor, axes_dim, theta: float) -> torch.Tensor:
    """(T, n_axes) positions -> (T, sum(axes_dim) / 2, 1, 2) float32 rows of (sin, cos), computed in float64."""
    out = []
    for i, d in enumerate(axes_dim):
        scale = torch.arange(0, d, 2, dtype=torch.float64, device=ids.device) / d
        ang = ids[:, i].double()[:, None] * (1.0 / (theta**scale))[None, :]
        out.append(torch.stack([torch.sin(ang), torch.cos(ang)], dim=-1))
    return torch.cat(out, dim=1).float().unsqueeze(2)


def flux_ids(txt_tokens: int, grid_h: int, grid_w: int, device=None) -> torch.Tensor:
    img = torch.zeros(grid_h, grid_w, 3, device=device)
    img[..., 1] = torch.arange(grid_h, device=device)[:, None]
    img[..., 2] = torch.arange(grid_w, device=device)[None, :]
    return torch.cat([torch.zeros(txt_tokens, 3, device=device), img.reshape(-1, 3)], dim=0)


def _timestep_embedding(t: torch.Tensor, dim: int = 256) -> torch.Tensor:
    half = dim // 2
    freqs = torch.exp(-math.log(10000.0) * torch.arange(half, dtype=torch.float32, device=t.device) / half)
    args = (t.float() * 1000.0)[:, None] * freqs[None, :]
    return torch.cat([torch.cos(args), torch.sin(args)], dim=-1)


def _init_svdq(lin: SVDQW4A4Linear, gen: torch.Generator) -> None:
    """int4 codes uniform in [-8, 7] (uniform random bytes), scales U(0.005, 0.02), smooth U(0.5, 4), LoRA N(0, 0.02),
    bias N(0, 0.01) -- drawn on the layer's device."""
    dev, dt = lin.qweight.device, lin.wscales.dtype
    r = lambda *s: torch.rand(*s, device=dev, generator=gen)  # noqa: E731
    n = lambda *s: torch.randn(*s, device=dev, generator=gen)  # noqa: E731
    with torch.no_grad():
        lin.qweight.copy_(torch.randint(0, 256, lin.qweight.shape, device=dev, generator=gen, dtype=torch.uint8).view(torch.int8))
        lin.wscales.copy_((r(*lin.wscales.shape) * 0.015 + 0.005).to(dt))
        lin.smooth_factor.copy_((r(*lin.smooth_factor.shape) * 3.5 + 0.5).to(dt))
        lin.smooth_factor_orig.copy_(lin.smooth_factor)
        lin.proj_down.copy_((n(*lin.proj_down.shape) * 0.02).to(dt))
        lin.proj_up.copy_((n(*lin.proj_up.shape) * 0.02).to(dt))
        if lin.bias is not None:
            lin.bias.copy_((n(*lin.bias.shape) * 0.01).to(dt))


def _init_awq(lin: AWQW4A16Linear, gen: torch.Generator) -> None:
    """uint4 codes uniform (uniform random int32 words), scales U(0.005, 0.02), zero-points uniform in [0, 15] stored
    as ``-zp * s``, bias N(0, 0.01)."""
    dev, dt = lin.qweight.device, lin.wscales.dtype
    with torch.no_grad():
        lin.qweight.copy_(torch.randint(-(2**31), 2**31 - 1, lin.qweight.shape, device=dev, generator=gen, dtype=torch.int64).to(torch.int32))
        s = (torch.rand(*lin.wscales.shape, device=dev, generator=gen) * 0.015 + 0.005).to(dt)
        zp = torch.randint(0, 16, lin.wzeros.shape, device=dev, generator=gen).float()
        lin.wscales.copy_(s)
        lin.wzeros.copy_((-(zp * s.float())).to(dt))
        if lin.bias is not None:
            lin.bias.copy_((torch.randn(*lin.bias.shape, device=dev, generator=gen) * 0.01).to(dt))


class _Attention(nn.Module):
    def __init__(self, cfg: FluxShapedConfig, joint: bool, single: bool, device, dtype):
        super().__init__()
        C, kw = cfg.hidden, dict(rank=cfg.rank, torch_dtype=dtype, device=device)
        self.heads, self.head_dim = cfg.heads, cfg.head_dim
        self.to_qkv = SVDQW4A4Linear(C, 3 * C, **kw)
        self.norm_q = nn.RMSNorm(cfg.head_dim, eps=1e-6, device=device, dtype=dtype)
        self.norm_k = nn.RMSNorm(cfg.head_dim, eps=1e-6, device=device, dtype=dtype)
        self.to_out = SVDQW4A4Linear(C, C, **kw)
        if joint:
            self.add_qkv_proj = SVDQW4A4Linear(C, 3 * C, **kw)
            self.norm_added_q = nn.RMSNorm(cfg.head_dim, eps=1e-6, device=device, dtype=dtype)
            self.norm_added_k = nn.RMSNorm(cfg.head_dim, eps=1e-6, device=device, dtype=dtype)
            self.to_add_out = SVDQW4A4Linear(C, C, **kw)
        self.joint = joint

    def forward(self, be, x, ctx, rot_img, rot_txt, mod_x=None, mod_ctx=None):
        B = x.shape[0]
        if self.joint and B == 1 and getattr(be, "writes_in_place", False):
            # both projections store into one (txt + img tokens, 3 C) buffer: no concatenation pass
            t_txt, t_img = ctx.shape[1], x.shape[1]
            qkv = torch.empty(1, t_txt + t_img, 3 * self.heads * self.head_dim, dtype=x.dtype, device=x.device)
            be.qkv(ctx, self.add_qkv_proj, self.norm_added_q, self.norm_added_k, rot_txt, mod=mod_ctx, out=qkv[0, :t_txt])
            be.qkv(x, self.to_qkv, self.norm_q, self.norm_k, rot_img, mod=mod_x, out=qkv[0, t_txt:])
        else:
            qkv = be.qkv(x, self.to_qkv, self.norm_q, self.norm_k, rot_img, mod=mod_x)
            if self.joint:
                qkv_ctx = be.qkv(ctx, self.add_qkv_proj, self.norm_added_q, self.norm_added_k, rot_txt, mod=mod_ctx)
                qkv = torch.cat([qkv_ctx, qkv], dim=1)  # token order [txt, img]
        q, k, v = (t.view(B, -1, self.heads, self.head_dim).transpose(1, 2) for t in qkv.chunk(3, dim=-1))
        o = be.attention(q, k, v)  # (B, H, T, D), scale D^-0.5, no mask
        o = o.transpose(1, 2).reshape(B, -1, self.heads * self.head_dim).to(q.dtype)
        if self.joint:
            t_txt = ctx.shape[1]
            return be.linear(o[:, t_txt:].contiguous(), self.to_out), be.linear(o[:, :t_txt].contiguous(), self.to_add_out)
        return be.linear(o, self.to_out)


class _DoubleBlock(nn.Module):
    def __init__(self, cfg: FluxShapedConfig, device, dtype):
        super().__init__()
        C, kw = cfg.hidden, dict(rank=cfg.rank, torch_dtype=dtype, device=device)
        self.norm1 = AWQW4A16Linear(C, 6 * C, torch_dtype=dtype, device=device)
        self.norm1_context = AWQW4A16Linear(C, 6 * C, torch_dtype=dtype, device=device)
        self.attn = _Attention(cfg, joint=True, single=False, device=device, dtype=dtype)
        self.ff_fc1 = SVDQW4A4Linear(C, cfg.mlp, **kw)
        self.ff_fc2 = SVDQW4A4Linear(cfg.mlp, C, act_unsigned=True, **kw)
        self.ffc_fc1 = SVDQW4A4Linear(C, cfg.mlp, **kw)
        self.ffc_fc2 = SVDQW4A4Linear(cfg.mlp, C, act_unsigned=True, **kw)
        self.C = C

    @staticmethod
    def _mod6(be, lin, temb, emb=None):
        if emb is None:
            emb = be.awq(F.silu(temb), lin)
        return emb.view(emb.shape[0], -1, 6).permute(2, 0, 1)  # interleaved split: channel c -> (c // 6, c % 6)

    def _forward_two_streams(self, be, side, x, ctx, mods_x, mods_ctx, rot_img, rot_txt):
        """The text stream's kernels on ``side``, the image stream's and the joint attention on the current stream.
        Tensors that cross from one stream to the other are registered with the allocator (record_stream)."""
        sh_a, sc_a, g_a, sh_m, sc_m, g_m = mods_x
        csh_a, csc_a, cg_a, csh_m, csc_m, cg_m = mods_ctx
        at, dev = self.attn, x.device
        main = torch.cuda.current_stream(dev)
        t_txt = ctx.shape[1]
        qkv = torch.empty(1, t_txt + x.shape[1], 3 * self.C, dtype=x.dtype, device=dev)
        for t in (ctx, csh_a, qkv):  # made on this stream (the six text vectors share one storage), used on the side one
            t.record_stream(side)
        side.wait_stream(main)
        with torch.cuda.stream(side):
            be.qkv(ctx, at.add_qkv_proj, at.norm_added_q, at.norm_added_k, rot_txt, mod=(csc_a, csh_a), out=qkv[0, :t_txt])
        be.qkv(x, at.to_qkv, at.norm_q, at.norm_k, rot_img, mod=(sc_a, sh_a), out=qkv[0, t_txt:])
        main.wait_stream(side)
        q, k, v = (t.view(1, -1, at.heads, at.head_dim).transpose(1, 2) for t in qkv.chunk(3, dim=-1))
        o = be.attention(q, k, v).transpose(1, 2).reshape(1, -1, self.C)
        o.record_stream(side)
        side.wait_stream(main)
        with torch.cuda.stream(side):
            ctx, st = be.gated_residual(ctx, cg_a, be.linear(o[:, :t_txt], at.to_add_out), want_stats=True)
            ctx, _ = be.gated_residual(ctx, cg_m, be.gelu_mlp(ctx, self.ffc_fc1, self.ffc_fc2, mod=(csc_m, csh_m, st)), clip=_fp16_clip(ctx))
        x, st = be.gated_residual(x, g_a, be.linear(o[:, t_txt:], at.to_out), want_stats=True)
        x, _ = be.gated_residual(x, g_m, be.gelu_mlp(x, self.ff_fc1, self.ff_fc2, mod=(sc_m, sh_m, st)))
        ctx.record_stream(main)  # read next on either stream
        return ctx, x

    def forward(self, be, x, ctx, temb, rot_img, rot_txt, embs=(None, None)):
        """``embs``: the outputs of ``norm1`` / ``norm1_context`` where the caller has already computed them."""
        # layer_norm(x) * scale + shift in front of each quantized linear runs inside its quantizer (mod=)
        sh_a, sc_a, g_a, sh_m, sc_m, g_m = self._mod6(be, self.norm1, temb, embs[0])
        csh_a, csc_a, cg_a, csh_m, csc_m, cg_m = self._mod6(be, self.norm1_context, temb, embs[1])
        side = be.side_stream(x.device) if x.shape[0] == 1 and hasattr(be, "side_stream") else None
        if side is not None:
            return self._forward_two_streams(be, side, x, ctx, (sh_a, sc_a, g_a, sh_m, sc_m, g_m),
                                             (csh_a, csc_a, cg_a, csh_m, csc_m, cg_m), rot_img, rot_txt)
        ax, ac = self.attn(be, x, ctx, rot_img, rot_txt, mod_x=(sc_a, sh_a), mod_ctx=(csc_a, csh_a))
        # x + gate * y in one kernel that also hands the next norm its row statistics
        x, st = be.gated_residual(x, g_a, ax, want_stats=True)
        x, _ = be.gated_residual(x, g_m, be.gelu_mlp(x, self.ff_fc1, self.ff_fc2, mod=(sc_m, sh_m, st)))
        ctx, st = be.gated_residual(ctx, cg_a, ac, want_stats=True)
        ctx, _ = be.gated_residual(ctx, cg_m, be.gelu_mlp(ctx, self.ffc_fc1, self.ffc_fc2, mod=(csc_m, csh_m, st)), clip=_fp16_clip(ctx))
        return ctx, x


class _SingleBlock(nn.Module):
    def __init__(self, cfg: FluxShapedConfig, device, dtype):
        super().__init__()
        C, kw = cfg.hidden, dict(rank=cfg.rank, torch_dtype=dtype, device=device)
        self.norm = AWQW4A16Linear(C, 3 * C, torch_dtype=dtype, device=device)
        self.mlp_fc1 = SVDQW4A4Linear(C, cfg.mlp, **kw)
        self.mlp_fc2 = SVDQW4A4Linear(cfg.mlp, C, act_unsigned=True, **kw)
        self.attn = _Attention(cfg, joint=False, single=True, device=device, dtype=dtype)
        self.C = C

    def forward(self, be, x, temb, rot, stats=None, emb=None):
        """``stats``: row statistics of x if the producer of x already has them; ``emb``: the output of ``norm`` if the
        caller has already computed it.  Returns (x, statistics of it)."""
        if emb is None:
            emb = be.awq(F.silu(temb), self.norm)
        shift, scale, gate = emb.view(emb.shape[0], -1, 3).permute(2, 0, 1)
        mod = (scale, shift, stats if stats is not None else be.norm_stats(x))  # one set for both consumers
        side = be.side_stream(x.device) if hasattr(be, "side_stream") else None
        if side is None:
            mlp = be.gelu_mlp(x, self.mlp_fc1, self.mlp_fc2, mod=mod)
            att = self.attn(be, x, None, rot, None, mod_x=mod)
        else:
            # the MLP branch on the second stream: its kernels fill the last, partly empty rounds of workgroups of the
            # attention branch's kernels and the other way round
            main = torch.cuda.current_stream(x.device)
            for t in (x, scale, mod[2]):
                t.record_stream(side)
            side.wait_stream(main)
            with torch.cuda.stream(side):
                mlp = be.gelu_mlp(x, self.mlp_fc1, self.mlp_fc2, mod=mod)
            att = self.attn(be, x, None, rot, None, mod_x=mod)
            main.wait_stream(side)
            mlp.record_stream(main)
        return be.gated_residual(x, gate, att, mlp, want_stats=True, clip=_fp16_clip(x))


class FluxShapedTransformer(nn.Module):
    def __init__(self, cfg: FluxShapedConfig | None = None, device="cuda", dtype=torch.bfloat16, seed: int = 0, backend=None):
        super().__init__()
        self.cfg = cfg = cfg or FluxShapedConfig()
        self.backend = backend or HipBackend()
        C = cfg.hidden
        kw = dict(device=device, dtype=dtype)
        self.x_embedder = nn.Linear(cfg.in_channels, C, **kw)
        self.context_embedder = nn.Linear(cfg.text_dim, C, **kw)
        self.time_in = nn.Sequential(nn.Linear(256, C, **kw), nn.SiLU(), nn.Linear(C, C, **kw))
        self.pooled_in = nn.Sequential(nn.Linear(cfg.pooled_dim, C, **kw), nn.SiLU(), nn.Linear(C, C, **kw))
        self.double_blocks = nn.ModuleList([_DoubleBlock(cfg, device, dtype) for _ in range(cfg.n_double)])
        self.single_blocks = nn.ModuleList([_SingleBlock(cfg, device, dtype) for _ in range(cfg.n_single)])
        self.norm_out_linear = nn.Linear(C, 2 * C, **kw)
        self.proj_out = nn.Linear(C, cfg.in_channels, **kw)
        gen = torch.Generator(device=device).manual_seed(seed)
        for m in self.modules():
            if isinstance(m, SVDQW4A4Linear):
                _init_svdq(m, gen)
            elif isinstance(m, AWQW4A16Linear):
                _init_awq(m, gen)
            elif isinstance(m, nn.Linear):
                with torch.no_grad():
                    m.weight.copy_((torch.randn(m.weight.shape, device=device, generator=gen) / math.sqrt(m.in_features)).to(dtype))
                    m.bias.zero_()
            elif isinstance(m, nn.RMSNorm):
                with torch.no_grad():
                    m.weight.copy_((torch.rand(m.weight.shape, device=device, generator=gen) + 0.5).to(dtype))
        self.requires_grad_(False)

    # names of nunchaku's FLUX model (what ``layout.convert_flux_state_dict`` produces, transformer_flux_v2.py:579-649)
    # -> names of this harness; first match wins
    _CHECKPOINT_NAMES = (
        (r"^transformer_blocks\.(\d+)\.norm1\.linear\.", r"double_blocks.\1.norm1."),
        (r"^transformer_blocks\.(\d+)\.norm1_context\.linear\.", r"double_blocks.\1.norm1_context."),
        (r"^transformer_blocks\.(\d+)\.attn\.to_out\.0\.", r"double_blocks.\1.attn.to_out."),
        (r"^transformer_blocks\.(\d+)\.attn\.", r"double_blocks.\1.attn."),
        (r"^transformer_blocks\.(\d+)\.ff\.net\.0\.proj\.", r"double_blocks.\1.ff_fc1."),
        (r"^transformer_blocks\.(\d+)\.ff\.net\.2\.", r"double_blocks.\1.ff_fc2."),
        (r"^transformer_blocks\.(\d+)\.ff_context\.net\.0\.proj\.", r"double_blocks.\1.ffc_fc1."),
        (r"^transformer_blocks\.(\d+)\.ff_context\.net\.2\.", r"double_blocks.\1.ffc_fc2."),
        (r"^single_transformer_blocks\.(\d+)\.norm\.linear\.", r"single_blocks.\1.norm."),
        (r"^single_transformer_blocks\.(\d+)\.", r"single_blocks.\1."),
        (r"^time_text_embed\.timestep_embedder\.linear_1\.", "time_in.0."),
        (r"^time_text_embed\.timestep_embedder\.linear_2\.", "time_in.2."),
        (r"^time_text_embed\.text_embedder\.linear_1\.", "pooled_in.0."),
        (r"^time_text_embed\.text_embedder\.linear_2\.", "pooled_in.2."),
        (r"^norm_out\.linear\.", "norm_out_linear."),
    )
    # tensors a checkpoint may carry that the int4 path does not use (NVFP4 scales, the un-fused smoothing factors)
    def release_packed_weights(self) -> int:
        """Let every ``SVDQW4A4Linear`` keep only the GEMM's working copy of its weight (``release_packed_weight``): a
        FLUX.1-sized model then holds about 9 GB of 4-bit weights instead of 15 GB.  Returns the bytes released."""
        from .linear import SVDQW4A4Linear

        freed = 0
        for m in self.modules():
            if isinstance(m, SVDQW4A4Linear):
                n = m.out_features * (m.in_features // 2)
                if m.qweight.untyped_storage().nbytes() >= n and m.release_packed_weight():
                    freed += n
        return freed

    _CHECKPOINT_IGNORED = (".smooth_factor_orig", ".wtscale", ".wcscales")

    @torch.no_grad()
    def load_converted(self, state_dict: dict, strict: bool = True) -> None:
        """Fill the model from a published int4 checkpoint: ``state_dict`` as ``layout.load_checkpoint`` reads it and
        ``layout.convert_flux_state_dict`` renames it (tensors still in checkpoint layout).  Names are mapped onto this
        harness, the tensors are loaded as they are, and every ``SVDQW4A4Linear`` is then turned into the natural layout
        once (``convert_svdq_linear_to_natural_layout``); AWQ tensors stay in TinyChat packing.  What the reference's
        ``from_pretrained`` does after building its model (transformer_flux_v2.py:419-435).  ``strict``: every tensor
        of the model must be in the file and every tensor of the file must have a place (except the ones the int4 path
        ignores)."""
        import re

        from .layout import convert_svdq_linear_to_natural_layout

        own = dict(self.named_parameters())
        own.update(dict(self.named_buffers()))
        mapped, unexpected = {}, []
        for key, value in state_dict.items():
            if key.endswith(self._CHECKPOINT_IGNORED):
                continue
            name = key
            for pat, rep in self._CHECKPOINT_NAMES:
                name, n = re.subn(pat, rep, key)
                if n:
                    break
            if name in own:
                mapped[name] = value
            else:
                unexpected.append(key)
        missing = [k for k in own if k not in mapped and not k.endswith(self._CHECKPOINT_IGNORED)]
        if strict and (missing or unexpected):
            raise KeyError(f"checkpoint does not match the model: missing {missing[:8]}{'...' if len(missing) > 8 else ''}, "
                           f"unexpected {unexpected[:8]}{'...' if len(unexpected) > 8 else ''}")  # fmt: skip
        for name, value in mapped.items():
            dst = own[name]
            if value.numel() != dst.numel():
                raise ValueError(f"{name}: checkpoint tensor has {tuple(value.shape)}, the model {tuple(dst.shape)}")
            # the checkpoint's 2-D views of the shuffled tensors differ from the logical shapes; the bytes are what counts
            src = value.to(dst.device)
            if src.dtype != dst.dtype:
                src = src.view(dst.dtype) if src.element_size() == dst.element_size() and not src.is_floating_point() else src.to(dst.dtype)
            dst.data = src.reshape(dst.shape).contiguous()
        for m in self.modules():
            if isinstance(m, SVDQW4A4Linear):
                convert_svdq_linear_to_natural_layout(m)

    @torch.no_grad()
    def _rot_parts(self, rot: torch.Tensor, t_txt: int):
        """The text and image rows of the rotary table as tensors of their own, the same two objects for as long as the
        table is the same tensor with the same contents: the operators keep a re-laid-out copy per table tensor, and a
        forward pass recorded into a graph must not make new ones."""
        hit = getattr(self, "_rot_split", None)
        if hit is not None and hit[0]() is rot and hit[1] == (rot.data_ptr(), rot._version, t_txt):
            return hit[2], hit[3]
        import weakref

        parts = (rot[:t_txt].contiguous(), rot[t_txt:].contiguous())
        self._rot_split = (weakref.ref(rot), (rot.data_ptr(), rot._version, t_txt), parts[0], parts[1])
        return parts

    def forward(self, latents, text, pooled, timestep, rot, backend=None):
        """latents (B, T_img, 64), text (B, T_txt, 4096), pooled (B, 768), timestep (B,) in [0, 1], rot the
        (T_txt + T_img, 64, 1, 2) rotary table (text rows first).  Returns the (B, T_img, 64) velocity."""
        be = backend or self.backend
        x = self.x_embedder(latents)
        ctx = self.context_embedder(text)
        temb = self.time_in(_timestep_embedding(timestep).to(x.dtype)) + self.pooled_in(pooled)
        t_txt = ctx.shape[1]
        rot_txt, rot_img = self._rot_parts(rot, t_txt)
        # every adaLN projection takes silu(temb) and nothing else: all of them first, layers of equal width in one launch
        nd = len(self.double_blocks)
        if hasattr(be, "awq_many"):
            embs = be.awq_many(F.silu(temb), [lin for blk in self.double_blocks for lin in (blk.norm1, blk.norm1_context)]
                               + [blk.norm for blk in self.single_blocks])  # fmt: skip
        else:
            embs = [None] * (2 * nd + len(self.single_blocks))
        for i, blk in enumerate(self.double_blocks):
            ctx, x = blk(be, x, ctx, temb, rot_img, rot_txt, embs=(embs[2 * i], embs[2 * i + 1]))
        if hasattr(be, "join"):
            be.join(x.device)  # the last block's text stream was produced on the side stream
        x = torch.cat([ctx, x], dim=1)
        stats = None
        for i, blk in enumerate(self.single_blocks):
            x, stats = blk(be, x, temb, rot, stats, emb=embs[2 * nd + i])
        x = x[:, t_txt:]
        scale, shift = self.norm_out_linear(F.silu(temb)).chunk(2, dim=1)
        x = F.layer_norm(x, (self.cfg.hidden,), eps=1e-6) * (1 + scale)[:, None] + shift[:, None]
        return self.proj_out(x)

    @torch.no_grad()
    def capture(self, latents, text, pooled, rot, backend=None):
        """Record one forward pass (all of its launches on both streams) into a HIP graph.  Returns
        ``step(latents, timestep) -> velocity``: it copies its arguments into the recorded input buffers, replays the
        graph and returns the recorded output buffer (overwritten by the next call).  ``text``, ``pooled`` and ``rot``
        are fixed at capture.  The ~1100 launches of a step then cost the host one call."""
        dev = latents.device
        s_lat, s_t = latents.clone(), torch.zeros(latents.shape[0], device=dev)
        warm = torch.cuda.Stream(dev)
        warm.wait_stream(torch.cuda.current_stream(dev))
        with torch.cuda.stream(warm):  # first uses (weight re-layouts, library workspaces) happen outside the graph
            for _ in range(2):
                self.forward(s_lat, text, pooled, s_t, rot, backend=backend)
        torch.cuda.current_stream(dev).wait_stream(warm)
        torch.cuda.synchronize(dev)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            out = self.forward(s_lat, text, pooled, s_t, rot, backend=backend)

        def step(lat, timestep):
            s_lat.copy_(lat)
            s_t.copy_(timestep)
            graph.replay()
            return out

        step.graph = graph  # keeps the recording (and its memory pool) alive with the callable
        return step

    @torch.no_grad()
    def denoise(self, latents, text, pooled, rot, steps: int = 4, backend=None, step_fn=None):
        """Euler steps of the rectified flow from t = 1 to t = 0 (FLUX.1-schnell runs 4).  ``step_fn``: a callable from
        :meth:`capture` to run the forward passes from a recorded HIP graph."""
        sig = torch.linspace(1.0, 0.0, steps + 1, device=latents.device)
        for i in range(steps):
            t = sig[i].expand(latents.shape[0])
            if step_fn is not None:
                v = step_fn(latents, t)
            else:
                v = self.forward(latents, text, pooled, t, rot, backend=backend)
            latents = (latents.float() + (sig[i + 1] - sig[i]) * v.float()).to(latents.dtype)
        return latents
