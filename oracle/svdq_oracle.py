"""
CPU oracle for the SVDQuant kernel path (TEST INFRASTRUCTURE -- never a product path).

This file restates, in plain fp32/int torch-CPU arithmetic, what the reference
computes for the activation quantizer, the W4A4 GEMM with its epilogues, and
the AWQ W4A16 GEMV.  Only ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` may import it; nothing under
``nunchaku_rocm_amd/`` does, and the product raises when its HIP library is
missing rather than falling back to anything here.

Each function names the reference lines it follows (paths relative to the
reference checkout).  How each function is pinned (none of them by re-typing
its own formula) is listed in ``tests/test_oracle_pins.py``:

=====================  =======================================================
function               pinned by
=====================  =======================================================
unpack_int4/pack_int4  round trip + hand-written byte examples + the nibble
                       order statement of gemm_w4a4.py:12-14
quantize_act           closed-form exact cases (power-of-two grids), range /
                       half-step invariants, zero-group rule, fp64 LoRA-down,
                       the C restatement in svdq_oracle.c (independent loops)
group_acc_i32          brute-force int64 loops on tiny inputs
gemm_w4a4              unit-scale exact integer GEMM, fp64 closed form
qk_norm_rope           fp64 RMSNorm + complex-multiplication RoPE
gelu_tanh              torch.nn.functional.gelu(approximate="tanh") in fp64
gelu_quant             composition: quantize_act(gelu(x)) identities
swiglu                 torch.nn.functional.silu in fp64, interleave inverse
awq_pack / awq_decode  mutual inverse, written from two different statements
                       of the layout (view/permute vs. index formula)
awq_gemv               fp64 dense dequantised matmul
awq_dequantize         fp64 q * s + z rounded once (q * s is exact), per-group
                       constancy, zero-point identity q = zp -> 0
flux_rope              closed form cos/sin of pos * theta**(-2i/d) in fp64
gated_residual         torch's own 16-bit CPU kernels, op by op (bit-equal)
layernorm_modulate     torch.nn.functional.layer_norm in fp64 and torch's own
                       bf16 elementwise kernels on the CPU
attention_fp16         fp64 softmax(q k^T * scale) v, independence of the key
                       block size, uniform-weights / constant-v / dominant-key
                       special cases
=====================  =======================================================

Floating point: every elementwise op below is an IEEE fp32 primitive on CPU
(cast, multiply, divide, max, add), so the int4 codes and bf16 scales are
bit-defined.  exp() inside GELU/SiLU is not bit-defined across libraries; the
contract for codes after GELU is "differ by at most 1 on < 1e-5 of entries"
(reference: tests/triton/test_native_epilogues.py:246-253).
"""

from __future__ import annotations

import torch

GROUP = 64  # int4 scale group along K (nunchaku/models/linear.py:92)
HEAD_DIM = 128  # nunchaku/ops/triton/gemm_w4a4.py:376
GELU_SHIFT = 0.171875  # nunchaku/ops/triton/gemm_w4a4.py:918,1299
RNE_MAGIC = 12582912.0  # 1.5 * 2**23, nunchaku/ops/triton/gemm_w4a4.py:1325
RMS_EPS = 1e-6  # nunchaku/ops/triton/gemm_w4a4.py:1251
SWIGLU_BLOCK = 16  # nunchaku/ops/triton/native/w4a4.py:73


# --------------------------------------------------------------------------------------
# nibble packing
# --------------------------------------------------------------------------------------
def unpack_int4(packed: torch.Tensor, signed: bool) -> torch.Tensor:
    """(rows, K/2) bytes -> (rows, K) int32 codes; element k is the low nibble of byte k//2 for
    even k, the high nibble for odd k (nunchaku/ops/triton/gemm_w4a4.py:12-14,
    nunchaku/ops/triton/native/w4a4.py:707-710).  Signed = two's complement."""
    b = packed.contiguous().view(torch.uint8).to(torch.int32)
    x = torch.stack([b & 0xF, b >> 4], dim=-1).reshape(b.shape[0], -1)
    if signed:
        x = torch.where(x >= 8, x - 16, x)
    return x


def pack_int4(codes: torch.Tensor) -> torch.Tensor:
    """(rows, K) integer codes (any sign) -> (rows, K/2) uint8, byte j = code[2j] | code[2j+1] << 4
    (nunchaku/ops/triton/gemm_w4a4.py:1448-1449)."""
    c = (codes.to(torch.int32) & 0xF).reshape(codes.shape[0], -1, 2)
    return (c[..., 0] | (c[..., 1] << 4)).to(torch.uint8)


# --------------------------------------------------------------------------------------
# activation quantizer
# --------------------------------------------------------------------------------------
def gelu_tanh(x: torch.Tensor) -> torch.Tensor:
    """nunchaku/ops/triton/_common.py:71-78, fp32."""
    x = x.float()
    inner = 0.79788456 * (x + 0.044715 * x * x * x)
    t = 2.0 / (1.0 + torch.exp(-2.0 * inner)) - 1.0
    return 0.5 * x * (1.0 + t)


def silu(x: torch.Tensor) -> torch.Tensor:
    """nunchaku/ops/triton/_common.py:91-95, fp32."""
    x = x.float()
    return x / (1.0 + torch.exp(-x))


def quantize_act(
    x: torch.Tensor,
    lora_down: torch.Tensor | None = None,
    smooth: torch.Tensor | None = None,
    unsigned: bool = False,
    shift: float = 0.0,
    fuse_gelu: bool = False,
    fuse_glu: bool = False,
):
    """Per-group-64 int4 activation quantizer with fused LoRA-down.

    Follows ``_quantize_tile_kernel`` (nunchaku/ops/triton/gemm_w4a4.py:1397-1455) op by op:
    cast to fp32; optional GLU/GELU; LoRA-down on the value rounded back to the 16-bit type,
    *before* shift and smoothing; ``x += shift``; ``x *= (1.0f / smooth)``; group max (abs for
    signed); ``scale = gmax / qmax``; the stored scale is rounded to the 16-bit type but the codes
    use the unrounded fp32 scale through ``x * (1.0f / scale_safe)``; round half to even by the
    1.5*2**23 add/subtract; clamp; pack low nibble first.

    Returns ``(packed (M, K/2) uint8, scales (K/64, M) of x.dtype, lora_act (M, R) fp32 or None,
    codes (M, K) int32)``.
    """
    T = x.dtype
    xf = x.float()
    if fuse_glu:
        K = xf.shape[1] // 2
        gate = xf[:, K:]
        xf = xf[:, :K] * (gate / (1.0 + torch.exp(-gate)))
    if fuse_gelu:
        xf = gelu_tanh(xf)
    M, K = xf.shape
    assert K % GROUP == 0
    lora_act = None
    if lora_down is not None:
        # fp32 accumulation of 16-bit products, K walked in 64-blocks (:1411-1417)
        lora_act = torch.zeros(M, lora_down.shape[1], dtype=torch.float32, device=x.device)
        xt = xf.to(T).float()
        ld = lora_down.float()
        for k0 in range(0, K, GROUP):
            lora_act += xt[:, k0 : k0 + GROUP] @ ld[k0 : k0 + GROUP]
    xf = xf + torch.tensor(shift, dtype=torch.float32, device=x.device)
    if smooth is not None:
        xf = xf * (torch.tensor(1.0, dtype=torch.float32, device=x.device) / smooth.float())[None, :]
    qmax = 15.0 if unsigned else 7.0
    xg = xf.reshape(M, K // GROUP, GROUP)
    gmax = xg.amax(dim=2) if unsigned else xg.abs().amax(dim=2)
    gmax = torch.clamp_min(gmax, 0.0)
    scale = gmax / torch.tensor(qmax, dtype=torch.float32, device=x.device)
    scale_safe = torch.where(scale == 0.0, torch.ones_like(scale), scale)
    q = xg * (torch.tensor(1.0, dtype=torch.float32, device=x.device) / scale_safe)[:, :, None]
    magic = torch.tensor(RNE_MAGIC, dtype=torch.float32, device=x.device)
    r = (q + magic) - magic
    lo, hi = (0.0, 15.0) if unsigned else (-8.0, 7.0)
    codes = torch.clamp(r, lo, hi).to(torch.int32).reshape(M, K)
    return pack_int4(codes), scale.to(T).t().contiguous(), lora_act, codes


# --------------------------------------------------------------------------------------
# W4A4 GEMM
# --------------------------------------------------------------------------------------
def group_acc_i32(act: torch.Tensor, wgt: torch.Tensor, act_unsigned: bool, groups=None) -> torch.Tensor:
    """Exact per-group integer dot products ``p[g, m, n] = sum_{k in g} a[m, k] * w[n, k]``
    (nunchaku/ops/triton/gemm_w4a4.py:477-483; |p| <= 64*15*8 so fp32 matmul is exact, as
    nunchaku/ops/triton/native/w4a4.py:713-720 relies on).  Returns int32 (G, M, N)."""
    a = unpack_int4(act, not act_unsigned).float()
    w = unpack_int4(wgt, True).float()
    G = a.shape[1] // GROUP
    groups = range(G) if groups is None else groups
    out = []
    for g in groups:
        sl = slice(g * GROUP, (g + 1) * GROUP)
        out.append((a[:, sl] @ w[:, sl].t()).to(torch.int32))
    return torch.stack(out)


def gemm_w4a4(
    act,
    wgt,
    ascales,
    wscales,
    bias=None,
    lora_act=None,
    lora_up=None,
    act_unsigned: bool = False,
) -> torch.Tensor:
    """fp32 result (before the final rounding to the 16-bit type) of the plain W4A4 GEMM:
    ``acc += (f32(p_g) * as[g, m]) * ws[g, n]`` sequentially over groups
    (nunchaku/ops/triton/gemm_w4a4.py:483), then LoRA-up on the hidden state rounded to the
    16-bit type, then bias (nunchaku/ops/triton/gemm_w4a4.py:181-205;
    nunchaku/ops/triton/native/w4a4.py:713-726)."""
    a = unpack_int4(act, not act_unsigned).float()
    w = unpack_int4(wgt, True).float()
    M, N = a.shape[0], w.shape[0]
    out = torch.zeros(M, N, dtype=torch.float32, device=a.device)
    for g in range(a.shape[1] // GROUP):
        sl = slice(g * GROUP, (g + 1) * GROUP)
        out += (a[:, sl] @ w[:, sl].t()) * ascales[g, :M].float()[:, None] * wscales[g, :N].float()[None, :]
    if lora_up is not None and lora_up.shape[1]:
        R = lora_up.shape[1]
        out += lora_act[:M, :R].to(lora_up.dtype).float() @ lora_up[:N].float().t()
    if bias is not None:
        out += bias[:N].float()
    return out


def gemm_w4a4_dense(act, wgt, ascales, wscales, bias=None, lora_act=None, lora_up=None, act_unsigned: bool = False):
    """The same sum written as one fp32 matmul of element-wise dequantised operands (the form the reference's
    parity tests use, tests/triton/test_w4a4.py:32-60); differs from :func:`gemm_w4a4` only by fp32 rounding order."""
    K = act.shape[1] * 2
    grp = torch.arange(K, device=act.device) // GROUP
    M, N = act.shape[0], wgt.shape[0]
    a = unpack_int4(act, not act_unsigned).float() * ascales.float()[grp, :M].t()
    w = unpack_int4(wgt, True).float() * wscales.float()[grp, :N].t()
    out = a @ w.t()
    if lora_up is not None and lora_up.shape[1]:
        out += lora_act[:M, : lora_up.shape[1]].to(lora_up.dtype).float() @ lora_up[:N].float().t()
    if bias is not None:
        out += bias[:N].float()
    return out


def qk_norm_rope(lin: torch.Tensor, norm_q, norm_k, rot: torch.Tensor) -> torch.Tensor:
    """Per-head RMSNorm (eps 1e-6) then RoPE on the Q and K thirds of ``lin`` (M, N) fp32, V
    untouched; ``rot`` (M, 128) fp32 rows of (sin, cos) pairs
    (nunchaku/ops/triton/gemm_w4a4.py:499-521; nunchaku/ops/triton/native/w4a4.py:729-740)."""
    M, N = lin.shape
    x = lin.float().clone().view(M, 3, N // 3 // HEAD_DIM, HEAD_DIM)
    sc = rot.float().reshape(M, 1, HEAD_DIM // 2, 2)
    sin, cos = sc[..., 0], sc[..., 1]
    for part, w in ((0, norm_q), (1, norm_k)):
        h = x[:, part]
        rstd = torch.rsqrt((h * h).sum(-1, keepdim=True) / HEAD_DIM + RMS_EPS)
        h = h * rstd * w.float()
        xe, xo = h[..., 0::2], h[..., 1::2]
        x[:, part] = torch.stack([xe * cos - xo * sin, xe * sin + xo * cos], -1).flatten(-2)
    return x.view(M, N)


def gelu_quant(lin: torch.Tensor, smooth, lora_down, dtype, shift: float = GELU_SHIFT):
    """GELU -> LoRA-down on the un-shifted, un-smoothed value -> +shift -> *1/smooth -> unsigned
    per-64 quantization of the fp32 GEMM tile ``lin`` (M, N), in the fused epilogue's op order
    (nunchaku/ops/triton/gemm_w4a4.py:730-778).  Returns (packed, scales (N/64, M), lora_act, codes)."""
    g = gelu_tanh(lin)
    packed, scales, _, codes = quantize_act(g, None, smooth, unsigned=True, shift=shift)
    lora = None
    if lora_down is not None:
        lora = g.to(dtype).float() @ lora_down.float()
    return packed, scales.to(dtype), lora, codes


def interleave_swiglu(n: int) -> torch.Tensor:
    """Row order that turns ``[gate (n/2) | up (n/2)]`` into 16-row blocks gate,up,gate,up...
    (nunchaku/ops/triton/native/w4a4.py:350-360)."""
    h, b = n // 2, SWIGLU_BLOCK
    g = torch.arange(h).view(h // b, b)
    return torch.stack([g, g + h], dim=1).reshape(-1)


def swiglu_quant(lin_interleaved: torch.Tensor, smooth, lora_down, dtype):
    """``silu(gate) * up`` on an interleaved-column fp32 GEMM tile, then the signed quantizer with
    LoRA-down (nunchaku/ops/triton/gemm_w4a4.py:998-1000 for the unfused composition, which rounds
    the GEMM output to the 16-bit type first; the fused epilogue of
    nunchaku/ops/triton/native/w4a4_gfx11.hip:722-790 works on the fp32 tile -- this function
    follows the fused form).  Returns (packed, scales (H/64, M), lora_act, codes)."""
    M, N = lin_interleaved.shape
    x = lin_interleaved.float().view(M, N // 32, 2, 16)
    y = (silu(x[:, :, 0]) * x[:, :, 1]).reshape(M, N // 2)
    packed, scales, _, codes = quantize_act(y, None, smooth, unsigned=False)
    lora = None
    if lora_down is not None:
        lora = y.to(dtype).float() @ lora_down.float()
    return packed, scales.to(dtype), lora, codes


# --------------------------------------------------------------------------------------
# AWQ W4A16
# --------------------------------------------------------------------------------------
def awq_pack(q: torch.Tensor) -> torch.Tensor:
    """Logical uint4 ``[oc, ic]`` int32 -> TinyChat int16 ``[oc/4, ic]``
    (nunchaku/models/text_encoders/tinychat_utils.py:76-106): four nibbles 8 apart along ic per
    int16, then the (oc/4, 4, ic/64, 16) -> (0, 2, 1, 3) interleave."""
    oc, ic = q.shape
    w = q.to(torch.int32).view(-1, 4, 8)
    w = w[:, 0] | (w[:, 1] << 4) | (w[:, 2] << 8) | (w[:, 3] << 12)
    w = w.view(oc // 4, 4, ic // 64, 16).permute(0, 2, 1, 3).reshape(oc // 4, ic)
    return w.to(torch.int16)


def awq_decode(packed_i16: torch.Tensor, n: int, k: int) -> torch.Tensor:
    """Inverse of :func:`awq_pack` written from the index statement of
    nunchaku/ops/triton/awq.py:29-47: logical (n, k) lives in stored int16 column
    ``e = 64*c + 16*(n%4) + d`` of row ``n//4`` with ``t = (k//32)*8 + k%8``, ``c = t//16``,
    ``d = t%16``, at bit ``4*((k%32)//8)``."""
    nn_ = torch.arange(n, device=packed_i16.device).view(-1, 1)
    kk = torch.arange(k, device=packed_i16.device).view(1, -1)
    a, b = nn_ // 4, nn_ % 4
    g, m, j = kk // 32, (kk % 32) // 8, kk % 8
    t = g * 8 + j
    e = (t // 16) * 64 + b * 16 + (t % 16)
    raw = packed_i16.to(torch.int32)[a.expand(n, k), e] & 0xFFFF
    return (raw >> (4 * m)) & 0xF


def awq_gemv(x: torch.Tensor, packed_i16: torch.Tensor, scales: torch.Tensor, zeros: torch.Tensor) -> torch.Tensor:
    """fp32 result of ``out[m, n] = sum_c s[c, n] * sum_{k in c} x[m, k] q[n, k] + z[c, n] * sum_{k in c} x[m, k]``
    (nunchaku/ops/triton/awq.py:160-182), group 64."""
    m, k = x.shape
    n = scales.shape[1]
    q = awq_decode(packed_i16, n, k).float()
    xf = x.float()
    out = torch.zeros(m, n, dtype=torch.float32, device=x.device)
    for c in range(k // GROUP):
        sl = slice(c * GROUP, (c + 1) * GROUP)
        dotq = xf[:, sl] @ q[:, sl].t()
        xsum = xf[:, sl].sum(dim=1, keepdim=True)
        out += scales[c].float()[None, :] * dotq + zeros[c].float()[None, :] * xsum
    return out


def awq_dequantize(packed_i16: torch.Tensor, scales: torch.Tensor, zeros: torch.Tensor, group_size: int) -> torch.Tensor:
    """Dense weight ``T(q * s + z)`` with fp32 arithmetic (nunchaku/ops/triton/awq.py:48-79): ``(n, k)`` in the dtype of
    ``scales``, scale group ``k // group_size``."""
    n = scales.shape[1]
    k = packed_i16.shape[1]
    q = awq_decode(packed_i16, n, k).float()
    grp = torch.arange(k, device=scales.device) // group_size
    s = scales.float().t()[:, grp]
    z = zeros.float().t()[:, grp]
    return (q * s + z).to(scales.dtype)


# --------------------------------------------------------------------------------------
# LayerNorm + adaLN modulate in front of a quantized linear
# --------------------------------------------------------------------------------------
def layernorm_modulate(x: torch.Tensor, scale: torch.Tensor, shift: torch.Tensor, eps: float = 1e-6) -> torch.Tensor:
    """nunchaku/models/normalization.py:97-104 and models/transformers/transformer_flux_v2.py:236-237 as three 16-bit
    elementwise steps: LayerNorm without affine (fp32 statistics, biased variance, ``(x - mean) * rstd`` rounded to the
    16-bit type), ``* scale`` rounded, ``+ shift`` rounded.  x (M, K); scale, shift (K,) or (batches, K)."""
    dt = x.dtype
    M, K = x.shape
    xf = x.float()
    mean = xf.mean(dim=1, keepdim=True)
    var = ((xf - mean) ** 2).mean(dim=1, keepdim=True)
    n = ((xf - mean) * (1.0 / torch.sqrt(var + eps))).to(dt)
    sc = scale.reshape(-1, K).repeat_interleave(M // scale.reshape(-1, K).shape[0], dim=0)
    sh = shift.reshape(-1, K).repeat_interleave(M // shift.reshape(-1, K).shape[0], dim=0)
    y = (n.float() * sc.float()).to(dt)
    return (y.float() + sh.float()).to(dt)


def gated_residual(x: torch.Tensor, gate: torch.Tensor, y: torch.Tensor, y2: torch.Tensor | None = None,
                   clip: float = 0.0) -> torch.Tensor:  # fmt: skip
    """nunchaku/models/transformers/transformer_flux_v2.py:233-234, :241-243 (``x + gate.unsqueeze(1) * y``) and
    :326-330 (``x + gate.unsqueeze(1) * (y + y2)``) as 16-bit elementwise steps: every +, * rounded to the dtype.
    x, y (B, S, C); gate (B, C).  ``clip``: the ``.clip(-65504, 65504)`` that follows in fp16 runs (:255-256, :340-341)."""
    dt = x.dtype
    t = y if y2 is None else (y.float() + y2.float()).to(dt)
    g = (gate.float()[:, None, :] * t.float()).to(dt)
    out = (x.float() + g.float()).to(dt)
    return out.clip(-clip, clip) if clip > 0 else out


# --------------------------------------------------------------------------------------
# Unmasked 16-bit attention
# --------------------------------------------------------------------------------------
def attention_fp16(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, block_n: int = 64) -> torch.Tensor:
    """nunchaku/ops/triton/attention.py:62-119, :139-141: q (B, H, Tq, D), k / v (B, H, Tkv, D) in fp16 or bf16 ->
    (B, Tq, H * D) of the same type.  q * (scale * log2 e) is rounded to the 16-bit type; per block of ``block_n``
    keys the scores are fp32, the running maximum m and sum l are fp32, p = exp2(s - m) is rounded to the 16-bit type
    for the p @ v product (fp32 accumulation) but enters l unrounded; the result is acc / l."""
    dt = q.dtype
    B, H, Tq, D = q.shape
    Tkv = k.shape[2]
    qs = (q.float() * (scale * 1.4426950408889634)).to(dt).float()
    kf, vf = k.float(), v.float()
    m = torch.full((B, H, Tq), float("-inf"))
    l = torch.zeros(B, H, Tq)
    acc = torch.zeros(B, H, Tq, D)
    for n0 in range(0, Tkv, block_n):
        s = qs @ kf[:, :, n0 : n0 + block_n].transpose(-1, -2)
        m_new = torch.maximum(m, s.amax(dim=-1))
        p = torch.exp2(s - m_new[..., None])
        alpha = torch.exp2(m - m_new)  # exp2(-inf) = 0 on the first block
        l = l * alpha + p.sum(dim=-1)
        acc = acc * alpha[..., None] + p.to(dt).float() @ vf[:, :, n0 : n0 + block_n]
        m = m_new
    out = acc / torch.where(l == 0, torch.ones_like(l), l)[..., None]
    return out.to(dt).transpose(1, 2).reshape(B, Tq, H * D)


# --------------------------------------------------------------------------------------
# FLUX rotary table
# --------------------------------------------------------------------------------------
def rope_axis(pos: torch.Tensor, dim: int, theta: float) -> torch.Tensor:
    """nunchaku/models/embeddings.py:11-52 for one axis: (T,) positions -> (T, dim/2, 2) fp32 (sin, cos)."""
    scale = torch.arange(0, dim, 2, dtype=torch.float64) / dim
    omega = 1.0 / (theta**scale)
    out = pos.double()[:, None] * omega[None, :]
    return torch.stack([torch.sin(out), torch.cos(out)], dim=-1).float()


def flux_rotary(ids: torch.Tensor, axes_dim=(16, 56, 56), theta: float = 10000.0) -> torch.Tensor:
    """nunchaku/models/embeddings.py:55-97: ids (T, n_axes) -> (T, sum(axes)/2, 1, 2) fp32."""
    emb = torch.cat([rope_axis(ids[:, i], axes_dim[i], theta) for i in range(ids.shape[1])], dim=1)
    return emb.unsqueeze(2)


def flux_ids(txt_tokens: int, grid_h: int, grid_w: int) -> torch.Tensor:
    """Text tokens are all-zero ids; image token (h, w) has ids (0, h, w); text first
    (nunchaku/models/transformers/transformer_flux_v2.py:510-537,556)."""
    img = torch.zeros(grid_h, grid_w, 3)
    img[..., 1] = torch.arange(grid_h)[:, None]
    img[..., 2] = torch.arange(grid_w)[None, :]
    return torch.cat([torch.zeros(txt_tokens, 3), img.reshape(-1, 3)], dim=0)


# --------------------------------------------------------------------------------------
# seeded synthetic inputs for the benchmark configurations
# --------------------------------------------------------------------------------------
def make_svdq_linear(K: int, N: int, R: int = 32, seed: int = 0, dtype=torch.bfloat16) -> dict:
    """Random-init SVDQuant linear in the natural layout: int4 codes uniform in [-8, 7], group
    scales U(0.005, 0.02), smooth U(0.5, 4), LoRA down/up N(0, 0.02), bias N(0, 0.01)."""
    g = torch.Generator().manual_seed(seed)
    codes = torch.randint(-8, 8, (N, K), generator=g, dtype=torch.int32)
    return {
        "qweight": pack_int4(codes).view(torch.int8),
        "wscales": (torch.rand(K // GROUP, N, generator=g) * 0.015 + 0.005).to(dtype),
        "smooth_factor": (torch.rand(K, generator=g) * 3.5 + 0.5).to(dtype),
        "proj_down": (torch.randn(K, R, generator=g) * 0.02).to(dtype),
        "proj_up": (torch.randn(N, R, generator=g) * 0.02).to(dtype),
        "bias": (torch.randn(N, generator=g) * 0.01).to(dtype),
    }


def make_activations(M: int, K: int, seed: int = 1, dtype=torch.bfloat16) -> torch.Tensor:
    """N(0, 1) activations with 1 % of the channels scaled x20 (outlier channels)."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(M, K, generator=g)
    n_out = max(1, round(0.01 * K))
    idx = torch.randperm(K, generator=g)[:n_out]
    x[:, idx] *= 20.0
    return x.to(dtype)


def make_awq_linear(K: int, N: int, seed: int = 2, dtype=torch.bfloat16) -> dict:
    """Stored codes u = w + 8 in [0, 15], scales U(0.005, 0.02), zero-points uniform in [0, 15];
    the stored ``wzeros`` tensor is ``-zp * s`` (nunchaku/models/text_encoders/tinychat_utils.py:187)."""
    g = torch.Generator().manual_seed(seed)
    q = torch.randint(0, 16, (N, K), generator=g, dtype=torch.int32)
    s = (torch.rand(K // GROUP, N, generator=g) * 0.015 + 0.005).to(dtype)
    zp = torch.randint(0, 16, (K // GROUP, N), generator=g).float()
    return {
        "codes": q,
        "qweight": awq_pack(q).view(torch.int32).reshape(N // 4, K // 2),
        "wscales": s,
        "wzeros": (-(zp * s.float())).to(dtype),
    }


def max_rel_err(a: torch.Tensor, ref: torch.Tensor) -> float:
    """max |a - ref| / max |ref| -- the reference self-test's error measure
    (nunchaku/ops/triton/native/w4a4.py:548-553)."""
    return ((a.float() - ref.float()).abs().max() / ref.float().abs().max().clamp_min(1e-30)).item()


def cosine(a: torch.Tensor, b: torch.Tensor) -> float:
    a, b = a.double().flatten(), b.double().flatten()
    return (a @ b / (a.norm() * b.norm()).clamp_min(1e-300)).item()

