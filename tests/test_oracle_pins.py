"""
Pins for the CPU oracle (no GPU needed).

The reference holds no golden vectors for this path (all of its tests draw inputs at run time on
"cuda"), so every oracle function is pinned here against something its own formula does not
contain: closed-form exact cases, brute force in Python integers, fp64 library routines
(``torch.nn.functional.gelu/silu/rms_norm``, complex multiplication for RoPE), mutual inverses
written from two different statements of a layout, and the independently written scalar C
restatement.  A dropped term, a wrong sign or nibble order, or a transposed operand fails at
least one of them.
"""

import math

import numpy as np
import pytest
import torch

from oracle import c_oracle
from oracle import svdq_oracle as O


# ----------------------------------------------------------------------------- nibbles
def test_unpack_hand_bytes():
    # byte 0xA3: element 0 = low nibble 3, element 1 = high nibble 0xA (= -6 signed)
    # byte 0x8F: element 2 = 0xF (= -1), element 3 = 8 (= -8)
    p = torch.tensor([[0xA3, 0x8F]], dtype=torch.uint8)
    assert O.unpack_int4(p, signed=False).tolist() == [[3, 10, 15, 8]]
    assert O.unpack_int4(p, signed=True).tolist() == [[3, -6, -1, -8]]
    assert O.pack_int4(torch.tensor([[3, -6, -1, -8]])).tolist() == [[0xA3, 0x8F]]


def test_pack_unpack_round_trip():
    g = torch.Generator().manual_seed(0)
    c = torch.randint(-8, 8, (5, 128), generator=g, dtype=torch.int32)
    assert torch.equal(O.unpack_int4(O.pack_int4(c), True), c)
    u = torch.randint(0, 16, (5, 128), generator=g, dtype=torch.int32)
    assert torch.equal(O.unpack_int4(O.pack_int4(u), False), u)


# ----------------------------------------------------------------------------- quantizer
def _pow2_grid_case(unsigned: bool, seed: int):
    """x = s * c / (1/smooth) on power-of-two grids: every fp32 op is exact, so the answer is known."""
    g = torch.Generator().manual_seed(seed)
    M, K = 7, 256
    lo, hi = (0, 15) if unsigned else (-7, 7)
    c = torch.randint(lo, hi + 1, (M, K), generator=g, dtype=torch.int32)
    c.view(M, K // 64, 64)[:, :, 5] = hi  # the group maximum is exactly qmax * s
    e = torch.randint(-6, 3, (M, K // 64), generator=g)
    s = torch.pow(2.0, e.float())
    smooth = torch.pow(2.0, torch.randint(-1, 3, (K,), generator=g).float())
    x = (c.float().view(M, K // 64, 64) * s[:, :, None]).view(M, K) * smooth[None, :]
    return x.to(torch.bfloat16), smooth.to(torch.bfloat16), c, s


@pytest.mark.parametrize("unsigned", [False, True])
def test_quantizer_exact_on_power_of_two_grid(unsigned):
    x, smooth, c, s = _pow2_grid_case(unsigned, 3)
    assert torch.equal(x.float(), x.float().to(torch.bfloat16).float())  # the inputs are exact in bf16
    packed, scales, _, codes = O.quantize_act(x, None, smooth, unsigned=unsigned)
    assert torch.equal(codes, c)
    assert torch.equal(scales.float().t(), s)
    assert torch.equal(O.unpack_int4(packed, not unsigned), c)


def test_quantizer_ties_round_half_to_even():
    # one group, scale exactly 1 (max 7): values k + 0.5 must round like Python's round()
    vals = [-6.5, -5.5, -2.5, -1.5, -0.5, 0.5, 1.5, 2.5, 3.5, 4.5, 5.5, 6.5, 7.0, 0.25, -0.75]
    x = torch.zeros(1, 64)
    x[0, : len(vals)] = torch.tensor(vals)
    _, scales, _, codes = O.quantize_act(x.to(torch.bfloat16))
    assert scales.float().item() == 1.0
    assert codes[0, : len(vals)].tolist() == [int(round(v)) for v in vals]


def test_quantizer_zero_and_nonpositive_groups():
    x = torch.zeros(2, 128, dtype=torch.bfloat16)
    x[0, 64:] = -3.0  # unsigned: all-non-positive group -> scale 0, codes clamp to 0
    x[1, :64] = 2.0
    _, s_u, _, c_u = O.quantize_act(x, unsigned=True)
    assert s_u.float()[1, 0].item() == 0.0 and c_u[0, 64:].abs().sum() == 0
    assert c_u[1, :64].eq(15).all()
    _, s_s, _, c_s = O.quantize_act(x, unsigned=False)
    assert s_s.float()[0, 0].item() == 0.0 and c_s[0, :64].abs().sum() == 0
    assert c_s[0, 64:].eq(-7).all() and c_s[1, :64].eq(7).all()


@pytest.mark.parametrize("unsigned", [False, True])
def test_quantizer_half_step_bound_and_lora(unsigned):
    x = O.make_activations(48, 512, seed=11)
    if unsigned:
        x = x.abs()
    lin = O.make_svdq_linear(512, 64, R=32, seed=12)
    packed, scales, lora, codes = O.quantize_act(x, lin["proj_down"], lin["smooth_factor"], unsigned=unsigned)
    lo, hi = (0, 15) if unsigned else (-8, 7)
    assert codes.min() >= lo and codes.max() <= hi
    # dequantised with the *unrounded* scale the error is at most half a step (fp64 arithmetic here)
    v = x.double() / lin["smooth_factor"].double()[None, :]
    vg = v.view(48, 8, 64)
    gmax = vg.amax(-1) if unsigned else vg.abs().amax(-1)
    step = gmax / (15 if unsigned else 7)
    err = (codes.double().view(48, 8, 64) * step[..., None] - vg).abs()
    assert (err <= 0.5 * step[..., None] * (1 + 1e-5) + 1e-12).all()
    # stored scale = bf16(step)
    assert ((scales.float().t().double() - step).abs() <= step * 2**-8).all()
    # LoRA-down is the plain product on the un-smoothed input
    ref = x.double() @ lin["proj_down"].double()
    assert (lora.double() - ref).abs().max() <= 1e-5 * ref.abs().max()


@pytest.mark.parametrize("unsigned,shift", [(False, 0.0), (True, 0.171875)])
def test_quantizer_matches_c_restatement_bit_exact(unsigned, shift):
    x = O.make_activations(40, 384, seed=21)
    if unsigned:
        x = (x.float().abs() * 0.1 - 0.1).to(torch.bfloat16)
    lin = O.make_svdq_linear(384, 64, R=16, seed=22)
    packed, scales, lora, _ = O.quantize_act(x, lin["proj_down"], lin["smooth_factor"], unsigned=unsigned, shift=shift)
    c_packed, c_scales, c_lora = c_oracle.quantize_act(x, lin["smooth_factor"], lin["proj_down"], unsigned, shift)
    assert torch.equal(packed, c_packed)
    assert torch.equal(scales.view(torch.int16), c_scales.view(torch.int16))
    assert (lora - c_lora).abs().max() <= 1e-5 * lora.abs().max()


def _rcp_order_input():
    import os
    import sys

    sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden"))
    from rcp_order_vectors import VECTORS, expected

    x = torch.zeros(len(VECTORS), 64, dtype=torch.float32)
    want = []
    for i, (v, gmax) in enumerate(VECTORS):
        x[i, 0], x[i, 1 + i] = gmax, v
        by_rcp, by_div = expected(v, gmax)
        assert by_rcp != by_div  # the vector does tell the two orders apart
        want.append(by_rcp)
    xb = x.to(torch.bfloat16)
    assert torch.equal(xb.float(), x)  # the values are bf16
    return xb, want


def test_quantizer_multiplies_by_the_reciprocal():
    """``x * (1 / scale)``, not ``x / scale`` (nunchaku/ops/triton/gemm_w4a4.py:1440): on these inputs the two give
    different codes, and the expected ones come from exact rational arithmetic (tests/golden/rcp_order_vectors.py), not from
    a restatement of the formula in floating point."""
    xb, want = _rcp_order_input()
    _, _, _, codes = O.quantize_act(xb)
    packed_c, _, _ = c_oracle.quantize_act(xb)
    codes_c = O.unpack_int4(packed_c, True)
    for i, w in enumerate(want):
        assert int(codes[i, 1 + i]) == w, (i, int(codes[i, 1 + i]), w)
        assert int(codes_c[i, 1 + i]) == w, (i, int(codes_c[i, 1 + i]), w)
        assert int(codes[i, 0]) == 7


# ----------------------------------------------------------------------------- integer group dots, GEMM
@pytest.mark.parametrize("act_unsigned", [False, True])
def test_group_acc_brute_force(act_unsigned):
    g = torch.Generator().manual_seed(5)
    M, N, K = 3, 4, 128
    act = torch.randint(0, 256, (M, K // 2), generator=g, dtype=torch.uint8)
    wgt = torch.randint(0, 256, (N, K // 2), generator=g, dtype=torch.uint8)
    p = O.group_acc_i32(act, wgt, act_unsigned)

    def nib(row, k, signed):
        v = (int(row[k // 2]) >> (4 * (k % 2))) & 0xF
        return v - 16 if signed and v >= 8 else v

    for gi in range(K // 64):
        for m in range(M):
            for n in range(N):
                s = sum(nib(act[m], k, not act_unsigned) * nib(wgt[n], k, True) for k in range(gi * 64, gi * 64 + 64))
                assert p[gi, m, n].item() == s
        assert torch.equal(c_oracle.group_acc_i32(act, wgt, gi, act_unsigned), p[gi])


@pytest.mark.parametrize("act_unsigned", [False, True])
def test_gemm_unit_scales_is_exact_integer_gemm(act_unsigned):
    g = torch.Generator().manual_seed(6)
    M, N, K = 16, 24, 256
    act = torch.randint(0, 256, (M, K // 2), generator=g, dtype=torch.uint8)
    wgt = torch.randint(0, 256, (N, K // 2), generator=g, dtype=torch.uint8)
    one_a = torch.ones(K // 64, M, dtype=torch.bfloat16)
    one_w = torch.ones(K // 64, N, dtype=torch.bfloat16)
    out = O.gemm_w4a4(act, wgt, one_a, one_w, act_unsigned=act_unsigned)
    a = O.unpack_int4(act, not act_unsigned).numpy().astype(np.int64)
    w = O.unpack_int4(wgt, True).numpy().astype(np.int64)
    assert np.array_equal(out.numpy().astype(np.int64), a @ w.T)


def test_gemm_fp64_closed_form_and_c_restatement():
    g = torch.Generator().manual_seed(7)
    M, N, K, R = 20, 12, 256, 16
    act = torch.randint(0, 256, (M, K // 2), generator=g, dtype=torch.uint8)
    wgt = torch.randint(0, 256, (N, K // 2), generator=g, dtype=torch.uint8)
    asc = (torch.rand(K // 64, M, generator=g) * 0.05 + 0.01).to(torch.bfloat16)
    wsc = (torch.rand(K // 64, N, generator=g) * 0.05 + 0.01).to(torch.bfloat16)
    bias = torch.randn(N, generator=g).to(torch.bfloat16)
    la = torch.randn(M, R, generator=g)
    lu = (torch.randn(N, R, generator=g) * 0.1).to(torch.bfloat16)
    out = O.gemm_w4a4(act, wgt, asc, wsc, bias, la, lu)
    # dense fp64: dequantise both operands element by element, one big matmul
    grp = torch.arange(K) // 64
    a = O.unpack_int4(act, True).double() * asc.double()[grp].t()
    w = O.unpack_int4(wgt, True).double() * wsc.double()[grp].t()
    ref = a @ w.t() + la.to(torch.bfloat16).double() @ lu.double().t() + bias.double()
    assert (out.double() - ref).abs().max() <= 2e-6 * ref.abs().max()
    # without LoRA the torch and C restatements perform the same fp32 ops in the same order
    o1 = O.gemm_w4a4(act, wgt, asc, wsc, bias)
    o2 = c_oracle.gemm_w4a4(act, wgt, asc, wsc, bias)
    assert torch.equal(o1, o2)
    o3 = c_oracle.gemm_w4a4(act, wgt, asc, wsc, bias, la, lu)
    assert (o3 - out).abs().max() <= 1e-5 * out.abs().max()


# ----------------------------------------------------------------------------- epilogues
def test_gelu_and_silu_match_library_fp64():
    x = torch.linspace(-8, 8, 4001)
    ref = torch.nn.functional.gelu(x.double(), approximate="tanh")
    assert (O.gelu_tanh(x).double() - ref).abs().max() < 2e-6
    assert (O.silu(x).double() - torch.nn.functional.silu(x.double())).abs().max() < 2e-6


def test_qk_norm_rope_against_complex_rotation():
    g = torch.Generator().manual_seed(8)
    M, H = 9, 2
    N = 3 * H * 128
    lin = torch.randn(M, N, generator=g)
    nq = (torch.rand(128, generator=g) + 0.5).to(torch.bfloat16)
    nk = (torch.rand(128, generator=g) + 0.5).to(torch.bfloat16)
    theta = torch.rand(M, 64, generator=g, dtype=torch.float64) * 6.28
    rot = torch.stack([torch.sin(theta), torch.cos(theta)], -1).float().reshape(M, 128)
    out = O.qk_norm_rope(lin, nq, nk, rot)
    x = lin.double().view(M, 3, H, 128)
    for part, w in ((0, nq), (1, nk)):
        h = torch.nn.functional.rms_norm(x[:, part], (128,), w.double(), eps=1e-6)
        z = torch.view_as_complex(h.reshape(M, H, 64, 2).contiguous())
        rz = z * torch.polar(torch.ones_like(theta), theta)[:, None]
        ref = torch.view_as_real(rz).reshape(M, H, 128)
        assert (out.view(M, 3, H, 128)[:, part].double() - ref).abs().max() < 2e-5
    assert torch.equal(out.view(M, 3, H * 128)[:, 2], lin.view(M, 3, H * 128)[:, 2])


def test_gelu_quant_is_quantizer_of_library_gelu():
    g = torch.Generator().manual_seed(9)
    M, N, R2 = 12, 256, 16
    lin = torch.randn(M, N, generator=g) * 2
    smooth = (torch.rand(N, generator=g) + 0.5).to(torch.bfloat16)
    ld = (torch.randn(N, R2, generator=g) * 0.1).to(torch.bfloat16)
    packed, scales, lora, codes = O.gelu_quant(lin, smooth, ld, torch.bfloat16)
    gl = torch.nn.functional.gelu(lin.double(), approximate="tanh")
    v = (gl + 0.171875) / smooth.double()
    step = v.view(M, N // 64, 64).amax(-1).clamp_min(0) / 15
    ref = torch.round(v.view(M, N // 64, 64) / step[..., None]).clamp(0, 15).view(M, N)
    diff = (codes.double() - ref).abs()
    assert diff.max() <= 1 and (diff > 0).double().mean() < 1e-3
    assert ((scales.float().t().double() - step).abs() <= step * 2**-8 + 1e-12).all()
    refl = gl.float().to(torch.bfloat16).double() @ ld.double()
    assert (lora.double() - refl).abs().max() <= 1e-4 * refl.abs().max()
    assert codes.min() >= 0  # gelu >= -0.17 so the shifted value is positive


def test_swiglu_interleave_and_quant():
    n = 128
    idx = O.interleave_swiglu(n)
    assert sorted(idx.tolist()) == list(range(n))
    cols = torch.arange(n).float()[idx].view(n // 32, 2, 16)  # what out.view(M, n//32, 2, 16) sees
    assert torch.equal(cols[:, 0].flatten(), torch.arange(n // 2).float())  # gate rows in order
    assert torch.equal(cols[:, 1].flatten(), torch.arange(n // 2, n).float())  # up rows in order
    g = torch.Generator().manual_seed(10)
    M = 6
    lin = torch.randn(M, n, generator=g)  # [gate | up]
    smooth = (torch.rand(n // 2, generator=g) + 0.5).to(torch.bfloat16)
    _, scales, _, codes = O.swiglu_quant(lin[:, idx], smooth, None, torch.bfloat16)
    y = torch.nn.functional.silu(lin[:, : n // 2].double()) * lin[:, n // 2 :].double() / smooth.double()
    step = y.abs().view(M, 1, 64).amax(-1) / 7
    ref = torch.round(y.view(M, 1, 64) / step[..., None]).clamp(-8, 7).view(M, 64)
    assert (codes.double() - ref).abs().max() <= 1 and (codes.double() != ref).double().mean() < 1e-2


# ----------------------------------------------------------------------------- AWQ
def test_awq_pack_decode_inverse_and_gemv_kernel_statement():
    g = torch.Generator().manual_seed(13)
    N, K = 16, 128
    q = torch.randint(0, 16, (N, K), generator=g, dtype=torch.int32)
    packed = O.awq_pack(q)
    assert packed.shape == (N // 4, K) and packed.dtype == torch.int16
    assert torch.equal(O.awq_decode(packed, N, K), q)
    # third statement of the layout (the streaming GEMV's, nunchaku/ops/triton/awq.py:137-144):
    # stored column e = 64c + 16b + d of packed row a, nibble m <-> (n, k) = (4a + b, 64c + 32(d//8) + 8m + d%8)
    pu = packed.to(torch.int32) & 0xFFFF
    for a in range(N // 4):
        for e in range(K):
            c, b, d = e // 64, (e % 64) // 16, e % 16
            for m in range(4):
                assert ((pu[a, e].item() >> (4 * m)) & 0xF) == q[4 * a + b, 64 * c + 32 * (d // 8) + 8 * m + d % 8].item()
    pk = packed.contiguous()
    lib = c_oracle.lib()
    for n in range(N):
        for k in range(0, K, 7):
            assert lib.oracle_awq_nibble(c_oracle._p(pk), K, n, k) == q[n, k].item()


@pytest.mark.parametrize("m", [1, 3])
def test_awq_gemv_fp64_dense(m):
    lin = O.make_awq_linear(256, 64, seed=14)
    g = torch.Generator().manual_seed(15)
    x = torch.randn(m, 256, generator=g).to(torch.bfloat16)
    packed = lin["qweight"].view(torch.int16).reshape(16, 256)
    out = O.awq_gemv(x, packed, lin["wscales"], lin["wzeros"])
    grp = torch.arange(256) // 64
    w = lin["codes"].double() * lin["wscales"].double()[grp].t() + lin["wzeros"].double()[grp].t()
    ref = x.double() @ w.t()
    assert (out.double() - ref).abs().max() <= 1e-5 * ref.abs().max()
    out_c = c_oracle.awq_gemv(x, packed, lin["wscales"], lin["wzeros"])
    assert (out_c - out).abs().max() <= 1e-5 * ref.abs().max()


@pytest.mark.parametrize("group_size", [32, 64, 128])
def test_awq_dequantize_fp64_and_zero_point(group_size):
    K, N = 256, 32
    g = torch.Generator().manual_seed(16)
    q = torch.randint(0, 16, (N, K), generator=g, dtype=torch.int32)
    s = (torch.rand(K // group_size, N, generator=g) * 0.015 + 0.005).to(torch.bfloat16)
    zp = torch.randint(0, 16, (K // group_size, N), generator=g)
    z = (-zp.float() * s.float()).to(torch.bfloat16)
    w = O.awq_dequantize(O.awq_pack(q), s, z, group_size)
    assert w.shape == (N, K) and w.dtype == torch.bfloat16
    grp = torch.arange(K) // group_size
    # q * s has at most 12 significant bits: the fp64 value of q * s + z is exact, so rounding it to fp32 and then to
    # bf16 is what fp32 arithmetic gives
    ref = (q.double() * s.double().t()[:, grp] + z.double().t()[:, grp]).float().to(torch.bfloat16)
    assert torch.equal(w, ref)
    # where the code equals the zero point the weight is the rounding error of -zp * s only
    hit = q == zp.t()[:, grp]
    assert hit.any() and (w[hit].float().abs() <= s.float().t()[:, grp][hit] * 16 * 2**-8).all()
    # codes that differ by one within a group differ by the scale (up to output rounding)
    w2 = O.awq_dequantize(O.awq_pack((q + 1).clamp(max=15)), s, z, group_size)
    step = (w2.float() - w.float())[q < 15]
    assert ((step - s.float().t()[:, grp][q < 15]).abs() <= 2**-7 * (w.float().abs()[q < 15] + s.float().max())).all()


# ----------------------------------------------------------------------------- FLUX rotary table
def test_flux_rotary_closed_form():
    ids = O.flux_ids(4, 3, 5)
    assert ids.shape == (4 + 15, 3) and ids[:4].abs().sum() == 0
    assert ids[4 + 1 * 5 + 2].tolist() == [0.0, 1.0, 2.0]
    rot = O.flux_rotary(ids)
    assert rot.shape == (19, 64, 1, 2) and rot.dtype == torch.float32
    t = 4 + 2 * 5 + 3  # h = 2, w = 3
    for pair, (axis_pos, d, i) in {0: (0.0, 16, 0), 8 + 5: (2.0, 56, 5), 8 + 28 + 27: (3.0, 56, 27)}.items():
        ang = axis_pos * 10000.0 ** (-(2 * i) / d)
        assert abs(rot[t, pair, 0, 0].item() - math.sin(ang)) < 1e-6
        assert abs(rot[t, pair, 0, 1].item() - math.cos(ang)) < 1e-6


# ---- attention ------------------------------------------------------------------------------------------------------
def _attn_inputs(B, H, Tq, Tkv, dtype, seed, spread=1.0):
    g = torch.Generator().manual_seed(seed)
    q = (torch.randn(B, H, Tq, 128, generator=g) * spread).to(dtype)
    k = (torch.randn(B, H, Tkv, 128, generator=g) * spread).to(dtype)
    v = torch.randn(B, H, Tkv, 128, generator=g).to(dtype)
    return q, k, v


def _attn_fp64(q, k, v, scale):
    w = torch.softmax(q.double() @ k.double().transpose(-1, -2) * scale, dim=-1)
    o = w @ v.double()
    return o.transpose(1, 2).reshape(q.shape[0], q.shape[2], -1)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("Tq,Tkv,block", [(70, 200, 64), (33, 64, 64), (5, 131, 32), (40, 77, 128)])
def test_attention_against_fp64_softmax(dtype, Tq, Tkv, block):
    q, k, v = _attn_inputs(2, 3, Tq, Tkv, dtype, seed=Tq + Tkv, spread=1.5)
    scale = 128**-0.5
    got = O.attention_fp16(q, k, v, scale, block_n=block).double()
    ref = _attn_fp64(q, k, v, scale)
    # the only roundings are q * scale, p and the output, each to the 16-bit type: 2^-8 relative for bf16
    tol = 2e-2 if dtype == torch.bfloat16 else 3e-3
    assert (got - ref).abs().max() <= tol * ref.abs().max()
    assert got.shape == (2, Tq, 3 * 128)


def test_attention_special_cases():
    scale = 128**-0.5
    q, k, v = _attn_inputs(1, 2, 16, 96, torch.float16, seed=5)
    # q = 0: uniform weights, the output is the mean of v over the keys (heads side by side in the last dimension)
    o = O.attention_fp16(torch.zeros_like(q), k, v, scale, block_n=32).double()
    mean = v.double().mean(dim=2)  # (1, 2, 128)
    assert (o - mean.reshape(1, 1, 256)).abs().max() < 2e-3
    # constant v rows: any weights return that row
    vc = v[:, :, :1].expand_as(v).contiguous()
    o = O.attention_fp16(q, k, vc, scale).double()
    assert (o - vc[:, :, 0].double().reshape(1, 1, 256)).abs().max() < 2e-3
    # one key dominates query t: the output row is that key's v (key index differs per query: a transposed or
    # mis-indexed product cannot pass)
    kk = torch.zeros(1, 2, 96, 128)
    qq = torch.zeros(1, 2, 16, 128)
    for t in range(16):
        qq[0, :, t, t] = 60.0
        kk[0, 0, 3 * t + 1, t] = 60.0
        kk[0, 1, 95 - 2 * t, t] = 60.0
    o = O.attention_fp16(qq.half(), kk.half(), v, scale, block_n=32).float()
    for t in range(16):
        assert torch.allclose(o[0, t, :128], v[0, 0, 3 * t + 1].float(), atol=1e-3)
        assert torch.allclose(o[0, t, 128:], v[0, 1, 95 - 2 * t].float(), atol=1e-3)
    # the key block size is an implementation choice: results agree to the rounding of p
    q, k, v = _attn_inputs(1, 1, 48, 300, torch.bfloat16, seed=9, spread=2.0)
    a = O.attention_fp16(q, k, v, scale, block_n=16).float()
    b = O.attention_fp16(q, k, v, scale, block_n=300).float()
    assert (a - b).abs().max() <= 2e-2 * b.abs().max()


# ---- checkpoint packer ----------------------------------------------------------------------------------------------
def test_pack_weight_fragment_rule_and_hand_positions():
    """mma.m16n8k32 B fragment (PTX ISA, 'Matrix Fragments for mma.m16n8k32'): lane = 4 * groupID + threadID_in_group
    owns column n = groupID and rows k = 8 * threadID_in_group .. + 7 of an 8 x 32 block, in one 32-bit register."""
    from oracle import mma_packer as P

    n, k = 256, 256
    codes = np.zeros((n, k), dtype=np.int32)
    tag = (np.arange(n)[:, None] * 7 + np.arange(k)[None, :] // 8) % 16  # constant over the 8 k of one word
    codes[:] = tag
    words = P.pack_weight(codes).view(np.uint32).reshape(-1)
    assert (words % 0x11111111 == 0).all()  # every word holds eight equal nibbles: words never mix rows or k-octets
    # word positions worked out by hand from the axis order [n_tile, k_tile, n_packs, n_lane, k_lane, n_pack, k_pack]
    where = {0: (0, 0), 1: (0, 32), 2: (8, 0), 3: (8, 32), 4: (0, 8), 16: (1, 0), 17: (1, 32), 128: (16, 0), 1024: (0, 64), 1024 * 4: (128, 0)}
    for w, (nn, kk) in where.items():
        assert words[w] == int(tag[nn, kk]) * 0x11111111, (w, nn, kk)
    # inside an 8 x 32 block: consecutive 4-word groups [n_pack, k_pack] of lane L = 4 * (n % 8) + (k / 8) % 4
    for lane in range(32):
        nn, kk = lane // 4, 8 * (lane % 4)
        assert words[4 * lane] == int(tag[nn, kk]) * 0x11111111
    # nibble order inside a word: k + j in bits 4 j
    codes = np.arange(n * k, dtype=np.int64).reshape(n, k) % 16
    b = P.pack_weight(codes.astype(np.int32))
    assert [int(b[0, 0]) & 0xF, int(b[0, 0]) >> 4, int(b[0, 1]) & 0xF] == [0, 1, 2]
    # a permutation of words: every (row, k-octet) appears exactly once
    ids = (np.arange(n)[:, None] * (k // 8) + np.arange(k)[None, :] // 8).astype(np.int64)
    seen = np.zeros(n * k // 8, dtype=np.int64)
    for nib in range(4):  # 16 bits of id, 4 bits at a time
        w = P.pack_weight(((ids >> (4 * nib)) & 0xF).astype(np.int32)).view(np.uint32).reshape(-1)
        seen |= (w & 0xF).astype(np.int64) << (4 * nib)
    assert sorted(seen.tolist()) == list(range(n * k // 8))


def test_pack_scale_and_lowrank_hand_positions():
    from oracle import mma_packer as P

    n, g = 256, 3
    s = (np.arange(n)[:, None] * 10 + np.arange(g)[None, :]).astype(np.float32)
    flat = P.pack_scale(s)
    # [n_group][g][a (8)][c (4)][b (2)][d (2)] with n = 16 a + 8 b + 2 c + d: positions 0..7 of a group hold
    # n = 0, 1, 8, 9, 2, 3, 10, 11
    assert (flat[:8] == s[[0, 1, 8, 9, 2, 3, 10, 11], 0]).all()
    assert (flat[128 : 128 + 4] == s[[0, 1, 8, 9], 1]).all()  # next group of the same 128 rows
    assert flat[3 * 128] == s[128, 0]  # next 128 rows
    assert sorted(flat.tolist()) == sorted(s.reshape(-1).tolist())
    v = np.arange(128, dtype=np.float32)
    assert (P.pack_scale(v)[:8] == [0, 1, 8, 9, 2, 3, 10, 11]).all()

    # low-rank, up factor (N, R): block (cp, rp) of 16 x 16, inside [n_lane 8][k_lane 4][n_pack 2][k_pack 2][2]
    N, R = 32, 32
    up = (np.arange(N)[:, None] * 100 + np.arange(R)[None, :]).astype(np.float32)
    pu = P.pack_lowrank_weight(up, down=False).reshape(-1)
    assert pu[:8].tolist() == [up[0, 0], up[0, 1], up[0, 8], up[0, 9], up[8, 0], up[8, 1], up[8, 8], up[8, 9]]
    assert pu[8] == up[0, 2] and pu[32] == up[1, 0]
    assert pu[256] == up[0, 16] and pu[512] == up[16, 0]  # blocks: rank blocks inside row blocks
    # down factor: packed from (rank, in_features), viewed (in_features, rank); the reference's inverse
    # (packer.py:340-373) restated as a loop gives the logical tensor back
    K = 48
    dn = (np.arange(R)[:, None] * 100 + np.arange(K)[None, :]).astype(np.float32)  # (rank, in_features)
    pd = P.pack_lowrank_weight(dn, down=True)
    assert pd.shape == (K, R)
    flat = pd.reshape(-1)
    assert flat[:4].tolist() == [dn[0, 0], dn[0, 1], dn[0, 8], dn[0, 9]] and flat[4] == dn[8, 0]
    assert flat[256] == dn[16, 0] and flat[512] == dn[0, 16]  # blocks: rank blocks inside in-feature blocks
    back = np.zeros_like(dn)
    for cp in range(K // 16):
        for rp in range(R // 16):
            blk = flat[(cp * (R // 16) + rp) * 256 :][:256].reshape(8, 4, 2, 2, 2)  # [n_lane][k_lane][n_pack][k_pack][e]
            for nl in range(8):
                for kl in range(4):
                    for ns in range(2):
                        for ks in range(2):
                            for e in range(2):
                                back[rp * 16 + ns * 8 + nl, cp * 16 + ks * 8 + kl * 2 + e] = blk[nl, kl, ns, ks, e]
    assert (back == dn).all()


# ---- LayerNorm + modulate -------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_layernorm_modulate_against_library(dtype):
    g = torch.Generator().manual_seed(3)
    M, K = 48, 384
    x = (torch.randn(M, K, generator=g) * 2 + 0.7).to(dtype)
    scale = (1 + 0.3 * torch.randn(2, K, generator=g)).to(dtype)
    shift = (0.2 * torch.randn(2, K, generator=g)).to(dtype)
    got = O.layernorm_modulate(x, scale, shift)
    # the mathematics, in fp64, with the batch split written out (rows 0..23 use vector 0)
    n64 = torch.nn.functional.layer_norm(x.double(), (K,), eps=1e-6)
    ref64 = torch.cat([n64[:24] * scale[0].double() + shift[0].double(), n64[24:] * scale[1].double() + shift[1].double()])
    ulp = 2**-7 if dtype == torch.bfloat16 else 2**-10
    assert ((got.double() - ref64).abs() <= 3 * ulp * ref64.abs() + 3 * ulp).all()
    # the rounding sequence: torch's own 16-bit CPU kernels, one op at a time
    lib = torch.nn.functional.layer_norm(x, (K,), eps=1e-6)
    lib = torch.cat([lib[:24] * scale[0] + shift[0], lib[24:] * scale[1] + shift[1]])
    mism = (got.view(torch.int16) != lib.view(torch.int16)).float().mean().item()
    assert mism < 2e-3 and (got.float() - lib.float()).abs().max() <= 2 * ulp * lib.float().abs().max()
    # a constant row has zero variance: the output is the shift
    xc = torch.full((16, K), 1.5).to(dtype)
    assert torch.equal(O.layernorm_modulate(xc, scale[0], shift[0]), shift[:1].expand(16, K).contiguous())


def test_gated_residual_is_torchs_op_sequence():
    g = torch.Generator().manual_seed(4)
    for dtype in (torch.bfloat16, torch.float16):
        x, y, y2 = (torch.randn(2, 5, 64, generator=g).to(dtype) for _ in range(3))
        gate = torch.randn(2, 64, generator=g).to(dtype)
        assert torch.equal(O.gated_residual(x, gate, y), x + gate.unsqueeze(1) * y)
        assert torch.equal(O.gated_residual(x, gate, y, y2), x + gate.unsqueeze(1) * (y + y2))
