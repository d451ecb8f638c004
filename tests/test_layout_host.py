"""Host logic of checkpoint ingestion that needs no GPU: state-dict key names and the safetensors reader
(reference: nunchaku/models/transformers/transformer_flux_v2.py:579-649, models/transformers/utils.py:32-60)."""

import json

import torch

from nunchaku_rocm_amd import layout


def test_flux_key_names():
    t = torch.zeros(1)
    legacy = {
        "transformer_blocks.0.qkv_proj.qweight": t,
        "transformer_blocks.0.qkv_proj_context.lora_down": t,
        "transformer_blocks.3.out_proj.smooth": t,
        "transformer_blocks.3.out_proj_context.smooth_orig": t,
        "transformer_blocks.1.mlp_fc1.lora_up": t,
        "transformer_blocks.1.mlp_context_fc2.wscales": t,
        "transformer_blocks.2.norm_added_k.weight": t,
        "transformer_blocks.2.norm_q.weight": t,
        "transformer_blocks.2.norm1.linear.qweight": t,
        "single_transformer_blocks.7.qkv_proj.smooth": t,
        "single_transformer_blocks.7.out_proj.bias": t,
        "single_transformer_blocks.7.mlp_fc1.lora_down": t,
        "single_transformer_blocks.7.norm_k.weight": t,
        "x_embedder.weight": t,
    }
    want = {
        "transformer_blocks.0.attn.to_qkv.qweight",
        "transformer_blocks.0.attn.add_qkv_proj.proj_down",
        "transformer_blocks.3.attn.to_out.0.smooth_factor",
        "transformer_blocks.3.attn.to_add_out.smooth_factor_orig",
        "transformer_blocks.1.ff.net.0.proj.proj_up",
        "transformer_blocks.1.ff_context.net.2.wscales",
        "transformer_blocks.2.attn.norm_added_k.weight",
        "transformer_blocks.2.attn.norm_q.weight",
        "transformer_blocks.2.norm1.linear.qweight",
        "single_transformer_blocks.7.attn.to_qkv.smooth_factor",
        "single_transformer_blocks.7.attn.to_out.bias",
        "single_transformer_blocks.7.mlp_fc1.proj_down",
        "single_transformer_blocks.7.attn.norm_k.weight",
        "x_embedder.weight",
    }
    got = layout.convert_flux_state_dict(legacy)
    assert set(got) == want
    assert all(v is t for v in got.values())


def test_load_checkpoint_reads_tensors_and_config(tmp_path):
    from safetensors.torch import save_file

    tensors = {"a.qweight": torch.arange(16, dtype=torch.int8).reshape(4, 4), "a.wscales": torch.ones(2, 4, dtype=torch.bfloat16)}
    config = {"num_layers": 19, "num_single_layers": 38}
    path = tmp_path / "m.safetensors"
    save_file(tensors, str(path), metadata={"config": json.dumps(config), "quantization_config": json.dumps({"weight": {"dtype": "int4"}})})
    sd, meta, cfg = layout.load_checkpoint(path)
    assert cfg == config and "quantization_config" in meta
    assert set(sd) == set(tensors) and torch.equal(sd["a.qweight"], tensors["a.qweight"])
    save_file(tensors, str(path))
    assert layout.load_checkpoint(path)[2] == {}


def test_unpackers_refuse_cpu_tensors_and_fp4():
    import pytest

    with pytest.raises(RuntimeError, match="no CPU implementation"):
        layout.unpack_weight_packed_nibbles(torch.zeros(128, 64, dtype=torch.int8), 128, 128)
    with pytest.raises(NotImplementedError):
        layout.unpack_scale(torch.zeros(8, 128, dtype=torch.bfloat16), 128, group_size=16)


def test_hand_over_layouts_on_the_host():
    """The pure-torch converters of the layouts the quantizer, the requantizing epilogues and the GEMM pass between
    them: inverses of each other, and the documented position of one element each."""
    g = torch.Generator().manual_seed(0)
    a = torch.randint(0, 256, (96, 160), dtype=torch.uint8, generator=g)
    b = layout.block_activations(a)
    assert b.shape == a.shape and torch.equal(layout.unblock_activations(b), a)
    rb, grp, h, r = 2, 3, 1, 7  # lane 32 h + r of (row block, group) = bytes 16 h .. of row 32 rb + r
    assert torch.equal(b.reshape(-1)[((rb * 5 + grp) * 64 + 32 * h + r) * 16 :][:16], a[32 * rb + r, 32 * grp + 16 * h :][:16])
    for unsigned in (False, True):
        c = layout.block_activations_f6(a, unsigned)
        assert c.shape == (96, 240) and torch.equal(layout.unblock_activations_f6(c, unsigned), a)
    c = layout.block_activations_f6(a, False).reshape(-1)
    rb, grp, h, r, p = 1, 2, 0, 9, 21  # code p of lane 32 h + r: value k = 2 p + h, sign << 5 | magnitude, at bits 6 p of 24 bytes
    lane = 32 * h + r
    base = (rb * 5 + grp) * 1536
    vec = bytes(torch.cat([c[base + 16 * lane :][:16], c[base + 1024 + 8 * lane :][:8]]).tolist())
    v = ((int(a[32 * rb + r, 32 * grp + p]) & 15) ^ 8) - 8  # k = 2 p: the low nibble of byte p of the group
    assert (int.from_bytes(vec, "little") >> (6 * p)) & 63 == (32 - v if v < 0 else v)
    s = torch.arange(16 * 96, dtype=torch.float32).reshape(16, 96)
    t = layout.block_scales(s)
    assert t.shape == s.shape and torch.equal(layout.unblock_scales(t), s)
    m, grp = 70, 11  # element ((m / 32) * (G / 8) + g / 8) * 256 + (m % 32) * 8 + g % 8
    assert t.reshape(-1)[((m // 32) * 2 + grp // 8) * 256 + (m % 32) * 8 + grp % 8] == s[grp, m]
