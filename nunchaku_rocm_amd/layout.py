"""Checkpoint ingestion: tensors as the published SVDQuant int4 checkpoints hold them -> the natural layouts of
``SVDQW4A4Linear`` (reference: nunchaku/ops/triton/layout.py:36-292; state-dict key names:
nunchaku/models/transformers/transformer_flux_v2.py:579-649; file metadata: nunchaku/models/transformers/utils.py:32-60).

The permutations run on the GPU through ``libsvdq_mi355x.so`` (``svdq_unpack_mma_*``): tensors must be CUDA tensors.
Only the int4 format is handled; the NVFP4 micro-scale layout (group size 16) is not.
"""

from __future__ import annotations

import json

import torch

from . import _lib

__all__ = [
    "unpack_weight",
    "unpack_weight_packed_nibbles",
    "unpack_scale",
    "unpack_lowrank_weight",
    "convert_svdq_linear_to_natural_layout",
    "convert_flux_state_dict",
    "load_checkpoint",
    "join_weight_planes",
]


def _flat16(t: torch.Tensor) -> torch.Tensor:
    if t.dtype not in (torch.float16, torch.bfloat16):
        raise ValueError(f"expected a float16 / bfloat16 tensor, got {t.dtype}")
    return t.contiguous()


def unpack_weight_packed_nibbles(packed: torch.Tensor, n: int, k: int, bits: int = 4) -> torch.Tensor:
    """Checkpoint ``qweight`` ``(n, k // 2)`` int8 -> natural ``(n, k // 2)`` uint8, column ``2 j`` in the low nibble
    of byte ``j``.  ``n`` and ``k`` are the padded sizes (multiples of 128)."""
    if bits != 4:
        raise NotImplementedError("packed-nibble output is only defined for 4-bit codes")
    _lib.require_cuda(packed)
    if packed.numel() * packed.element_size() != n * k // 2:
        raise ValueError(f"packed weight holds {packed.numel() * packed.element_size()} bytes, expected {n * k // 2}")
    src = packed.contiguous()
    out = torch.empty(n, k // 2, dtype=torch.uint8, device=packed.device)
    with torch.cuda.device(packed.device):
        _lib.check(_lib.load().svdq_unpack_mma_weight(src.data_ptr(), out.data_ptr(), n, k, k // 2, _lib.stream_of(src)))
    return out


def unpack_weight(packed: torch.Tensor, n: int, k: int, bits: int = 4) -> torch.Tensor:
    """Checkpoint ``qweight`` -> logical ``(n, k)`` int32 codes in ``[0, 16)`` (not sign-interpreted)."""
    b = unpack_weight_packed_nibbles(packed, n, k, bits=bits).to(torch.int32)
    return torch.stack([b & 0xF, b >> 4], dim=-1).reshape(n, k)


def unpack_scale(packed: torch.Tensor, n: int, group_size: int, bits: int = 4, warp_n: int = 128) -> torch.Tensor:
    """Checkpoint scale tensor -> ``(k // group_size, n)`` (``wscales``), or ``(n,)`` for ``group_size=-1`` (``bias``,
    ``smooth_factor``, ``wcscales``: the checkpoint keeps them in the same lane order)."""
    if bits != 4 or warp_n != 128:
        raise NotImplementedError("only the 4-bit packer with warp_n = 128 is implemented")
    if group_size == 16:
        raise NotImplementedError("NVFP4 micro-scales (group size 16) are not implemented: int4 checkpoints only")
    _lib.require_cuda(packed)
    src = _flat16(packed)
    groups = 1 if group_size == -1 else src.numel() // n
    if groups * n != src.numel():
        raise ValueError(f"scale tensor of {src.numel()} elements does not divide into rows of {n}")
    out = torch.empty(groups, n, dtype=src.dtype, device=src.device)
    with torch.cuda.device(src.device):
        _lib.check(_lib.load().svdq_unpack_mma_scale(src.data_ptr(), out.data_ptr(), n, groups, n, _lib.stream_of(src)))
    return out.reshape(n) if group_size == -1 else out


def unpack_lowrank_weight(weight: torch.Tensor, down: bool) -> torch.Tensor:
    """Checkpoint low-rank factor -> natural: ``down=False``: ``proj_up`` ``(out_features, rank)``; ``down=True``:
    the checkpoint's ``(in_features, rank)`` tensor -> ``proj_down`` ``(in_features, rank)``.  (The reference's packer
    method of this name returns ``(rank, in_features)`` for ``down=True`` and its caller transposes; here the
    transposed result comes out directly.)"""
    _lib.require_cuda(weight)
    src = _flat16(weight)
    c, r = src.shape
    out = torch.empty(c, r, dtype=src.dtype, device=src.device)
    with torch.cuda.device(src.device):
        _lib.check(_lib.load().svdq_unpack_mma_lowrank(src.data_ptr(), out.data_ptr(), c, r, int(bool(down)), r, _lib.stream_of(src)))
    return out


def convert_svdq_linear_to_natural_layout(linear) -> None:
    """Convert one ``SVDQW4A4Linear`` in place from the checkpoint layout to the natural one.  Call exactly once per
    loaded module: the conversion is not idempotent.  ``smooth_factor_orig`` is not read by any kernel and is left
    as it is."""
    n, half_k = linear.qweight.shape
    k = 2 * half_k
    with torch.no_grad():
        linear.qweight.data = unpack_weight_packed_nibbles(linear.qweight.data, n, k).view(torch.int8)
        linear.wscales.data = unpack_scale(linear.wscales.data, n, group_size=linear.group_size)
        if linear.bias is not None:
            linear.bias.data = unpack_scale(linear.bias.data, n, group_size=-1)
        linear.smooth_factor.data = unpack_scale(linear.smooth_factor.data, k, group_size=-1)
        if getattr(linear, "wcscales", None) is not None:
            linear.wcscales.data = unpack_scale(linear.wcscales.data, n, group_size=-1)
        if linear.proj_down.numel() > 0:
            linear.proj_down.data = unpack_lowrank_weight(linear.proj_down.data, down=True)
        if linear.proj_up.numel() > 0:
            linear.proj_up.data = unpack_lowrank_weight(linear.proj_up.data, down=False)


# legacy FLUX checkpoint module names -> names of the diffusers-style model, per block family; first match wins
_DOUBLE_BLOCK_NAMES = (
    (".mlp_context_fc1.", ".ff_context.net.0.proj."),
    (".mlp_context_fc2.", ".ff_context.net.2."),
    (".mlp_fc1.", ".ff.net.0.proj."),
    (".mlp_fc2.", ".ff.net.2."),
    (".qkv_proj_context.", ".attn.add_qkv_proj."),
    (".qkv_proj.", ".attn.to_qkv."),
    (".norm_added_q.", ".attn.norm_added_q."),
    (".norm_added_k.", ".attn.norm_added_k."),
    (".norm_q.", ".attn.norm_q."),
    (".norm_k.", ".attn.norm_k."),
    (".out_proj_context.", ".attn.to_add_out."),
    (".out_proj.", ".attn.to_out.0."),
)
_SINGLE_BLOCK_NAMES = (
    (".qkv_proj.", ".attn.to_qkv."),
    (".out_proj.", ".attn.to_out."),
    (".norm_q.", ".attn.norm_q."),
    (".norm_k.", ".attn.norm_k."),
)


def _rename(key: str, table) -> str:
    for old, new in table:
        if old in key:
            key = key.replace(old, new)
            break
    return key


def convert_flux_state_dict(state_dict: dict[str, torch.Tensor]) -> dict[str, torch.Tensor]:
    """Rename the keys of a legacy FLUX SVDQuant checkpoint to the names ``NunchakuFluxTransformer2DModelV2`` uses;
    tensors are passed through untouched, keys outside the transformer blocks keep their names."""
    out = {}
    for key, value in state_dict.items():
        if "single_transformer_blocks." in key:
            table = _SINGLE_BLOCK_NAMES
        elif "transformer_blocks." in key:
            table = _DOUBLE_BLOCK_NAMES
        else:
            out[key] = value
            continue
        new_key = _rename(key, table)
        new_key = new_key.replace(".lora_down", ".proj_down").replace(".lora_up", ".proj_up")
        if ".smooth_orig" in key:
            new_key = new_key.replace(".smooth_orig", ".smooth_factor_orig")
        elif ".smooth" in key:
            new_key = new_key.replace(".smooth", ".smooth_factor")
        out[new_key] = value
    return out


def load_checkpoint(path, device: str | torch.device = "cpu") -> tuple[dict[str, torch.Tensor], dict[str, str], dict]:
    """Read one ``.safetensors`` checkpoint: ``(state_dict, metadata, config)`` where ``config`` is the model config
    the file carries as JSON under the ``config`` metadata key (``{}`` if absent)."""
    from safetensors import safe_open

    state_dict = {}
    with safe_open(str(path), framework="pt", device=str(device)) as f:
        metadata = dict(f.metadata() or {})
        for key in f.keys():
            state_dict[key] = f.get_tensor(key)
    config = json.loads(metadata["config"]) if "config" in metadata else {}
    return state_dict, metadata, config


def join_weight_planes(planes: torch.Tensor, n: int, k: int) -> torch.Tensor:
    """Packed ``(n, k // 2)`` int8 weight back from the GEMM's working copy (``svdq_split_weight_planes``): the inverse of
    the code part of that re-layout, for modules that released their packed weight and are asked for it again
    (``state_dict``).  Per (block of 32 rows, stage of two scale groups) the copy holds three 1 KB blocks: lane
    ``parity * 32 + row`` owns, per group, 32 six-bit codes ``sign | magnitude`` (code ``p`` = the nibble of its parity of
    the row's packed byte ``p`` of the group) as 24 little-endian bytes; blocks 0 and 1 = bytes 0-15 of the stage's two
    groups, block 2 = bytes 16-23 of both.  Plain torch operations on the tensor's device; one-off, not fast."""
    nb, G = (n + 31) // 32, k // 64
    nst = (G + 1) // 2
    codes = planes[: nb * nst * 3072].view(nb, nst, 3, 64, 16)
    by = torch.empty(nb, nst, 2, 64, 24, dtype=torch.uint8, device=planes.device)  # (.., group of the stage, lane, byte)
    by[:, :, 0, :, :16] = codes[:, :, 0]
    by[:, :, 1, :, :16] = codes[:, :, 1]
    by[:, :, 0, :, 16:] = codes[:, :, 2, :, :8]
    by[:, :, 1, :, 16:] = codes[:, :, 2, :, 8:]
    shifts = torch.arange(8, dtype=torch.uint8, device=planes.device)
    bits = ((by[..., None] >> shifts) & 1).reshape(nb, nst, 2, 64, 32, 6)  # little-endian bit stream -> 32 codes of 6 bits
    weights = (1 << torch.arange(6, device=planes.device)).to(torch.int16)
    code = (bits.to(torch.int16) * weights).sum(-1)  # (nb, nst, 2, lane, position)
    value = torch.where(code >= 32, -(code - 32), code)  # sign | magnitude -> [-8, 8)
    nib = (value & 0xF).to(torch.uint8).view(nb, nst * 2, 2, 32, 32)  # (nb, group, parity, row, packed byte)
    packed = nib[:, :, 0] | (nib[:, :, 1] << 4)  # (nb, group, row, packed byte)
    packed = packed[:, :G].permute(0, 2, 1, 3).reshape(nb * 32, G * 32)
    return packed[:n].contiguous().view(torch.int8)


def block_activations(act: torch.Tensor) -> torch.Tensor:
    """Packed activations ``(rows, K/2)`` (rows a multiple of 32, K of 64) -> the same bytes in the order the GEMM's fp8
    main loop reads them (what the quantizer writes with ``out_blocked=True``): per 32 rows and group of 64 values 1 KB,
    lane ``32 h + r`` holding bytes ``16 h .. 16 h + 15`` of row ``r``'s 32.  Same shape; pure torch."""
    rows, kb = act.shape
    assert rows % 32 == 0 and kb % 32 == 0, "rows must be a multiple of 32 and K of 64"
    return act.reshape(rows // 32, 32, kb // 32, 2, 16).permute(0, 2, 3, 1, 4).contiguous().reshape(rows, kb)


def block_activations_f6(act: torch.Tensor, unsigned: bool = False) -> torch.Tensor:
    """Packed activations ``(rows, K/2)`` (rows a multiple of 32, K of 64) -> ``(rows, 3K/4)`` bytes: the same values as
    fp6 (e2m3) codes ``sign << 5 | magnitude`` in the order the GEMM's fp8 main loop reads them with ``act_blocked=2``
    (what the quantizer writes with ``out_blocked=2``).  Per 32 rows and group of 64 values 1536 bytes: lane
    ``32 h + r`` owns the 32 values ``k = 2 p + h`` of row ``r``'s group, code ``p`` in bits ``6 p .. 6 p + 5`` of 24
    bytes, whose first 16 lie at byte ``16 lane`` and whose last 8 at byte ``1024 + 8 lane``.  Pure torch."""
    rows, kb = act.shape
    assert rows % 32 == 0 and kb % 32 == 0, "rows must be a multiple of 32 and K of 64"
    a = act.to(torch.int16)
    v = torch.stack([a & 15, a >> 4], dim=-1).reshape(rows, kb * 2)  # nibble values, low nibble = even k
    if not unsigned:
        v = (v ^ 8) - 8
    code = torch.where(v < 0, 32 - v, v)  # sign << 5 | magnitude
    code = code.reshape(rows // 32, 32, kb // 32, 32, 2).permute(0, 2, 4, 1, 3)  # [row block][group][h][r][p]
    bits = (code.unsqueeze(-1) >> torch.arange(6, device=act.device)) & 1  # [...][p][bit]
    bits = bits.reshape(*code.shape[:-1], 24, 8)
    by = (bits << torch.arange(8, device=act.device)).sum(-1).to(torch.uint8)  # [rb][g][h][r][24]
    by = by.reshape(rows // 32, kb // 32, 64, 24)
    out = torch.cat([by[..., :16].reshape(rows // 32, kb // 32, 1024), by[..., 16:].reshape(rows // 32, kb // 32, 512)], dim=-1)
    return out.reshape(rows, kb * 3 // 2)


def unblock_activations_f6(blocked: torch.Tensor, unsigned: bool = False) -> torch.Tensor:
    """Inverse of :func:`block_activations_f6`: ``(rows, 3K/4)`` fp6 codes in lane order -> packed ``(rows, K/2)``.
    (A signed zero decodes to zero whatever its sign bit.)"""
    rows, kb3 = blocked.shape
    assert rows % 32 == 0 and kb3 % 48 == 0, "rows must be a multiple of 32 and K of 64"
    g = kb3 // 48
    b = blocked.reshape(rows // 32, g, 1536)
    by = torch.cat([b[..., :1024].reshape(rows // 32, g, 64, 16), b[..., 1024:].reshape(rows // 32, g, 64, 8)], dim=-1)
    bits = (by.to(torch.int16).unsqueeze(-1) >> torch.arange(8, device=blocked.device)) & 1
    bits = bits.reshape(rows // 32, g, 64, 32, 6)
    code = (bits << torch.arange(6, device=blocked.device)).sum(-1)  # [rb][g][lane][p]
    v = torch.where(code >= 32, -(code - 32), code)
    v = v.reshape(rows // 32, g, 2, 32, 32).permute(0, 3, 1, 4, 2).reshape(rows, g * 32, 2)  # [row][byte][nibble]
    v = v & 15
    return (v[..., 0] | (v[..., 1] << 4)).to(torch.uint8)


def block_scales(scales: torch.Tensor) -> torch.Tensor:
    """Activation scales ``(K/64, rows)`` (K a multiple of 512, rows of 32) -> the same values in the order the GEMM reads
    them with ``act_blocked=3`` (what the quantizer writes with ``out_blocked=3``): per 32 rows and eight groups 512
    bytes, row ``r``'s eight scales side by side at element ``8 r``.  Same shape; pure torch."""
    g, rows = scales.shape
    assert g % 8 == 0 and rows % 32 == 0, "K must be a multiple of 512 and rows of 32"
    return scales.reshape(g // 8, 8, rows // 32, 32).permute(2, 0, 3, 1).contiguous().reshape(g, rows)


def unblock_scales(blocked: torch.Tensor) -> torch.Tensor:
    """Inverse of :func:`block_scales`."""
    g, rows = blocked.shape
    assert g % 8 == 0 and rows % 32 == 0, "K must be a multiple of 512 and rows of 32"
    return blocked.reshape(rows // 32, g // 8, 32, 8).permute(1, 3, 0, 2).contiguous().reshape(g, rows)


def unblock_activations(blocked: torch.Tensor) -> torch.Tensor:
    """Inverse of :func:`block_activations`."""
    rows, kb = blocked.shape
    assert rows % 32 == 0 and kb % 32 == 0, "rows must be a multiple of 32 and K of 64"
    return blocked.reshape(rows // 32, kb // 32, 2, 32, 16).permute(0, 3, 1, 2, 4).contiguous().reshape(rows, kb)
