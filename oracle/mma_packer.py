"""
CPU restatement of the checkpoint packer (TEST INFRASTRUCTURE -- never a product path).

The published SVDQuant int4 checkpoints store the tensors of a quantized linear in the order NVIDIA's
``mma.m16n8k32`` register fragments want them.  This file restates the FORWARD direction (logical tensor -> bytes on
disk) in numpy, from the reference's packer (paths relative to the reference checkout):

=====================  ==============================================  ============================================
function               follows                                         pinned by (tests/test_oracle_pins.py)
=====================  ==============================================  ============================================
pack_weight            nunchaku/lora/flux/packer.py:173-226            the PTX fragment rule (lane = 4 * (n % 8) +
                                                                       (k / 8) % 4 owns 8 consecutive k of one n),
                                                                       hand-computed word positions, bijectivity
pack_scale             nunchaku/lora/flux/packer.py:228-262            hand-computed positions, bijectivity
pack_lowrank_weight    nunchaku/lora/flux/packer.py:300-338            hand-computed positions, the reference's own
                                                                       inverse statement (:340-373) restated as an
                                                                       index loop, bijectivity
=====================  ==============================================  ============================================

The product's inverse (``nunchaku_rocm_amd/csrc/layout.hip``) is written as closed-form index arithmetic, this file
as axis reshuffles: a wrong axis order or a swapped pair of sizes in either one breaks the round trip.
"""

from __future__ import annotations

import numpy as np

# geometry of the 4-bit packer with warp_n = 128 (packer.py:76-124): 8 x 4 lanes, a lane register holds 8 nibbles,
# two registers per lane along n and along k, eight lane-blocks along n per 128-row tile, one along k per 64 columns
N_TILE, K_TILE = 128, 64
N_PACKS, N_PACK, N_LANES = 8, 2, 8
K_PACKS, K_PACK, K_LANES, REG_K = 1, 2, 4, 8


def pack_weight(codes: np.ndarray) -> np.ndarray:
    """(n, k) integer codes 0..15 -> (n, k / 2) uint8 as on disk (packer.py:173-226).  n % 128 == 0, k % 128 == 0."""
    n, k = codes.shape
    assert n % N_TILE == 0 and k % (2 * K_TILE) == 0
    x = (codes.astype(np.uint32) & 0xF).reshape(n // N_TILE, N_PACKS, N_PACK, N_LANES, 1, k // K_TILE, K_PACKS, K_PACK, K_LANES, REG_K)
    #        axes: 0 n_tile  1 n_packs  2 n_pack  3 n_lane  4 reg_n  5 k_tile  6 k_packs  7 k_pack  8 k_lane  9 reg_k
    x = x.transpose(0, 5, 6, 1, 3, 8, 2, 7, 4, 9)
    words = (x << (4 * np.arange(REG_K, dtype=np.uint32))).sum(axis=-1, dtype=np.uint32)  # nibble j of a word = reg_k j
    return np.ascontiguousarray(words).view(np.uint8).reshape(n, k // 2)  # little endian


def pack_scale(scale: np.ndarray) -> np.ndarray:
    """(n, groups) (or (n,) for a per-channel vector) -> flat on-disk order (packer.py:228-262, warp_n = 128:
    s_pack_size 4, 32 lanes, one pack)."""
    n = scale.shape[0]
    assert n % 128 == 0
    x = scale.reshape(n // 128, 1, 8, 2, 4, 2, -1)
    return np.ascontiguousarray(x.transpose(0, 6, 1, 2, 4, 3, 5)).reshape(-1)


def pack_lowrank_weight(weight: np.ndarray, down: bool) -> np.ndarray:
    """Low-rank factor -> on-disk tensor (packer.py:300-338).  ``down``: weight is (rank, in_features) and the result is
    viewed (in_features, rank); otherwise weight is (out_features, rank) and keeps its shape."""
    if down:
        r, c = weight.shape
        x = weight.reshape(r // 16, 16, c // 16, 16).transpose(2, 0, 1, 3)
    else:
        c, r = weight.shape
        x = weight.reshape(c // 16, 16, r // 16, 16).transpose(0, 2, 1, 3)
    x = x.reshape(c // 16, r // 16, N_PACK, N_LANES, 1, K_PACK, K_LANES, 2)
    return np.ascontiguousarray(x.transpose(0, 1, 3, 6, 2, 5, 4, 7)).reshape(c, r)
