"""Writes tests/golden/svdq_small.npz: seeded inputs and the CPU oracle's outputs for one small case of every operator.

The reference holds no golden vectors for this path, so these are regression anchors, not reference outputs: they pin
the oracle (and through it the GPU kernels) against drifting between revisions.  Run from the repo root:
    python tests/golden/make_fixtures.py
16-bit tensors are stored as int16 bit patterns (numpy has no bfloat16)."""

import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle import mma_packer as P  # noqa: E402
from oracle import svdq_oracle as O  # noqa: E402


def bits(t: torch.Tensor) -> np.ndarray:
    return t.contiguous().view(torch.int16).numpy()


def main() -> None:
    M, K, N, R = 48, 256, 128, 16
    lin = O.make_svdq_linear(K, N, R=R, seed=11)
    x = O.make_activations(M, K, seed=12)
    q, s, la, codes = O.quantize_act(x, lin["proj_down"], lin["smooth_factor"])
    acc = O.group_acc_i32(q, lin["qweight"], False, groups=[1])[0]
    y = O.gemm_w4a4(q, lin["qweight"], s, lin["wscales"], lin["bias"], la, lin["proj_up"]).to(torch.bfloat16)
    awq = O.make_awq_linear(256, 128, seed=13)
    xv = torch.randn(2, 256, generator=torch.Generator().manual_seed(14)).to(torch.bfloat16)
    yv = O.awq_gemv(xv, awq["qweight"].view(torch.int16).reshape(32, 256), awq["wscales"], awq["wzeros"]).to(torch.bfloat16)
    g = torch.Generator().manual_seed(15)
    aq, ak, av = (torch.randn(1, 2, 40, 128, generator=g).to(torch.bfloat16) for _ in range(3))
    ao = O.attention_fp16(aq, ak[:, :, :37], av[:, :, :37], 128**-0.5)
    sc, sh = (torch.randn(K, generator=g).to(torch.bfloat16) for _ in range(2))
    xm = O.layernorm_modulate(x, sc, sh)
    wcodes = O.unpack_int4(lin["qweight"], signed=False).to(torch.int32).numpy()
    out = {
        "x": bits(x), "smooth": bits(lin["smooth_factor"]), "proj_down": bits(lin["proj_down"]), "proj_up": bits(lin["proj_up"]),
        "qweight": lin["qweight"].view(torch.uint8).numpy(), "wscales": bits(lin["wscales"]), "bias": bits(lin["bias"]),
        "q_codes": q.numpy(), "q_scales": bits(s), "q_lora_act": la.numpy(), "group1_acc": acc.numpy(), "gemm_out": bits(y),
        "awq_qweight": awq["qweight"].numpy(), "awq_wscales": bits(awq["wscales"]), "awq_wzeros": bits(awq["wzeros"]),
        "awq_x": bits(xv), "awq_out": bits(yv),
        "attn_q": bits(aq), "attn_k": bits(ak), "attn_v": bits(av), "attn_out": bits(ao),
        "norm_scale": bits(sc), "norm_shift": bits(sh), "norm_out": bits(xm),
        "packed_qweight": P.pack_weight(wcodes), "packed_wscales": P.pack_scale(bits(lin["wscales"].t())),
    }  # fmt: skip
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "svdq_small.npz")
    np.savez_compressed(path, **out)
    print(path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
