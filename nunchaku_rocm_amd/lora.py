"""Run-time LoRA on single layers (reference: nunchaku/lora/runtime.py:442-525 ``_LoraHook``, ``attach_lora``,
``detach_lora``): an SVDQuant linear already carries a 16-bit low-rank branch, so ``sum_i (x @ down_i.T) @ up_i.T`` is
added by widening that branch, R = 32 + sum of the LoRA ranks, padded with zero columns to a multiple of 16; the
quantizer and the GEMM take any such R.  Layers without a low-rank branch get a forward hook.  Parsing LoRA files and
mapping their names onto a model are the reference's tooling and are not part of this package."""

from __future__ import annotations

import torch
from torch import nn

from .linear import SVDQW4A4Linear


class _LoraHook:
    """Forward hook adding ``sum_i up_i(down_i(x))`` to a layer without a low-rank branch."""

    def __init__(self):
        self.pairs: list[tuple[torch.Tensor, torch.Tensor]] = []

    def __call__(self, module, args, output):
        x = args[0]
        if self.pairs and self.pairs[0][0].device != x.device:  # the model moved since the LoRAs were attached
            self.pairs = [(d.to(x.device), u.to(x.device)) for d, u in self.pairs]
        for down, up in self.pairs:
            output = output + ((x.to(down.dtype) @ down.t()) @ up.t()).to(output.dtype)
        return output


def attach_lora(module: nn.Module, pairs: list[tuple[torch.Tensor, torch.Tensor]]) -> None:
    """
    Add ``sum_i (x @ down_i.T) @ up_i.T`` to one layer's output; ``down`` is ``(r, in)``, ``up`` is ``(out, r)`` with
    the strength already folded in.  Undo with :func:`detach_lora`.  Convolution LoRAs are not handled.
    """
    detach_lora(module)
    if any(isinstance(d, tuple) for d, _ in pairs):
        raise NotImplementedError("convolution LoRA")
    if isinstance(module, SVDQW4A4Linear):
        base_down, base_up = module.proj_down.data, module.proj_up.data
        n_in, n_out = base_down.shape[0], base_up.shape[0]
        downs = [d.t() for d, _ in pairs]
        ups = [u for _, u in pairs]
        for d, u in zip(downs, ups):
            if d.shape[0] != n_in or u.shape[0] != n_out or d.shape[1] != u.shape[1]:
                raise ValueError(f"LoRA pair {tuple(d.t().shape)} / {tuple(u.shape)} does not fit a {n_in} -> {n_out} layer")
        pad = -(base_down.shape[1] + sum(d.shape[1] for d in downs)) % 16
        if pad:
            downs.append(torch.zeros(n_in, pad))
            ups.append(torch.zeros(n_out, pad))
        dev, dt = base_down.device, base_down.dtype
        module._lora_base = (base_down, base_up)
        module.proj_down.data = torch.cat([base_down] + [d.to(dev, dt) for d in downs], 1).contiguous()
        module.proj_up.data = torch.cat([base_up] + [u.to(dev, dt) for u in ups], 1).contiguous()
        module.rank = module.proj_down.shape[1]
    else:
        p = next(p for p in module.parameters() if p.is_floating_point())  # AWQ layers also hold packed integers
        hook = _LoraHook()
        hook.pairs = [(d.to(p.device, p.dtype), u.to(p.device, p.dtype)) for d, u in pairs]
        module._lora_hook = hook
        module._lora_hook_handle = module.register_forward_hook(hook)


def detach_lora(module: nn.Module) -> None:
    """Remove what :func:`attach_lora` added (no-op if nothing is attached)."""
    if hasattr(module, "_lora_base"):
        base_down, base_up = module._lora_base
        dev = module.proj_down.device  # the model may have moved since the LoRAs were attached
        module.proj_down.data, module.proj_up.data = base_down.to(dev), base_up.to(dev)
        module.rank = module.proj_down.shape[1]
        del module._lora_base
    if hasattr(module, "_lora_hook"):
        module._lora_hook_handle.remove()
        del module._lora_hook, module._lora_hook_handle
