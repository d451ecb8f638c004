"""The reference's acceptance bar for requantized activations (tests/triton/test_native_epilogues.py:246-253, where its
fused kernel is held against its unfused Triton path): codes differ by at most one step on fewer than 1e-5 of the
entries, stored scales differ on fewer than 1e-4 (bf16) / 1e-3 (fp16) of the entries and then by one step of their own.
Such differences come from fp32 roundings of the GEMM output that move a value across a rounding midpoint.  On inputs
too small for the rates to mean anything, a single differing entry is let through."""

import torch


def assert_requantized_like_the_reference(codes, ref_codes, scales, ref_scales, dtype, what="", scale_rate_factor=1.0,
                                          scale_steps=1.0, code_rate_factor=1.0):  # fmt: skip
    diff = (codes.to(torch.int32) - ref_codes.to(torch.int32)).abs()
    nbad = int((diff > 0).sum())
    rate = nbad / diff.numel()
    sbad = int((scales.view(torch.int16) != ref_scales.view(torch.int16)).sum())
    srate = sbad / scales.numel()
    print(f"  {what}codes differ on {nbad} of {diff.numel()} ({rate:.2e}), scales on {sbad} of {scales.numel()} ({srate:.2e})", flush=True)
    assert int(diff.max()) <= 1, f"{what}a code is off by {int(diff.max())}"
    assert rate < 1e-5 * code_rate_factor or nbad <= 1, f"{what}code mismatch rate {rate:.2e}"
    bar = (1e-4 if dtype == torch.bfloat16 else 1e-3) * scale_rate_factor
    assert srate < bar or sbad <= 1, f"{what}scale mismatch rate {srate:.2e} (bar {bar:.0e})"
    ulp = 2.0**-7 if dtype == torch.bfloat16 else 2.0**-10
    sdiff = (scales.float() - ref_scales.float()).abs()
    assert bool((sdiff <= ref_scales.float().abs() * scale_steps * ulp + 1e-7).all()), f"{what}a scale is off by more than its step"
    return rate, srate
