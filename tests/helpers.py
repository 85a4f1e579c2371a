"""Shared helpers of the GPU parity tests."""

from typing import Dict, List, Sequence

import torch

# Tolerance of the parity contract for fp16/bf16 outputs with fp32 accumulation.
MAX_ABS = 2e-2
REL_L2 = 5e-3


def _ulp(expected: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """Spacing of `dtype` at the magnitude of each expected value (fp16: 10 mantissa bits, bf16: 7)."""
    bits = 10 if dtype == torch.float16 else 7
    mag = expected.abs().clamp_min(2.0 ** -14)
    return torch.exp2(torch.floor(torch.log2(mag)) - bits)


def assert_close(actual: torch.Tensor, expected: torch.Tensor, what: str = "", max_abs: float = MAX_ABS,
                 rel_l2: float = REL_L2, rounded: Sequence[torch.Tensor] = ()):
    """max-abs <= 2e-2 and rel-L2 <= 5e-3.  Where the spacing of the fp16/bf16 values involved exceeds that
    (|value| >= 2 in bf16), the per-element limit is the sum of the spacings of every rounding the value went
    through: its own, and those of the tensors in `rounded` (same shape).  y += delta rounds delta to the output
    type, adds in fp32 and rounds again; two correct fp32 dot products that differ in summation order can put
    delta on neighbouring values, and the second rounding can move the two sums apart by one more step (ties)."""
    a = actual.detach().double().cpu()
    e = expected.detach().double().cpu()
    assert a.shape == e.shape, (what, a.shape, e.shape)
    assert torch.isfinite(a).all(), f"{what}: non-finite output"
    diff = (a - e).abs()
    err = diff.max().item() if a.numel() else 0.0
    spacing = torch.zeros_like(e)
    if actual.dtype in (torch.float16, torch.bfloat16):
        spacing += _ulp(e, actual.dtype)
    for t in rounded:
        spacing += _ulp(t.detach().double().cpu(), t.dtype)
    limit = torch.maximum(torch.full_like(e, max_abs), spacing * 1.0001)
    denom = e.norm().item()
    l2 = ((a - e).norm().item() / denom) if denom > 0 else (a - e).norm().item()
    over = int((diff > limit).sum().item()) if a.numel() else 0
    assert over == 0 and l2 <= rel_l2, (
        f"{what}: {over} elements over the limit, max-abs {err:.3e} (limit {max_abs} or the roundings' spacing), "
        f"rel-L2 {l2:.3e} (limit {rel_l2})")
    return err, l2


def ptr_table(tensors: Sequence[torch.Tensor], device, null_at: Sequence[int] = ()) -> torch.Tensor:
    addrs = [0 if (i in null_at or t is None) else t.data_ptr() for i, t in enumerate(tensors)]
    return torch.tensor(addrs, dtype=torch.int64, device=device)


def randn(shape, std, gen, dtype, device) -> torch.Tensor:
    return (torch.randn(shape, generator=gen, dtype=torch.float32) * std).to(dtype).to(device)


def stored_sgmv_a(a_lhr: torch.Tensor, r: int) -> torch.Tensor:
    """[L, h_in, r] -> the prefill storage of LoraWeights: [L, r, h_in] for 16 <= r <= 128."""
    return a_lhr.transpose(1, 2).contiguous() if 16 <= r <= 128 else a_lhr.contiguous()
