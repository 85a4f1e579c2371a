"""Shared helpers of the GPU parity tests."""

from typing import Dict, List, Sequence

import torch

# Tolerance of the parity contract for fp16/bf16 outputs with fp32 accumulation.
MAX_ABS = 2e-2
REL_L2 = 5e-3


def assert_close(actual: torch.Tensor, expected: torch.Tensor, what: str = "", max_abs: float = MAX_ABS,
                 rel_l2: float = REL_L2):
    a = actual.detach().double().cpu()
    e = expected.detach().double().cpu()
    assert a.shape == e.shape, (what, a.shape, e.shape)
    assert torch.isfinite(a).all(), f"{what}: non-finite output"
    err = (a - e).abs().max().item() if a.numel() else 0.0
    denom = e.norm().item()
    l2 = ((a - e).norm().item() / denom) if denom > 0 else (a - e).norm().item()
    assert err <= max_abs and l2 <= rel_l2, f"{what}: max-abs {err:.3e} (limit {max_abs}), rel-L2 {l2:.3e} (limit {rel_l2})"
    return err, l2


def ptr_table(tensors: Sequence[torch.Tensor], device, null_at: Sequence[int] = ()) -> torch.Tensor:
    addrs = [0 if (i in null_at or t is None) else t.data_ptr() for i, t in enumerate(tensors)]
    return torch.tensor(addrs, dtype=torch.int64, device=device)


def randn(shape, std, gen, dtype, device) -> torch.Tensor:
    return (torch.randn(shape, generator=gen, dtype=torch.float32) * std).to(dtype).to(device)


def stored_sgmv_a(a_lhr: torch.Tensor, r: int) -> torch.Tensor:
    """[L, h_in, r] -> the prefill storage of LoraWeights: [L, r, h_in] for 16 <= r <= 128."""
    return a_lhr.transpose(1, 2).contiguous() if 16 <= r <= 128 else a_lhr.contiguous()
