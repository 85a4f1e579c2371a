"""TEST INFRASTRUCTURE - not part of the product.

CPU restatement of what the reference computes on the multi-adapter LoRA hot path, used
only as the checker in tests/, in __graft_entry__.smoke() and as the timed CPU baseline
of bench.py.  Nothing under lorax_amd/ imports this package.

Each function names the reference lines it restates.  How each one is pinned (the checks
live in tests/test_oracle.py):

  fallback_layer_type   the reference's own non-kernel branch, written with the same torch
                        ops in the same order (layers.py:169-211).  Pinned against an fp64
                        brute-force gather-matmul on small inputs with a bf16/fp16-sized
                        tolerance, against sgmv_ref/bgmv_ref (three independent
                        formulations must agree), by linearity in B and by the
                        "other adapters' tokens get exactly zero" property.
  sgmv_ref              server/tests/utils/test_sgmv.py:16-39 (lora_ref_impl).  Pinned as
                        above and by the empty-segment cases of that test (:46-47).
  bgmv_ref              docstring at punica.py:199-217 + kernel text bgmv_impl.cuh:24-27,
                        141,157-159,189-190.  The reference has NO test of BGMV numerics:
                        PARITY UNPINNED by any reference vector; pinned here only through
                        the equivalence with fallback_layer_type and the fp64 brute force.
  find_segments_ref     utils/segments.py:6-26.  Pinned by the golden vectors of
                        server/tests/utils/test_segments.py:10-18.
  concat_segments_ref   utils/segments.py:29-55.  Golden vectors test_segments.py:29-45.
  rank_groups_ref       adapters/lora.py:320-375 (rank grouping and decode indices).
                        Golden vectors server/tests/utils/test_lora.py:112-128.
  pad_to_min_rank_ref   punica.py:57-76.  Pinned by closed form (target rank table) and the
                        product-preservation property of test_sgmv.py:108-127.
  sgmv_tmp_size_ref     sgmv_cutlass.cuh:54-58 = 60 bytes per problem (closed form).
"""

from typing import Dict, Iterable, List, Optional, Sequence, Tuple

import torch

MIN_RANK_CUSTOM = 16
MAX_RANK_CUSTOM = 128
SGMV_BLOCK_SIZE = 16


def orient_for_rank_ref(t: torch.Tensor, rank: int) -> torch.Tensor:
    """punica.py:83-86."""
    if MIN_RANK_CUSTOM <= rank <= MAX_RANK_CUSTOM:
        return t.transpose(0, 1)
    return t


def fallback_layer_type(
    result: torch.Tensor,
    input: torch.Tensor,
    adapter_indices: torch.Tensor,
    adapter_set: Iterable[int],
    lora_a: Dict[int, torch.Tensor],
    lora_b: Dict[int, torch.Tensor],
    layer_id: int,
    start_idx: int,
    end_idx: int,
) -> torch.Tensor:
    """The "vanilla PyTorch" branch of LoraLinear.forward_layer_type with forward_lora inlined
    (layers.py:169-211, world size 1, no speculative tokens).

    lora_a[i] is adapter i's stored A stack ([L, r, h_in] for 16 <= r <= 128, else [L, h_in, r]),
    lora_b[i] its B stack [L, r, h_out]; adapters missing from lora_a have no weights for the
    layer.  Every adapter multiplies ALL rows and a 0/1 mask keeps its own (layers.py:179,210);
    rounding to the tensor dtype happens after x@A, after (.)@B and after the += (layers.py:206,
    210,190).
    """
    for adapter_index in adapter_set:
        if adapter_index not in lora_a:
            continue
        mask = (adapter_indices == adapter_index).to(input.dtype).view(-1, 1)
        b = lora_b[adapter_index][layer_id, :, :]
        a = orient_for_rank_ref(lora_a[adapter_index][layer_id, :, :], b.size(0))
        a_out = input @ a
        result[:, start_idx:end_idx] += (a_out @ b) * mask
    return result


def sgmv_ref(
    y: torch.Tensor,
    x: torch.Tensor,
    wa: Sequence[Optional[torch.Tensor]],
    wb: Sequence[Optional[torch.Tensor]],
    s_start: Sequence[int],
    s_end: Sequence[int],
    layer_idx: int,
    lora_rank: int,
) -> torch.Tensor:
    """Segment-wise y[s:e] += (x[s:e] @ A_i) @ B_i (test_sgmv.py:16-39). wa[i] is [L, r, h_in] unless
    the rank is below 16, then [L, h_in, r]; entries of empty segments may be None."""
    for i in range(len(wa)):
        s, e = int(s_start[i]), int(s_end[i])
        if e - s <= 0:
            continue
        a = wa[i][layer_idx]
        if not lora_rank < MIN_RANK_CUSTOM:
            a = a.t()
        v = x[s:e] @ a
        y[s:e] = y[s:e] + v @ wb[i][layer_idx]
    return y


def bgmv_ref(
    y: torch.Tensor,
    x: torch.Tensor,
    w_T_all: Sequence[torch.Tensor],
    indices: Sequence[int],
    layer_idx: int,
    scale: float = 1.0,
) -> torch.Tensor:
    """One BGMV call: y[b] += T(scale * x[b] @ W[indices[b]][layer_idx].T) for indices[b] >= 0, fp32
    accumulation (punica.py:199-217; bgmv_impl.cuh:24-27,141). W stacks are [L, h_out, h_in]."""
    for b, idx in enumerate(indices):
        idx = int(idx)
        if idx < 0:
            continue
        w = w_T_all[idx][layer_idx].float()
        delta = (w @ x[b].float()) * scale
        y[b] = (y[b].float() + delta.to(y.dtype).float()).to(y.dtype)
    return y


def lora_delta_f64(
    x: torch.Tensor,
    adapter_of_token: Sequence[int],
    a_hr: Dict[int, torch.Tensor],
    b_rh: Dict[int, torch.Tensor],
) -> torch.Tensor:
    """Brute-force fp64 gather-matmul: delta[t] = x[t] @ A_i @ B_i with i = adapter_of_token[t], zero if
    i has no weights. a_hr[i] is [h_in, r], b_rh[i] is [r, h_out], whatever their dtype."""
    h_out = next(iter(b_rh.values())).size(1)
    out = torch.zeros((x.size(0), h_out), dtype=torch.float64)
    xd = x.double()
    for t, i in enumerate(adapter_of_token):
        i = int(i)
        if i in a_hr:
            out[t] = (xd[t] @ a_hr[i].double()) @ b_rh[i].double()
    return out


def find_segments_ref(adapter_indices: Sequence[int]) -> Tuple[List[int], List[int]]:
    """utils/segments.py:6-26 as a plain scan: boundaries where the value changes."""
    values = [int(v) for v in adapter_indices]
    bounds, owners = [0], []
    for i in range(1, len(values)):
        if values[i] != values[i - 1]:
            bounds.append(i)
            owners.append(values[i - 1])
    if values:
        bounds.append(len(values))
        owners.append(values[-1])
    return bounds, owners


def concat_segments_ref(batches: Sequence[Tuple[Sequence[int], Sequence[int]]]) -> Tuple[List[int], List[int]]:
    """utils/segments.py:29-55 on plain lists: shift later batches by the tokens before them and merge the
    run across a seam when both sides belong to the same adapter."""
    bounds: List[int] = []
    owners: List[int] = []
    for seg, idx in batches:
        seg, idx = [int(v) for v in seg], [int(v) for v in idx]
        if bounds:
            seg = [v + bounds[-1] for v in seg[1:]]
            if owners and owners[-1] == idx[0]:
                idx = idx[1:]
                bounds.pop()
        bounds.extend(seg)
        owners.extend(idx)
    return bounds, owners


def rank_groups_ref(
    segment_indices: Sequence[int],
    adapter_indices: Sequence[int],
    rank_of_adapter: Dict[int, int],
) -> Dict[int, Tuple[List[int], List[int]]]:
    """adapters/lora.py:320-375 for decode: rank -> (segment positions in the group, per-token index into
    the group's pointer slice or -1). rank_of_adapter holds only adapters with weights for the layer."""
    groups: Dict[int, List[int]] = {}
    for pos, adapter in enumerate(segment_indices):
        if adapter in rank_of_adapter:
            groups.setdefault(rank_of_adapter[adapter], []).append(pos)
    out = {}
    for rank, positions in groups.items():
        first_slot: Dict[int, int] = {}
        for loc, pos in enumerate(positions):
            first_slot.setdefault(segment_indices[pos], loc)
        per_token = [
            first_slot[a] if (a in rank_of_adapter and rank_of_adapter[a] == rank) else -1 for a in adapter_indices
        ]
        out[rank] = (positions, per_token)
    return out


def pad_to_min_rank_ref(t: torch.Tensor, dim: int, min_rank: int) -> torch.Tensor:
    """punica.py:57-76 via explicit zero concatenation."""
    rank = t.size(dim)
    target = min_rank if rank <= min_rank else ((rank + SGMV_BLOCK_SIZE - 1) // SGMV_BLOCK_SIZE) * SGMV_BLOCK_SIZE
    if target == rank:
        return t
    shape = list(t.shape)
    shape[dim] = target - rank
    return torch.cat([t, torch.zeros(shape, dtype=t.dtype, device=t.device)], dim=dim)


def sgmv_tmp_size_ref(num_problems: int) -> int:
    """sgmv_cutlass.cuh:54-58: 3 pointers, 3 int64 and a 3 x int32 GemmCoord per problem."""
    return num_problems * (3 * 8 + 3 * 8 + 3 * 4)
