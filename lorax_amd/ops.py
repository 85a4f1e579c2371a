"""The six LoRA operators of lorax_server/utils/ops (bgmv_shrink / bgmv_expand / bgmv_expand_slice /
sgmv_shrink / sgmv_expand / sgmv_expand_slice) on the HIP kernels of this package, plus bgmv_lora_slices
and sgmv_lora_slices, which run the update of several column slices that share their input with one shrink
launch for all of them (decode: and one expand launch).

Same names, argument orders and meaning as the reference's Triton operators, which index ONE stacked
weight tensor per layer - lora_a_weights [num_loras, r, h_in], lora_b_weights [num_loras, h_out, r], an
optional singleton second dimension - with per-token (bgmv) or per-sequence (sgmv) adapter numbers, -1
meaning "no adapter".  Those two stacked layouts are exactly the [L, r, h_in] / [L, h_out, r] stacks the
kernels here read, with one layer: entry i of the stack is "adapter i, layer 0", so the only thing added is
a table of the stack entries' addresses, cached per weight tensor.

Differences from the Triton operators, all invisible in the final result:
  * the shrink operators add to `output_tensor` (the reference stores when its SPLIT_K is 1 and adds
    otherwise, bgmv_shrink.py:72-75; its callers always pass zeros);
  * an fp32 `output_tensor` of a shrink receives sums already rounded to the input type - the value the
    reference's expand operators round the buffer to before they use it (CAST_TYPE, sgmv_expand.py:160-165);
  * an fp32 `inputs` of an expand is rounded to the weight type on the way in, as CAST_TYPE does;
  * `override_config`, `batches` and `max_seq_length` are accepted and ignored.
"""

from collections import OrderedDict
from typing import Dict, Optional, Tuple

import torch

from lorax_amd import _native
from lorax_amd.sgmv import get_tmp_tensor, get_tmp_tensor_for_size

_TABLE_CACHE: "OrderedDict[Tuple[int, int, int, str], torch.Tensor]" = OrderedDict()
_TABLE_CACHE_SIZE = 1024


def _stacked(weights: torch.Tensor, what: str) -> torch.Tensor:
    if weights.ndim == 4:  # shape: (lora_num, 1, rows, cols), bgmv_shrink.py:110-112
        assert weights.size(1) == 1
        weights = weights.squeeze(dim=1)
    else:
        assert weights.ndim == 3, f"{what} must be [num_loras, rows, cols]"
    assert weights.is_contiguous()
    assert weights.dtype in (torch.float16, torch.bfloat16)
    return weights


def stack_table(weights: torch.Tensor) -> torch.Tensor:
    """int64 device tensor with the address of every entry of a stacked weight tensor [num_loras, rows, cols]."""
    key = (weights.data_ptr(), weights.size(0), weights.stride(0), str(weights.device))
    table = _TABLE_CACHE.get(key)
    if table is None:
        step = weights.stride(0) * weights.element_size()
        table = weights.data_ptr() + torch.arange(weights.size(0), dtype=torch.int64) * step
        table = table.to(weights.device)
        _TABLE_CACHE[key] = table
        if len(_TABLE_CACHE) > _TABLE_CACHE_SIZE:
            _TABLE_CACHE.popitem(last=False)
    else:
        _TABLE_CACHE.move_to_end(key)
    return table


def segment_bounds(b_seq_start_loc: torch.Tensor, seq_len_tensor: torch.Tensor,
                   lora_indices_tensor: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """int32 segment starts and ends for the SGMV kernels; sequences without an adapter become empty
    segments, whose weight pointers are never read."""
    start = b_seq_start_loc.to(torch.int32)
    length = torch.where(lora_indices_tensor >= 0, seq_len_tensor, torch.zeros_like(seq_len_tensor))
    return start, start + length.to(torch.int32)


def _segment_pointers(weights: torch.Tensor, lora_indices_tensor: torch.Tensor) -> torch.Tensor:
    return stack_table(weights)[lora_indices_tensor.clamp(min=0)]


def _check_rows(inputs: torch.Tensor, output_tensor: torch.Tensor):
    assert inputs.is_contiguous()
    assert output_tensor.is_contiguous()
    assert inputs.size(0) == output_tensor.size(0)


def _shrink_output(inputs: torch.Tensor, output_tensor: torch.Tensor):
    """The tensor the kernel adds to, and what to do afterwards when that is not output_tensor itself."""
    if output_tensor.dtype == inputs.dtype:
        return output_tensor, None
    assert output_tensor.dtype == torch.float32
    staged = torch.zeros(output_tensor.shape, dtype=inputs.dtype, device=inputs.device)
    return staged, lambda: output_tensor.add_(staged)


@torch.inference_mode()
def bgmv_shrink(
    inputs: torch.Tensor,
    lora_a_weights: torch.Tensor,
    output_tensor: torch.Tensor,
    lora_indices_tensor: torch.Tensor,
    scaling: float = 1.0,
    override_config: Optional[Dict[str, int]] = None,
):
    """output_tensor[t] += scaling * (inputs[t] @ lora_a_weights[idx[t]].T) for idx[t] >= 0 (bgmv_shrink.py:80-153)."""
    assert inputs.dtype == lora_a_weights.dtype
    assert inputs.dtype in (torch.float16, torch.bfloat16)
    lora_a_weights = _stacked(lora_a_weights, "lora_a_weights")
    assert inputs.size(1) == lora_a_weights.size(-1)
    _check_rows(inputs, output_tensor)
    assert output_tensor.size(1) == lora_a_weights.size(-2)
    out, finish = _shrink_output(inputs, output_tensor)
    _native.bgmv_multi([(out, inputs, stack_table(lora_a_weights), lora_indices_tensor, 0, None)], 0, scaling, True)
    if finish is not None:
        finish()


def _expand_inputs(inputs: torch.Tensor, lora_b_weights: torch.Tensor) -> torch.Tensor:
    assert inputs.dtype in (torch.float16, torch.bfloat16, torch.float32)
    if inputs.dtype == torch.float32:  # CAST_TYPE, bgmv_expand.py:118-123
        inputs = inputs.to(lora_b_weights.dtype)
    assert inputs.dtype == lora_b_weights.dtype
    assert inputs.size(1) == lora_b_weights.size(-1)
    return inputs


@torch.inference_mode()
def bgmv_expand_slice(
    inputs: torch.Tensor,
    lora_b_weights: torch.Tensor,
    output_tensor: torch.Tensor,
    lora_indices_tensor: torch.Tensor,
    slice_offset: int,
    slice_size: int,
    add_inputs: bool = True,
    override_config: Optional[Dict[str, int]] = None,
):
    """output_tensor[t, slice] (+)= inputs[t] @ lora_b_weights[idx[t]].T for idx[t] >= 0
    (bgmv_expand_slice.py:82-168)."""
    lora_b_weights = _stacked(lora_b_weights, "lora_b_weights")
    inputs = _expand_inputs(inputs, lora_b_weights)
    _check_rows(inputs, output_tensor)
    assert slice_size == lora_b_weights.size(-2)
    _native.bgmv_multi(
        [(output_tensor, inputs, stack_table(lora_b_weights), lora_indices_tensor, slice_offset, slice_size)],
        0, 1.0, add_inputs,
    )


@torch.inference_mode()
def bgmv_expand(
    inputs: torch.Tensor,
    lora_b_weights: torch.Tensor,
    output_tensor: torch.Tensor,
    lora_indices_tensor: torch.Tensor,
    add_inputs: bool = True,
    override_config: Optional[Dict[str, int]] = None,
):
    """bgmv_expand.py:82-160: the slice operator over the whole width of output_tensor."""
    width = lora_b_weights.size(-2)
    assert output_tensor.size(1) == width
    bgmv_expand_slice(inputs, lora_b_weights, output_tensor, lora_indices_tensor, 0, width, add_inputs)


def build_slot_plan(slots) -> "torch.Tensor":
    """Routing plan (host, int64 [chunks, 8]) of a decode batch over STACKED weights: `slots` holds every token's
    entry number in the stacked tensors, negative = no adapter.  One record per chunk of up to four tokens of one
    entry: [count, four token rows (unused ones repeat the first), entry, entry, 0] - the records of
    lorax_bgmv_multi with entry numbers where a pointer-table plan holds addresses, so ONE plan serves every layer
    and projection of the step."""
    import numpy as np

    slots = np.asarray(slots, dtype=np.int64).reshape(-1)
    routed = np.nonzero(slots >= 0)[0]
    n = routed.shape[0]
    if n == 0:
        return torch.zeros((0, _native.PLAN_RECORD_WORDS), dtype=torch.int64)
    order = routed[np.argsort(slots[routed], kind="stable")]  # grouped by entry, token order inside a group
    entry = slots[order]
    pos = np.arange(n)
    starts = np.r_[True, entry[1:] != entry[:-1]]
    rank = pos - np.maximum.accumulate(np.where(starts, pos, 0))  # position inside the entry's group
    heads = rank % 4 == 0
    chunk = np.cumsum(heads) - 1
    records = np.zeros((int(chunk[-1]) + 1, _native.PLAN_RECORD_WORDS), dtype=np.int64)
    records[:, 0] = np.bincount(chunk)
    records[:, 1:5] = order[heads][:, None]
    records[chunk, 1 + rank % 4] = order
    records[:, 5] = records[:, 6] = entry[heads]
    return torch.from_numpy(records)


@torch.inference_mode()
def bgmv_lora_slices(
    inputs: torch.Tensor,
    slices,
    output_tensor: torch.Tensor,
    lora_indices_tensor: torch.Tensor,
    scaling: float = 1.0,
    plan: Optional[torch.Tensor] = None,
):
    """bgmv_shrink followed by bgmv_expand_slice(add_inputs=True) for several column slices of output_tensor that
    share `inputs` (q/k/v, gate/up): `slices` is a sequence of (lora_a_weights, lora_b_weights, slice_offset,
    slice_size), ranks may differ.  No counterpart among the reference's operators, which its wrapper calls once
    per slice (punica.py:750-773); here the shrinks of up to 16 slices are one launch and their expands another,
    and the intermediate is kept in the type of `inputs` and never zero-filled (the shrink overwrites the rows
    of routed tokens and the expand reads no others).
    `plan`: the batch's routing plan over stack entries (build_slot_plan of lora_indices_tensor, on the device).
    With it no workgroup scans lora_indices_tensor, and slices of rank 8 or 16 with a small A slab run shrink and
    expand in ONE launch per rank (scaling 1 only: that kernel scales the update, the two-launch path the
    intermediate, and only at 1 do both round alike)."""
    assert inputs.dtype in (torch.float16, torch.bfloat16)
    assert inputs.is_contiguous() and output_tensor.is_contiguous()
    assert inputs.size(0) == output_tensor.size(0)
    jobs = []
    for lora_a_weights, lora_b_weights, slice_offset, slice_size in slices:
        a = _stacked(lora_a_weights, "lora_a_weights")
        b = _stacked(lora_b_weights, "lora_b_weights")
        assert a.dtype == inputs.dtype and b.dtype == inputs.dtype
        assert inputs.size(1) == a.size(-1) and a.size(-2) == b.size(-1) and slice_size == b.size(-2)
        jobs.append((a, b, a.size(-2), slice_offset, slice_size))
    if plan is not None and scaling == 1.0 and all(
            _native.bgmv_lora_fits(r, inputs.size(1), size) for _, _, r, _, size in jobs):
        step = _native.MAX_FUSED_BGMV_PROBLEMS
        for rank in sorted({r for _, _, r, _, _ in jobs}):
            same = [j for j in jobs if j[2] == rank]
            for i in range(0, len(same), step):
                chunk = same[i : i + step]
                _native.bgmv_lora_multi([(output_tensor, inputs, plan, off, size) for _, _, _, off, size in chunk],
                                        rank, 0, 1.0, stacks=[(a, b) for a, b, _, _, _ in chunk])
        return
    step = _native.MAX_BGMV_PROBLEMS
    tokens = inputs.size(0)
    for i in range(0, len(jobs), step):
        chunk = jobs[i : i + step]
        flat = torch.empty((tokens * sum(r for _, _, r, _, _ in chunk),), dtype=inputs.dtype, device=inputs.device)
        bufs, pos = [], 0
        for _, _, r, _, _ in chunk:
            bufs.append(flat[pos : pos + tokens * r].view(tokens, r))
            pos += tokens * r
        if plan is not None:
            plans = [plan] * len(chunk)
            _native.bgmv_multi([(v, inputs, None, None, 0, None) for v in bufs], 0, scaling, False, plans,
                               stacks=[a for a, _, _, _, _ in chunk])
            _native.bgmv_multi([(output_tensor, v, None, None, off, size) for v, (_, _, _, off, size) in zip(bufs, chunk)],
                               0, 1.0, True, plans, stacks=[b for _, b, _, _, _ in chunk])
            continue
        _native.bgmv_multi([(v, inputs, stack_table(a), lora_indices_tensor, 0, None)
                            for v, (a, _, _, _, _) in zip(bufs, chunk)], 0, scaling, False)
        _native.bgmv_multi([(output_tensor, v, stack_table(b), lora_indices_tensor, off, size)
                            for v, (_, b, _, off, size) in zip(bufs, chunk)], 0, 1.0, True)


@torch.inference_mode()
def sgmv_shrink(
    inputs: torch.Tensor,
    lora_a_weights: torch.Tensor,
    output_tensor: torch.Tensor,
    b_seq_start_loc: torch.Tensor,
    seq_len_tensor: torch.Tensor,
    lora_indices_tensor: torch.Tensor,
    batches: int,
    max_seq_length: int,
    scaling: float,
    bounds: Optional[Tuple[torch.Tensor, torch.Tensor]] = None,
):
    """output_tensor[s:e] += scaling * (inputs[s:e] @ lora_a_weights[idx].T) for every sequence with idx >= 0
    (sgmv_shrink.py:101-196).  `bounds` may carry segment_bounds(...) of the same three tensors, computed once per
    batch by the caller."""
    assert inputs.dtype == lora_a_weights.dtype
    assert inputs.dtype in (torch.float16, torch.bfloat16)
    lora_a_weights = _stacked(lora_a_weights, "lora_a_weights")
    assert inputs.size(1) == lora_a_weights.size(-1)
    assert b_seq_start_loc.size(0) == batches
    assert lora_indices_tensor.size(0) == batches
    _check_rows(inputs, output_tensor)
    s_start, s_end = bounds if bounds is not None else segment_bounds(b_seq_start_loc, seq_len_tensor,
                                                                        lora_indices_tensor)
    out, finish = _shrink_output(inputs, output_tensor)
    _native.sgmv_shrink(out, inputs, _segment_pointers(lora_a_weights, lora_indices_tensor), s_start, s_end,
                        get_tmp_tensor(inputs.device), 0, scaling)
    if finish is not None:
        finish()


@torch.inference_mode()
def sgmv_lora_slices(
    inputs: torch.Tensor,
    slices,
    output_tensor: torch.Tensor,
    b_seq_start_loc: torch.Tensor,
    seq_len_tensor: torch.Tensor,
    lora_indices_tensor: torch.Tensor,
    batches: int,
    max_seq_length: int,
    scaling: float = 1.0,
    bounds: Optional[Tuple[torch.Tensor, torch.Tensor]] = None,
):
    """sgmv_shrink followed by sgmv_expand_slice(add_inputs=True) for several column slices of output_tensor that
    share `inputs` (q/k/v, gate/up): `slices` is a sequence of (lora_a_weights, lora_b_weights, slice_offset,
    slice_size).  No counterpart among the reference's operators (its wrapper calls them once per slice,
    punica.py:750-773): slices of one rank shrink together, up to a summed rank of 128 per launch, so `inputs`
    is read once per launch; the intermediate is kept in the type of `inputs`."""
    assert inputs.dtype in (torch.float16, torch.bfloat16)
    assert inputs.is_contiguous() and output_tensor.is_contiguous()
    assert inputs.size(0) == output_tensor.size(0)
    assert b_seq_start_loc.size(0) == batches and lora_indices_tensor.size(0) == batches
    s_start, s_end = bounds if bounds is not None else segment_bounds(b_seq_start_loc, seq_len_tensor,
                                                                        lora_indices_tensor)
    by_rank: Dict[int, list] = {}
    for lora_a_weights, lora_b_weights, slice_offset, slice_size in slices:
        a = _stacked(lora_a_weights, "lora_a_weights")
        b = _stacked(lora_b_weights, "lora_b_weights")
        assert a.dtype == inputs.dtype and b.dtype == inputs.dtype
        assert inputs.size(1) == a.size(-1) and a.size(-2) == b.size(-1) and slice_size == b.size(-2)
        by_rank.setdefault(a.size(-2), []).append((a, b, slice_offset, slice_size))
    tmp = get_tmp_tensor(inputs.device)
    tmp_expand = get_tmp_tensor_for_size(batches, inputs.device)
    tokens = inputs.size(0)
    for r, jobs in by_rank.items():
        step = max(1, min(_native.MAX_SGMV_SHRINK_PROBLEMS, 128 // r))
        for i in range(0, len(jobs), step):
            chunk = jobs[i : i + step]
            bufs = list(torch.zeros((len(chunk), tokens, r), dtype=inputs.dtype, device=inputs.device).unbind(0))
            _native.sgmv_shrink_multi(bufs, inputs, [_segment_pointers(a, lora_indices_tensor) for a, _, _, _ in chunk],
                                      s_start, s_end, tmp, 0, scaling)
            for v, (_, b, off, size) in zip(bufs, chunk):
                _native.sgmv_expand(output_tensor, v, _segment_pointers(b, lora_indices_tensor), s_start, s_end,
                                    tmp_expand, 0, off, size, transposed=True, accumulate=True)


@torch.inference_mode()
def sgmv_expand_slice(
    inputs: torch.Tensor,
    lora_b_weights: torch.Tensor,
    output_tensor: torch.Tensor,
    b_seq_start_loc: torch.Tensor,
    seq_len_tensor: torch.Tensor,
    lora_indices_tensor: torch.Tensor,
    batches: int,
    max_seq_length: int,
    slice_offset: int,
    slice_size: int,
    add_inputs: bool = False,
    bounds: Optional[Tuple[torch.Tensor, torch.Tensor]] = None,
):
    """output_tensor[s:e, slice] (+)= inputs[s:e] @ lora_b_weights[idx].T for every sequence with idx >= 0
    (sgmv_expand_slice.py:109-205)."""
    lora_b_weights = _stacked(lora_b_weights, "lora_b_weights")
    inputs = _expand_inputs(inputs, lora_b_weights)
    assert b_seq_start_loc.size(0) == batches
    assert lora_indices_tensor.size(0) == batches
    assert slice_size == lora_b_weights.size(-2)
    _check_rows(inputs, output_tensor)
    s_start, s_end = bounds if bounds is not None else segment_bounds(b_seq_start_loc, seq_len_tensor,
                                                                        lora_indices_tensor)
    _native.sgmv_expand(output_tensor, inputs, _segment_pointers(lora_b_weights, lora_indices_tensor), s_start, s_end,
                        get_tmp_tensor_for_size(batches, inputs.device), 0, slice_offset, slice_size,
                        transposed=True, accumulate=add_inputs)


@torch.inference_mode()
def sgmv_expand(
    inputs: torch.Tensor,
    lora_b_weights: torch.Tensor,
    output_tensor: torch.Tensor,
    b_seq_start_loc: torch.Tensor,
    seq_len_tensor: torch.Tensor,
    lora_indices_tensor: torch.Tensor,
    batches: int,
    max_seq_length: int,
    add_inputs: bool = False,
    bounds: Optional[Tuple[torch.Tensor, torch.Tensor]] = None,
):
    """sgmv_expand.py:106-198: the slice operator over the whole width of output_tensor."""
    width = lora_b_weights.size(-2)
    assert output_tensor.size(1) == width
    sgmv_expand_slice(inputs, lora_b_weights, output_tensor, b_seq_start_loc, seq_len_tensor, lora_indices_tensor,
                      batches, max_seq_length, 0, width, add_inputs, bounds)
