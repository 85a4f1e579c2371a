"""LoRA-augmented linear layers: the callers of the SGMV/BGMV kernels.

Mirrors ``lorax_server/utils/layers.py:59-300``: ``LoraLinear.forward_layer_type`` (the
"legacy punica" branch, :107-167), ``TensorParallelMultiAdapterLinear`` (fused q/k/v and
gate/up outputs, one column slice per layer name, :217-255) and
``TensorParallelAdapterRowLinear`` (o_proj / down_proj, :270-289).

Deliberate differences from the reference:
  * its third branch, the per-adapter masked matmul loop (:169-211), is not part of this
    package: a batch the kernels cannot take raises instead of silently running dense
    PyTorch code;
  * a projection that owns only a column slice of the fused output is written in place
    through the kernels' column window instead of through a zero-filled staging tensor
    and a second pass (:109-112,166-167).  Every token belongs to at most one rank
    group, so both orders round identically;
  * in prefill the shrink overwrites the rows of the segments in v, so v is not zero-filled first
    (utils/punica.py:176-178 allocates zeros); the expand reads no other rows;
  * the LM head takes the same kernels (MultiAdapterHead): the reference excludes it from its kernel path
    (adapters/lora.py:243-247) and runs the dense loop, because its BGMV kernels stop at 65 535 columns;
  * in decode, the projections of one layer that share an input (q/k/v, gate/up) go to the
    GPU as ONE shrink launch and ONE expand launch per rank (``lorax_bgmv_multi``), and the
    shrink overwrites v, so there is no zero-fill (:146).  A decode-size BGMV is shorter
    than a kernel launch; the reference issues 3 launches per projection and rank.
"""

from collections import defaultdict
from typing import List, Optional, Sequence, Tuple

import torch
from torch import nn

from lorax_amd import _native
from lorax_amd.adapters import LORA, AdapterBatchData, BatchLoraWeights
from lorax_amd._native import MAX_SGMV_SHRINK_PROBLEMS
from lorax_amd.sgmv import (
    MAX_RANK_CUSTOM,
    get_shrink_scratch,
    get_tmp_expand_size,
    has_sgmv,
    lora_a_sgmv_cutlass,
    lora_a_sgmv_resident,
    lora_b_sgmv_cutlass,
    lora_b_sgmv_cutlass_slice,
    resident_shrink_applies,
)


class SingleProcessGroup:
    """A process group of one rank (the reference's FakeGroup, utils/dist.py:19-45)."""

    def size(self) -> int:
        return 1

    def rank(self) -> int:
        return 0


class LoraLinear(nn.Module):
    def __init__(self, base_layer, layer_id: int, process_group=None):
        super().__init__()
        self.base_layer = base_layer
        self.layer_id = layer_id
        self.process_group = process_group if process_group is not None else SingleProcessGroup()

    def _lora_data(self, adapter_data: AdapterBatchData, layer_type: str) -> Optional[BatchLoraWeights]:
        layer_data = adapter_data.data.get(layer_type)
        data = layer_data.get(LORA) if layer_data is not None else None
        if data is None:
            return None  # no adapter in the batch targets this projection
        if not has_sgmv():
            raise RuntimeError("LoRA kernels unavailable: liblorax_hip.so is not loaded or DISABLE_SGMV is set")
        if not data.can_vectorize(self.process_group):
            raise RuntimeError(
                f"layer type {layer_type!r}: ranks {sorted(data.rank_data)} are outside what the LoRA kernels "
                "cover (rank / world_size <= 128)"
            )
        return data

    def forward_layer_types(
        self,
        result: torch.Tensor,
        input: torch.Tensor,
        adapter_data: AdapterBatchData,
        slices: Sequence[Tuple[str, int, int]],
    ) -> torch.Tensor:
        """Adds the LoRA deltas of several projections that share `input`; projection `name` owns the
        columns [start, end) of `result`."""
        tensor_parallel = self.process_group.size() > 1
        decode_jobs = defaultdict(list)  # (wave, rank) -> [(rank_segments, start, width)]
        stacked_jobs = []  # (lora_a_stack, lora_b_stack, start, width) of projections served by stacked weights
        prefill_jobs = defaultdict(list)  # (rank, segment tables) -> [(rank_segments, start, width)]
        for name, start, end in slices:
            data = self._lora_data(adapter_data, name)
            if data is None:
                continue
            # Stacked weights of preloaded adapters (utils/layers.py:79-105): one index into a
            # [num_adapters, ...] stack per token instead of pointer tables per rank.
            key = (name, self.layer_id)
            wrapper = adapter_data.punica_wrapper
            if (
                wrapper is not None
                and wrapper.enabled
                and key in adapter_data.layer_to_lora_weights
                and input.shape[0] <= wrapper.max_batch_size
            ):
                lora_a_weights, lora_b_weights = adapter_data.layer_to_lora_weights[key]
                stacked_jobs.append((lora_a_weights, lora_b_weights, start, end - start))
                continue
            sliced = end - start != result.shape[1]
            for group_key, rs in data.rank_data.items():
                r = rs.rank  # the kernels' rank: that of the group, or of its chunk of a rank above 128
                if not data.use_sgmv:
                    if rs.lora_a_ptr is None or rs.lora_b_ptr is None:
                        continue
                    # the chunks of one adapter update the same elements of the result: one launch per chunk number
                    wave = group_key[1] if isinstance(group_key, tuple) else 0
                    decode_jobs[(wave, r)].append((rs, start, end - start))
                    continue
                # Prefill reads the resident stacks ([L, r, h_in] and [L, h_out, r], the ones decode uses);
                # the reference's prefill layouts are only touched for shapes the resident-layout shrink
                # does not take.
                if rs.lora_a_t_ptr is not None and resident_shrink_applies(r, input.size(1), input.size(0)):
                    if rs.segments_key is not None and rs.lora_b_t_ptr is not None and not tensor_parallel:
                        prefill_jobs[(r, rs.segments_key)].append((rs, start, end - start))
                        continue
                    whole = rs.num_long_segments == rs.segment_starts.numel()  # the plans cover the long segments
                    v = lora_a_sgmv_resident(
                        input, get_shrink_scratch(input.device), rs.lora_a_t_ptr, rs.segment_starts, rs.segment_ends,
                        self.layer_id, r, zero_fill=tensor_parallel, tiles=rs.shrink_tiles if whole else None,
                    )
                else:
                    if rs.lora_a_ptr is None:
                        raise RuntimeError(
                            f"rank chunk of {r} over h_in={input.size(1)}: no kernel takes this shape from the resident "
                            "layout, and rank chunks have no other"
                        )
                    v = lora_a_sgmv_cutlass(
                        input, rs.tmp_shrink, rs.lora_a_ptr, rs.segment_starts, rs.segment_ends, self.layer_id, r
                    )
                if tensor_parallel:
                    v = self.collect_lora_a(v)
                if rs.lora_b_t_ptr is not None:
                    whole = rs.num_long_segments == rs.segment_starts.numel()
                    lora_b_sgmv_cutlass_slice(
                        result, v, rs.tmp_expand, rs.lora_b_t_ptr, rs.segment_starts, rs.segment_ends,
                        self.layer_id, start, end - start, transposed=True, tiles=rs.expand_tiles if whole else None,
                    )
                elif sliced:
                    lora_b_sgmv_cutlass_slice(
                        result, v, rs.tmp_expand, rs.lora_b_ptr, rs.segment_starts, rs.segment_ends,
                        self.layer_id, start, end - start,
                    )
                else:
                    lora_b_sgmv_cutlass(
                        result, v, rs.tmp_expand, rs.lora_b_ptr, rs.segment_starts, rs.segment_ends, self.layer_id
                    )

        # Prefill: projections of one rank with the same segment tables (q/k/v, gate/up of adapters that target
        # them all) shrink together, as many per launch as fit a summed rank of 128 - x is read once per
        # launch; the reference issues one shrink per projection (utils/layers.py:121-133).
        for (r, _), group in prefill_jobs.items():
            if _native.sgmv_lora_fits(r, input.size(1), input.size(0), max(width for _, _, width in group)):
                # a short batch is bound by launches: shrink and expand of up to four projections in one
                step = _native.MAX_FUSED_BGMV_PROBLEMS
                for i in range(0, len(group), step):
                    first = group[i][0]
                    _native.sgmv_lora_multi(
                        [(result, rs.lora_a_t_ptr, rs.lora_b_t_ptr, start, width) for rs, start, width in group[i : i + step]],
                        input, first.segment_starts, first.segment_ends, r, self.layer_id,
                    )
                continue
            # Many segments of a few rows (decode tokens inside a prefill batch): the tables list them last and a
            # routing plan covers their rows.  The segment kernels then take the long segments only and the
            # per-token kernels the rest - they stream an adapter's weights faster than one row tile per segment
            # can, and once for up to four rows.  Both write disjoint rows of v and of the result.
            first = group[0][0]
            plans = [rs.short_plan for rs, _, _ in group]
            # (the per-token kernels number rows and plan records with 16 bits; beyond that the segment kernels
            # take the whole tables, which still list every segment)
            split = (all(p is not None for p in plans) and input.size(0) <= _native.MAX_BGMV_TOKENS
                     and all(p.size(0) <= _native.MAX_BGMV_TOKENS for p in plans))
            n_long = first.num_long_segments if split else first.segment_starts.numel()
            starts, ends = first.segment_starts[:n_long], first.segment_ends[:n_long]
            # the tables' row-tile plans cover their first num_long_segments entries
            planned = n_long == first.num_long_segments
            shrink_tiles = first.shrink_tiles if planned else None
            expand_tiles = first.expand_tiles if planned else None
            # v needs no zero-fill: the shrinks overwrite the rows of their segments and the expands read no others
            flat = torch.empty((len(group), input.size(0), r), dtype=input.dtype, device=input.device)
            vs = list(flat.unbind(0))
            step = max(1, min(MAX_SGMV_SHRINK_PROBLEMS, MAX_RANK_CUSTOM // r))
            # (no long segment at all: the per-token launches do the whole update)
            for i in range(0, len(group) if n_long > 0 else 0, step):
                _native.sgmv_shrink_multi(
                    vs[i : i + step], input, [rs.lora_a_t_ptr[:n_long] for rs, _, _ in group[i : i + step]],
                    starts, ends, get_shrink_scratch(input.device), self.layer_id, 1.0, False, shrink_tiles,
                )
            batch = _native.MAX_BGMV_PROBLEMS
            if split:  # the short rows of every projection of the group in one launch
                for i in range(0, len(group), batch):
                    _native.bgmv_multi([(v, input, None, None, 0, None) for v in vs[i : i + batch]], self.layer_id,
                                       1.0, accumulate=False, plans=plans[i : i + batch])
            for v, (rs, start, width) in zip(vs, group) if n_long > 0 else ():
                lora_b_sgmv_cutlass_slice(
                    result, v, rs.tmp_expand[: get_tmp_expand_size(n_long)], rs.lora_b_t_ptr[:n_long], starts, ends,
                    self.layer_id, start, width, transposed=True, tiles=expand_tiles,
                )
            if split:
                for i in range(0, len(group), batch):
                    _native.bgmv_multi(
                        [(result, v, None, None, start, width)
                         for v, (_, start, width) in zip(vs[i : i + batch], group[i : i + batch])],
                        self.layer_id, 1.0, accumulate=True, plans=plans[i : i + batch],
                    )

        if stacked_jobs:  # the reference calls add_lora once per projection (utils/layers.py:92-104)
            adapter_data.punica_wrapper.add_lora_slices(
                result, input, stacked_jobs, 1.0, callback=self.collect_lora_a if tensor_parallel else None
            )

        # Decode.  When every job of the call has a small A slab (rank 8 or 16, moderate widths), shrink and
        # expand run in one launch per rank and v never leaves the chip.  Otherwise all rank groups of all
        # projections go out together: one shrink launch and one expand launch per 16 problems, whatever the
        # mix of ranks (the reference issues a pair of launches per projection and rank, layers.py:146-164).
        waves = sorted({wave for wave, _ in decode_jobs})
        if len(waves) > 1:
            for wave in waves:
                self._decode(result, input, {k: v for k, v in decode_jobs.items() if k[0] == wave}, tensor_parallel)
            return result
        return self._decode(result, input, decode_jobs, tensor_parallel)

    def _decode(self, result, input, decode_jobs, tensor_parallel):
        """The decode launches of forward_layer_types for jobs that touch disjoint elements of `result`:
        decode_jobs maps (wave, rank) to [(rank_segments, start, width)]."""
        jobs = [(r, rs, start, width) for (_, r), rank_jobs in decode_jobs.items() for rs, start, width in rank_jobs]
        all_fused = bool(jobs) and not tensor_parallel and all(
            rs.plan is not None and _native.bgmv_lora_fits(r, input.size(1), width) for r, rs, _, width in jobs
        )
        if all_fused:
            step = _native.MAX_FUSED_BGMV_PROBLEMS
            for r in sorted({r for _, r in decode_jobs}):
                single = [j for j in jobs if j[0] == r]
                for i in range(0, len(single), step):
                    _native.bgmv_lora_multi(
                        [(result, input, rs.plan, start, width) for _, rs, start, width in single[i : i + step]],
                        r, self.layer_id,
                    )
            return result
        step = _native.MAX_BGMV_PROBLEMS
        for i in range(0, len(jobs), step):
            chunk = jobs[i : i + step]
            # v needs no zero-fill: the shrink overwrites the rows of routed tokens and the expand reads
            # no others.  One buffer, one [T, r] slice of it per problem.
            widths = [r for r, _, _, _ in chunk]
            flat = torch.empty((input.size(0) * sum(widths),), dtype=input.dtype, device=input.device)
            vs, pos = [], 0
            for r in widths:
                vs.append(flat[pos : pos + input.size(0) * r].view(input.size(0), r))
                pos += input.size(0) * r
            plans = [rs.plan for _, rs, _, _ in chunk]
            if any(p is None for p in plans):
                plans = None  # tables not built by BatchLoraWeights.load: the kernels group tokens themselves
            _native.bgmv_multi(
                [(v, input, rs.lora_a_ptr, rs.indices, 0, None) for v, (_, rs, _, _) in zip(vs, chunk)],
                self.layer_id, 1.0, accumulate=False, plans=plans,
            )
            if tensor_parallel:
                vs = [self.collect_lora_a(v) for v in vs]
            _native.bgmv_multi(
                [(result, v, rs.lora_b_ptr, rs.indices, start, width) for v, (_, rs, start, width) in zip(vs, chunk)],
                self.layer_id, 1.0, accumulate=True, plans=plans,
            )
        return result

    def forward_layer_type(
        self,
        result: torch.Tensor,
        input: torch.Tensor,
        adapter_data: AdapterBatchData,
        layer_type: str,
        start_idx: int,
        end_idx: int,
    ) -> torch.Tensor:
        """One projection, with the reference's signature (utils/layers.py:66-74)."""
        return self.forward_layer_types(result, input, adapter_data, [(layer_type, start_idx, end_idx)])

    def collect_lora_a(self, a_out: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError("tensor-parallel exchange of the shrink output is outside this package")


class TensorParallelMultiAdapterLinear(LoraLinear):
    """Column-parallel projection(s) sharing one input: q/k/v or gate/up (utils/layers.py:217-255)."""

    def __init__(self, base_layer, layer_id: int, layer_names: List[str], sizes: Optional[List[int]], process_group=None):
        super().__init__(base_layer, layer_id, process_group)
        self.layer_names = layer_names
        self.sizes = sizes

    @classmethod
    def load(cls, base_layer, layer_id, layer_names, sizes, process_group=None):
        return cls(base_layer, layer_id, layer_names, sizes, process_group)

    def forward(self, input: torch.Tensor, adapter_data: AdapterBatchData) -> torch.Tensor:
        result = self.base_layer(input)
        out_shape = result.shape
        if input.dim() >= 3:
            # (batch, seq, hidden) models: the kernels want one row per token
            input = input.reshape(-1, input.shape[-1])
            result = result.reshape(-1, result.shape[-1])
        world = self.process_group.size()
        slices = []
        offset = 0
        for i, name in enumerate(self.layer_names):
            start = offset // world
            if self.sizes is not None:
                offset += self.sizes[i]
                end = offset // world
            else:
                end = result.shape[1]
            slices.append((name, start, end))
        result = self.forward_layer_types(result, input, adapter_data, slices)
        return result.reshape(out_shape)


class TensorParallelAdapterRowLinear(LoraLinear):
    """Row-parallel projection: o_proj / down_proj (utils/layers.py:270-289)."""

    def __init__(self, base_layer, layer_id: int, layer_name: str, process_group=None):
        super().__init__(base_layer, layer_id, process_group)
        self.layer_name = layer_name

    @classmethod
    def load(cls, base_layer, layer_id, layer_name, process_group=None):
        return cls(base_layer, layer_id, layer_name, process_group)

    def forward(self, input: torch.Tensor, adapter_data: AdapterBatchData) -> torch.Tensor:
        result = self.base_layer(input)
        stride = result.shape[-1] // self.process_group.size()
        start = self.process_group.rank() * stride
        self.forward_layer_type(result, input, adapter_data, self.layer_name, start, start + stride)
        return result


class MultiAdapterHead(TensorParallelAdapterRowLinear):
    """The LM head with LoRA (utils/layers.py:303-326).  In a prefill batch its input holds one row per request
    (the last token's hidden state); BatchLoraWeights.load has recounted the segment bounds in those rows from
    prefill_head_indices, so the same kernels apply.  Returns (logits, speculative_logits); the Medusa heads
    that would fill the second slot are not part of this package, so it is always None."""

    def forward(self, input: torch.Tensor, adapter_data: AdapterBatchData):
        return super().forward(input, adapter_data), None
