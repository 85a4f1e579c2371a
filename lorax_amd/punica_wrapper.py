"""PunicaWrapper: routing state of one batch for the stacked-weight LoRA operators of lorax_amd.ops.

Drop-in for the class of the same name in lorax_server/utils/punica.py (:392-793): same constructor,
same public methods and properties, same meaning of every argument.  The reference reaches it from
LoraLinear.forward_layer_type (utils/layers.py:79-105) with the stacks models/model.py:289-334 builds for
preloaded adapters - lora_a_weights [num_adapters, r, h_in] and lora_b_weights [num_adapters, h_out, r]
per (layer type, layer).

What it keeps per batch is what the HIP kernels consume, in the form they consume it:
  * token slots: int64, the stack entry of every token, -1 = base model (BGMV);
  * runs: int32 bounds [n + 1] and int64 owners [n] of the maximal runs of tokens with one adapter (SGMV).
    They are the batch's own adapter_segments / segment_indices when the metadata object carries them
    (AdapterBatchMetadata does), so a prefill step computes nothing on the device and never waits for it.
The reference's int64 views (start, length and owner per run, punica.py:485-503) are derived from the run
table on request.  The index tensors of the LoRA vocabulary embeddings and of long-context RoPE
(convert_mapping, punica.py:283-388) belong to layers outside the LoRA linear path and are not built.
"""

from typing import Callable, List, Optional, Sequence, Tuple

import torch

from lorax_amd import ops

Slice = Tuple[torch.Tensor, torch.Tensor, int, int]  # (lora_a stack, lora_b stack, first column, width)


def _runs_of(slots: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """Bounds (int64 [n + 1]) and owners ([n]) of the maximal runs of equal values in a 1-D tensor."""
    n = slots.numel()
    if n == 0:
        return slots.new_zeros(1, dtype=torch.int64), slots.new_zeros(0)
    change = torch.nonzero(slots[1:] != slots[:-1]).flatten() + 1
    edge = slots.new_tensor([0], dtype=torch.int64)
    bounds = torch.cat([edge, change.to(torch.int64), edge + n])
    return bounds, slots[bounds[:-1]]


def compute_meta(token_lora_tensor: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, int, int, bool]:
    """(run starts, run lengths, run owners, number of runs, longest run, batch uses no adapter at all) of a
    per-token adapter tensor: neighbouring requests with one adapter count as one run.  Same tuple as
    punica.py:258-281."""
    bounds, owners = _runs_of(token_lora_tensor)
    starts, lengths = bounds[:-1], bounds[1:] - bounds[:-1]
    count = owners.numel()
    longest = int(lengths.max().item()) if count else 0
    nothing_routed = count == 1 and int(owners[0].item()) == -1
    return starts, lengths, owners, count, longest, nothing_routed


class PunicaWrapper:
    def __init__(self, max_num_batched_tokens: int, max_batches: int, device: str, enabled: bool):
        self.enabled = enabled
        self.max_batch_size = max_batches
        self.is_prefill = False
        self.no_lora = False
        self.batch_size = -1  # runs in the current prefill batch
        # lengths of [token slots, request slots, and three tensors this path does not build]
        self.indices_len: List[Optional[int]] = [None] * 5
        # fixed buffers, so that a captured graph keeps reading the same addresses from step to step
        self._token_lora_indices = torch.empty(max_num_batched_tokens, dtype=torch.int64, device=device)
        self._sampler_indices = torch.empty(max_num_batched_tokens, dtype=torch.int64, device=device)
        self._run_bounds = torch.zeros(max_batches + 1, dtype=torch.int32, device=device)
        self._run_owners = torch.empty(max_batches, dtype=torch.int64, device=device)
        self._kernel_bounds: Optional[Tuple[torch.Tensor, torch.Tensor]] = None
        self._max_length: Optional[int] = None
        # decode: the batch's routing plan over stack entries (ops.build_slot_plan), one record per chunk of up
        # to four tokens of one adapter, in a fixed buffer; _plan_records of them are in use
        self._plan = torch.zeros((max_num_batched_tokens, 8), dtype=torch.int64, device=device)
        self._plan_records: Optional[int] = None
        self._plan_filled = 0  # records of the buffer that may be non-zero

    # ---- routing state ----------------------------------------------------------------------------

    def update_metadata(self, meta, prefill: bool):
        """Takes over the routing of one batch.  Adapter index 0 is the base model, so a token's stack entry is
        its adapter index minus one and base-model tokens get -1 (punica.py:420-438)."""
        count = meta.adapter_indices.shape[-1]
        torch.sub(meta.adapter_indices, 1, out=self._token_lora_indices[:count])
        self.indices_len[0] = count
        self.is_prefill = bool(prefill)
        self._plan_records = None
        if not prefill:
            # Routing plan of the decode step: tokens grouped by adapter on the host (one copy of the indices
            # down, as the table builder of the pointer-table path makes, and one copy of the records up), so
            # that no workgroup of the step's launches scans the index tensor and the projections of rank 8 / 16
            # run shrink and expand in one launch.
            if self._token_lora_indices.is_cuda and count <= self._plan.size(0):
                records = ops.build_slot_plan(meta.adapter_indices.detach().cpu().numpy() - 1)
                n, stale = records.size(0), self._plan_filled
                self._plan[:n].copy_(records, non_blocking=True)
                if stale > n:  # records of the batch before: all-zero records are padding the kernels skip, so a
                    self._plan[n:stale].zero_()  # captured step that reads a fixed number of records stays right
                self._plan_records = self._plan_filled = n
            return
        bounds = getattr(meta, "adapter_segments", None)
        owners = getattr(meta, "segment_indices", None)
        if bounds is not None and owners is not None and bounds.numel() == len(owners) + 1:
            # the batch's own run table: nothing to compute
            owner_slots = torch.as_tensor(list(owners), dtype=torch.int64) - 1
            self._set_runs(bounds, owner_slots.to(self._run_owners.device, non_blocking=True),
                           all(o == 0 for o in owners))
        else:
            self._update_prefill_metada(self._token_lora_indices, count)

    def _set_runs(self, bounds: torch.Tensor, owner_slots: torch.Tensor, nothing_routed: bool) -> None:
        n = owner_slots.numel()
        if n > self.max_batch_size:
            raise ValueError(f"{n} runs of tokens exceed max_batches={self.max_batch_size}")
        self._run_bounds[: n + 1].copy_(bounds)
        self._run_owners[:n].copy_(owner_slots)
        self.batch_size = n
        self.no_lora = nothing_routed
        self._max_length = None
        # what the SGMV kernels read: runs of the base model become empty segments
        starts, ends = self._run_bounds[:n], self._run_bounds[1 : n + 1]
        self._kernel_bounds = (starts, torch.where(self._run_owners[:n] >= 0, ends, starts))

    def _update_prefill_metada(self, token_lora_tensor: torch.Tensor, indices_len: int) -> None:
        """Run table from a per-token slot tensor, for metadata objects that carry no run table (the name,
        spelling included, is the reference's, punica.py:472)."""
        bounds, owners = _runs_of(token_lora_tensor[:indices_len])
        nothing_routed = owners.numel() == 1 and int(owners[0].item()) == -1
        self._set_runs(bounds, owners, nothing_routed)

    def set_sampler_indices(self, sampler_indices: torch.Tensor):
        """Stack entry per request, read by add_lora_logits (the second tensor of convert_mapping,
        punica.py:362-363)."""
        n = sampler_indices.shape[-1]
        self._sampler_indices[:n].copy_(sampler_indices)
        self.indices_len[1] = n

    @property
    def max_length(self) -> int:
        """Longest run of the prefill batch; computed (one device read) only if somebody asks."""
        if self._max_length is None:
            n = self.batch_size
            spans = self._run_bounds[1 : n + 1] - self._run_bounds[:n]
            self._max_length = int(spans.max().item()) if n > 0 else 0
        return self._max_length

    @property
    def prefill_metadata(self) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, int, int]:
        """(run starts, run lengths, stack entry per run with -1 = none, number of runs, longest run), the
        tuple of punica.py:485-503, as int64 tensors derived from the run table."""
        n = self.batch_size
        starts = self._run_bounds[:n].to(torch.int64)
        lengths = self._run_bounds[1 : n + 1].to(torch.int64) - starts
        return starts, lengths, self._run_owners[:n], n, self.max_length

    @property
    def token_lora_indices(self) -> torch.Tensor:
        """Stack entry of every token of the batch, -1 = no adapter (punica.py:505-512)."""
        return self._token_lora_indices[: self.indices_len[0]]

    @property
    def sampler_indices(self) -> torch.Tensor:
        """Stack entry of every request (punica.py:514-521)."""
        return self._sampler_indices[: self.indices_len[1]]

    # ---- single operators ---------------------------------------------------------------------------
    # One private dispatcher serves the reference's per-phase method names.

    def _run(self, kind: str, y: torch.Tensor, x: torch.Tensor, w_t_all: torch.Tensor, *, scale: float = 1.0,
             add_input: bool = True, window: Optional[Tuple[int, int]] = None) -> None:
        if self.is_prefill:
            if self.no_lora:  # nothing is routed: no launch (punica.py:557-559)
                return
            starts, ends = self._kernel_bounds
            lengths = ends - starts
            owners, n = self._run_owners[: self.batch_size], self.batch_size
            if kind == "shrink":
                ops.sgmv_shrink(x, w_t_all, y, starts, lengths, owners, n, 0, scale, bounds=self._kernel_bounds)
            elif window is None:
                ops.sgmv_expand(x, w_t_all, y, starts, lengths, owners, n, 0, add_input, bounds=self._kernel_bounds)
            else:
                ops.sgmv_expand_slice(x, w_t_all, y, starts, lengths, owners, n, 0, window[0], window[1], add_input,
                                      bounds=self._kernel_bounds)
            return
        slots = self.token_lora_indices
        if kind == "shrink":
            ops.bgmv_shrink(x, w_t_all, y, slots, scale)
        elif window is None:
            ops.bgmv_expand(x, w_t_all, y, slots, add_input)
        else:
            ops.bgmv_expand_slice(x, w_t_all, y, slots, window[0], window[1], add_input)

    def _in_phase(self, prefill: bool, *args, **kwargs) -> None:
        saved, self.is_prefill = self.is_prefill, prefill
        try:
            self._run(*args, **kwargs)
        finally:
            self.is_prefill = saved

    def shrink_prefill(self, y, x, w_t_all, scale: float):
        self._in_phase(True, "shrink", y, x, w_t_all, scale=scale)

    def shrink_decode(self, y, x, w_t_all, scale: float):
        self._in_phase(False, "shrink", y, x, w_t_all, scale=scale)

    def expand_prefill(self, y, x, w_t_all, add_input: bool):
        self._in_phase(True, "expand", y, x, w_t_all, add_input=add_input)

    def expand_decode(self, y, x, w_t_all, add_input: bool):
        self._in_phase(False, "expand", y, x, w_t_all, add_input=add_input)

    def expand_slice_prefill(self, y, x, w_t_all, y_offset: Optional[int], y_slice_size: Optional[int], add_input: bool):
        self._in_phase(True, "expand", y, x, w_t_all, add_input=add_input, window=(y_offset, y_slice_size))

    def expand_slice_decode(self, y, x, w_t_all, y_offset: Optional[int], y_slice_size: Optional[int], add_input: bool):
        self._in_phase(False, "expand", y, x, w_t_all, add_input=add_input, window=(y_offset, y_slice_size))

    def add_shrink(self, y: torch.Tensor, x: torch.Tensor, w_t_all: torch.Tensor, scale: float):
        """y += scale * x @ w_t_all[slot].T, the product with LoRA A (punica.py:636-652)."""
        self._run("shrink", y, x, w_t_all, scale=scale)

    def add_expand(self, y: torch.Tensor, x: torch.Tensor, w_t_all: torch.Tensor, add_input: bool = True):
        """y (+)= x @ w_t_all[slot].T, the product with LoRA B (punica.py:654-671)."""
        self._run("expand", y, x, w_t_all, add_input=add_input)

    def add_expand_slice(self, y: torch.Tensor, x: torch.Tensor, w_t_all: torch.Tensor, y_offset: Optional[int],
                         y_slice_size: Optional[int], add_input: bool = True):
        """add_expand into the columns [y_offset, y_offset + y_slice_size) of y (punica.py:673-687)."""
        self._run("expand", y, x, w_t_all, add_input=add_input, window=(y_offset, y_slice_size))

    # ---- whole LoRA updates -------------------------------------------------------------------------

    def add_lora_slices(self, y: torch.Tensor, x: torch.Tensor, slices: Sequence[Slice], scale: float,
                        callback: Optional[Callable] = None, buffer: Optional[torch.Tensor] = None) -> None:
        """y[:, first : first + width] += scale * (x @ A[slot].T) @ B[slot].T for every slice; the slices share x.

        Without anything that must see the intermediate product (a `callback` that gathers it across ranks, a
        caller-owned `buffer`), all slices go to the kernels together: in decode one shrink launch and one
        expand launch for the lot, in prefill one shrink launch per summed rank of 128 and one expand per
        slice.  The intermediate then stays in the type of x; the reference's fp32 buffer is rounded to the
        weight type by its expand operators before they multiply (CAST_TYPE, sgmv_expand.py:160-165), so y is
        the same and the buffer costs half the traffic and no conversion launch."""
        if not slices:
            return
        rows_y, rows_x = y.view(-1, y.shape[-1]), x.view(-1, x.shape[-1])
        half = rows_x.dtype in (torch.float16, torch.bfloat16)
        together = (callback is None and buffer is None and half
                    and all(a.dtype == rows_x.dtype and b.dtype == rows_x.dtype for a, b, _, _ in slices))
        if together:
            if not self.is_prefill:
                plan = self._plan[: self._plan_records] if self._plan_records is not None else None
                ops.bgmv_lora_slices(rows_x, slices, rows_y, self.token_lora_indices, scale, plan=plan)
            elif not self.no_lora:
                starts, ends = self._kernel_bounds
                ops.sgmv_lora_slices(rows_x, slices, rows_y, starts, ends - starts, self._run_owners[: self.batch_size],
                                     self.batch_size, 0, scale, bounds=self._kernel_bounds)
            return
        for lora_a, lora_b, first, width in slices:
            mid = buffer
            if mid is None:
                mid = torch.zeros((rows_x.size(0), lora_b.size(-1)), dtype=rows_x.dtype, device=rows_x.device)
            self._run("shrink", mid, rows_x, lora_a, scale=scale)
            if callback is not None:
                mid = callback(mid)  # e.g. all-gather / all-reduce of the intermediate across ranks
            whole = first == 0 and width == rows_y.shape[1]
            self._run("expand", rows_y, mid, lora_b, add_input=True, window=None if whole else (first, width))

    def add_lora(self, y: torch.Tensor, x: torch.Tensor, wa_t_all: torch.Tensor, wb_t_all: torch.Tensor, scale: float,
                 y_offset: Optional[int] = None, y_slice_size: Optional[int] = None, *,
                 buffer: Optional[torch.Tensor] = None, callback: Optional[Callable] = None):
        """y[i] += x[i] @ wa_t_all[slot[i]].T @ wb_t_all[slot[i]].T * scale, in place, optionally into a column
        window of y (punica.py:689-740)."""
        if y_offset is None and y_slice_size is None:
            y_offset, y_slice_size = 0, y.shape[-1]
        self.add_lora_slices(y, x, [(wa_t_all, wb_t_all, y_offset, y_slice_size)], scale, callback=callback,
                             buffer=buffer)

    def add_lora_packed_nslice(self, y: torch.Tensor, x: torch.Tensor, lora_a_stacked: Tuple[torch.Tensor, ...],
                               lora_b_stacked: Tuple[torch.Tensor, ...], scale: float,
                               output_slices: Tuple[int, ...]) -> None:
        """add_lora for the slices of a packed projection (q/k/v, gate/up) laid out one after the other in y
        (punica.py:742-767)."""
        firsts = [sum(output_slices[:i]) for i in range(len(output_slices))]
        self.add_lora_slices(y, x, list(zip(lora_a_stacked, lora_b_stacked, firsts, output_slices)), scale)

    def add_lora_logits(self, y: torch.Tensor, x: torch.Tensor, wa_t_all: torch.Tensor, wb_t_all: torch.Tensor, scale,
                        *, buffer: Optional[torch.Tensor] = None) -> None:
        """The LoRA of the LM head: one row per request, routed by the request slots (set_sampler_indices),
        always with the per-token kernels (punica.py:769-793)."""
        rows_y, rows_x = y.view(-1, y.shape[-1]), x.view(-1, x.shape[-1])
        mid = buffer
        if mid is None:
            mid = torch.zeros((rows_x.size(0), wb_t_all.size(-1)), dtype=rows_x.dtype, device=rows_x.device)
        ops.bgmv_shrink(rows_x, wa_t_all, mid, self.sampler_indices, scale)
        ops.bgmv_expand(mid, wb_t_all, rows_y, self.sampler_indices, add_inputs=True)
