"""PunicaWrapper: the metadata holder and operator front end of the reference's stacked-weight LoRA path
(lorax_server/utils/punica.py:256-793, derived from vLLM), over the HIP operators of lorax_amd.ops.

The reference reaches this path from LoraLinear.forward_layer_type (utils/layers.py:79-105) with the
stacks model.py:289-334 builds for preloaded adapters: lora_a_weights [num_adapters, r, h_in] and
lora_b_weights [num_adapters, h_out, r] per (layer type, layer).  Only the methods on that path and the
metadata they read are here: update_metadata, the prefill metadata, token_lora_indices, add_shrink,
add_expand, add_expand_slice, add_lora, add_lora_packed_nslice and add_lora_logits.  The index tensors of
the LoRA vocabulary embeddings and of long-context RoPE (convert_mapping, punica.py:283-388) belong to
layers outside the LoRA linear path and are not built.
"""

from typing import Callable, List, Optional, Tuple

import torch

from lorax_amd import ops


def compute_meta(token_lora_tensor: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, int, int, bool]:
    """Run-length metadata of a prefill batch (punica.py:256-280): start, length and adapter number of every run
    of consecutive tokens with the same adapter, the number of runs, the longest run, and whether the batch
    uses no adapter at all."""
    lora_indices_tensor, seq_length_tensor = torch.unique_consecutive(token_lora_tensor, return_counts=True)
    cum_result = torch.cumsum(seq_length_tensor, dim=0)
    b_seq_start_tensor = torch.zeros_like(seq_length_tensor)
    b_seq_start_tensor[1:].copy_(cum_result[:-1])
    max_length = seq_length_tensor.max().item()
    batch_size = lora_indices_tensor.size(0)
    no_lora = bool(batch_size == 1 and lora_indices_tensor == -1)
    return (b_seq_start_tensor, seq_length_tensor, lora_indices_tensor, batch_size, max_length, no_lora)


class PunicaWrapper:
    """State of one batch for the stacked-weight operators (punica.py:392-418)."""

    def __init__(self, max_num_batched_tokens: int, max_batches: int, device: str, enabled: bool):
        self._token_lora_indices = torch.empty(max_num_batched_tokens, dtype=torch.long, device=device)
        self._sampler_indices = torch.empty(max_num_batched_tokens, dtype=torch.long, device=device)
        # token_lora_indices, sampler_indices and three index tensors of layers outside the LoRA linear path
        self.indices_len: List[Optional[int]] = [None] * 5
        self._seq_start_locs = torch.empty(max_batches, dtype=torch.long, device=device)
        self._seq_lengths = torch.empty(max_batches, dtype=torch.long, device=device)
        self._lora_indices_per_batch = torch.empty(max_batches, dtype=torch.long, device=device)
        # int32 segment bounds for the SGMV kernels, derived once per batch from the three tensors above
        self._segment_starts = torch.empty(max_batches, dtype=torch.int32, device=device)
        self._segment_ends = torch.empty(max_batches, dtype=torch.int32, device=device)
        self.max_batch_size = max_batches
        self.max_length: int = 0
        self.batch_size: int = -1
        self.is_prefill = False
        self.no_lora = False
        self.enabled = enabled

    # ---- metadata ------------------------------------------------------------------------------

    def update_metadata(self, meta, prefill: bool):
        """punica.py:420-438.  Adapter index 0 is the base model, so the stack entry of a token is its
        adapter index minus one and base-model tokens get -1."""
        base_indices = meta.adapter_indices - 1
        self._token_lora_indices[: base_indices.shape[0]].copy_(base_indices)
        self.indices_len[0] = base_indices.shape[-1]
        if prefill:
            self._update_prefill_metada(self._token_lora_indices, base_indices.shape[-1])
            self.is_prefill = True
        else:
            self.is_prefill = False

    def set_sampler_indices(self, sampler_indices: torch.Tensor):
        """Adapter number per request for add_lora_logits (the second tensor of convert_mapping,
        punica.py:362-363)."""
        self._sampler_indices[: sampler_indices.shape[0]].copy_(sampler_indices)
        self.indices_len[1] = sampler_indices.shape[-1]

    def _update_prefill_metada(self, token_lora_tensor: torch.Tensor, indices_len: int) -> None:
        """punica.py:472-483, plus the kernels' int32 segment bounds."""
        (b_seq_start_tensor, seq_length_tensor, lora_indices_tensor, batch_size, max_length, no_lora) = compute_meta(
            token_lora_tensor[:indices_len]
        )
        self._seq_start_locs[: b_seq_start_tensor.shape[0]].copy_(b_seq_start_tensor)
        self._seq_lengths[: seq_length_tensor.shape[0]].copy_(seq_length_tensor)
        self._lora_indices_per_batch[: lora_indices_tensor.shape[0]].copy_(lora_indices_tensor)
        starts, ends = ops.segment_bounds(b_seq_start_tensor, seq_length_tensor, lora_indices_tensor)
        self._segment_starts[:batch_size].copy_(starts)
        self._segment_ends[:batch_size].copy_(ends)
        self.batch_size = batch_size
        self.max_length = max_length
        self.no_lora = no_lora

    @property
    def prefill_metadata(self) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, int, int]:
        """(sequence starts, sequence lengths, adapter number per sequence with -1 = none, number of
        sequences after merging neighbours with the same adapter, longest sequence), punica.py:485-503."""
        return (
            self._seq_start_locs[: self.batch_size],
            self._seq_lengths[: self.batch_size],
            self._lora_indices_per_batch[: self.batch_size],
            self.batch_size,
            self.max_length,
        )

    @property
    def _bounds(self) -> Tuple[torch.Tensor, torch.Tensor]:
        return self._segment_starts[: self.batch_size], self._segment_ends[: self.batch_size]

    @property
    def token_lora_indices(self) -> torch.Tensor:
        """Stack entry of every token of the batch, -1 = no adapter (punica.py:505-512)."""
        return self._token_lora_indices[: self.indices_len[0]]

    @property
    def sampler_indices(self) -> torch.Tensor:
        """punica.py:514-521."""
        return self._sampler_indices[: self.indices_len[1]]

    # ---- operators -----------------------------------------------------------------------------

    def shrink_prefill(self, y: torch.Tensor, x: torch.Tensor, w_t_all: torch.Tensor, scale: float):
        if self.no_lora:  # punica.py:557-559
            return
        ops.sgmv_shrink(x, w_t_all, y, *self.prefill_metadata, scale, bounds=self._bounds)

    def shrink_decode(self, y: torch.Tensor, x: torch.Tensor, w_t_all: torch.Tensor, scale: float):
        ops.bgmv_shrink(x, w_t_all, y, self.token_lora_indices, scale)

    def expand_prefill(self, y: torch.Tensor, x: torch.Tensor, w_t_all: torch.Tensor, add_input: bool):
        if self.no_lora:
            return
        ops.sgmv_expand(x, w_t_all, y, *self.prefill_metadata, add_input, bounds=self._bounds)

    def expand_decode(self, y: torch.Tensor, x: torch.Tensor, w_t_all: torch.Tensor, add_input: bool):
        ops.bgmv_expand(x, w_t_all, y, self.token_lora_indices, add_input)

    def expand_slice_prefill(self, y: torch.Tensor, x: torch.Tensor, w_t_all: torch.Tensor, y_offset: Optional[int],
                             y_slice_size: Optional[int], add_input: bool):
        if self.no_lora:
            return
        ops.sgmv_expand_slice(x, w_t_all, y, *self.prefill_metadata, y_offset, y_slice_size, add_input,
                              bounds=self._bounds)

    def expand_slice_decode(self, y: torch.Tensor, x: torch.Tensor, w_t_all: torch.Tensor, y_offset: Optional[int],
                            y_slice_size: Optional[int], add_input: bool):
        ops.bgmv_expand_slice(x, w_t_all, y, self.token_lora_indices, y_offset, y_slice_size, add_input)

    def add_shrink(self, y: torch.Tensor, x: torch.Tensor, w_t_all: torch.Tensor, scale: float):
        """y += x @ w_t_all[idx].T * scale, the product with LoRA A (punica.py:643-660)."""
        shrink_fun: Callable = self.shrink_prefill if self.is_prefill else self.shrink_decode
        shrink_fun(y, x, w_t_all, scale)

    def add_expand(self, y: torch.Tensor, x: torch.Tensor, w_t_all: torch.Tensor, add_input: bool = True):
        """y (+)= x @ w_t_all[idx].T, the product with LoRA B (punica.py:662-680)."""
        expand_fun: Callable = self.expand_prefill if self.is_prefill else self.expand_decode
        expand_fun(y, x, w_t_all, add_input)

    def add_expand_slice(self, y: torch.Tensor, x: torch.Tensor, w_t_all: torch.Tensor, y_offset: Optional[int],
                         y_slice_size: Optional[int], add_input: bool = True):
        """As add_expand, into columns [y_offset, y_offset + y_slice_size) of y (punica.py:682-696)."""
        expand_slice_fun: Callable = self.expand_slice_prefill if self.is_prefill else self.expand_slice_decode
        expand_slice_fun(y, x, w_t_all, y_offset, y_slice_size, add_input)

    def add_lora(
        self,
        y: torch.Tensor,
        x: torch.Tensor,
        wa_t_all: torch.Tensor,
        wb_t_all: torch.Tensor,
        scale: float,
        y_offset: Optional[int] = None,
        y_slice_size: Optional[int] = None,
        *,
        buffer: Optional[torch.Tensor] = None,
        callback: Optional[Callable] = None,
    ):
        """y[i] += x[i] @ wa_t_all[idx[i]].T @ wb_t_all[idx[i]].T * scale, in place (punica.py:698-748).

        Without a `buffer` from the caller the intermediate x @ A is kept in the type of x instead of the
        reference's fp32: its expand operators round the fp32 buffer to the weight type before they multiply
        (CAST_TYPE), so y is the same and the buffer costs half the traffic and no conversion launch."""
        y_org = y
        y = y.view(-1, y.shape[-1])
        x = x.view(-1, x.shape[-1])
        r = wb_t_all.size(-1)
        if buffer is None:
            buffer = torch.zeros((x.size(0), r), dtype=x.dtype, device=x.device)
        self.add_shrink(buffer, x, wa_t_all, scale)
        if callback is not None:
            # callback used to aggregate intermediate results (i.e., allreduce, allgather)
            buffer = callback(buffer)
        if y_offset is None and y_slice_size is None:
            self.add_expand(y, buffer, wb_t_all, add_input=True)
        else:
            self.add_expand_slice(y, buffer, wb_t_all, y_offset, y_slice_size, add_input=True)
        y = y.view_as(y_org)

    def add_lora_slices(self, y: torch.Tensor, x: torch.Tensor, slices, scale: float,
                        callback: Optional[Callable] = None) -> None:
        """add_lora for several column slices of y that share x; `slices` is a sequence of
        (wa_t_all, wb_t_all, y_offset, y_slice_size).  Without a callback between shrink and expand the shrinks
        of the slices run together (decode: one launch, and one for all expands; prefill: one launch per summed
        rank of 128); otherwise one add_lora per slice."""
        if not slices:
            return
        y2 = y.view(-1, y.shape[-1])
        x2 = x.view(-1, x.shape[-1])
        batched = (callback is None and x2.dtype in (torch.float16, torch.bfloat16)
                   and all(wa.dtype == x2.dtype and wb.dtype == x2.dtype for wa, wb, _, _ in slices))
        if batched and not self.is_prefill:
            ops.bgmv_lora_slices(x2, slices, y2, self.token_lora_indices, scale)
            return
        if batched:
            if not self.no_lora:  # punica.py:557-559
                ops.sgmv_lora_slices(x2, slices, y2, *self.prefill_metadata, scale, bounds=self._bounds)
            return
        for wa_t_all, wb_t_all, y_offset, y_slice_size in slices:
            whole = y_offset == 0 and y_slice_size == y2.shape[1]
            self.add_lora(y2, x2, wa_t_all, wb_t_all, scale, None if whole else y_offset,
                          None if whole else y_slice_size, callback=callback)

    def add_lora_packed_nslice(
        self,
        y: torch.Tensor,
        x: torch.Tensor,
        lora_a_stacked: Tuple[torch.Tensor, ...],
        lora_b_stacked: Tuple[torch.Tensor, ...],
        scale: float,
        output_slices: Tuple[int, ...],
    ) -> None:
        """add_lora for every slice of a packed projection (q/k/v, gate/up), punica.py:750-773."""
        slices, offset_left = [], 0
        for slice_idx in range(len(output_slices)):
            slices.append((lora_a_stacked[slice_idx], lora_b_stacked[slice_idx], offset_left, output_slices[slice_idx]))
            offset_left += output_slices[slice_idx]
        self.add_lora_slices(y, x, slices, scale)

    def add_lora_logits(
        self,
        y: torch.Tensor,
        x: torch.Tensor,
        wa_t_all: torch.Tensor,
        wb_t_all: torch.Tensor,
        scale,
        *,
        buffer: Optional[torch.Tensor] = None,
    ) -> None:
        """The LoRA of the LM head, always per-token (punica.py:775-793); needs set_sampler_indices."""
        y_org = y
        y = y.view(-1, y.shape[-1])
        x = x.view(-1, x.shape[-1])
        r = wb_t_all.size(-1)
        if buffer is None:
            buffer = torch.zeros((x.size(0), r), dtype=x.dtype, device=x.device)
        ops.bgmv_shrink(x, wa_t_all, buffer, self.sampler_indices, scale)
        ops.bgmv_expand(buffer, wb_t_all, y, self.sampler_indices, add_inputs=True)
        y = y.view_as(y_org)
