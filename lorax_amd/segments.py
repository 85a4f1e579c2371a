"""Run-length segmentation of per-token adapter indices.

Mirror of ``lorax_server/utils/segments.py``: ``find_segments`` (:6-26) turns the
per-token adapter index list into segment boundaries plus one adapter index per
segment, and ``SegmentConcatBuilder`` (:29-55) joins the segmentations of batches that
are concatenated, merging the run that straddles a seam.
"""

from typing import List, Tuple, Union

import numpy as np
import torch


def find_segments(adapter_indices: Union[torch.Tensor, List[int]]) -> Tuple[List[int], List[int]]:
    """Returns (boundaries, adapter index per run): run i covers tokens
    [boundaries[i], boundaries[i+1]). An empty input gives ([0], [])."""
    if isinstance(adapter_indices, torch.Tensor):
        values = adapter_indices.detach().cpu().numpy()  # one device->host copy, no per-item sync
    else:
        values = np.asarray(adapter_indices)
    n = int(values.shape[0])
    if n == 0:
        return [0], []
    change = np.flatnonzero(values[1:] != values[:-1]) + 1
    starts = np.concatenate(([0], change))
    boundaries = np.concatenate((starts, [n]))
    return boundaries.tolist(), values[starts].tolist()


class SegmentConcatBuilder:
    """Accumulates (boundaries tensor, run indices) pairs of consecutive batches."""

    def __init__(self):
        self.adapter_segment_indices: List[int] = []
        self.adapter_segment_tensors: List[torch.Tensor] = []

    def concat(self, adapter_segments: torch.Tensor, segment_indices: List[int]):
        if self.adapter_segment_tensors:
            # later batches drop their leading 0 and are shifted by the tokens seen so far
            shift = self.adapter_segment_tensors[-1][-1]
            adapter_segments = adapter_segments[1:] + shift
        if self.adapter_segment_indices and self.adapter_segment_indices[-1] == segment_indices[0]:
            # same adapter on both sides of the seam: one run, so the previous batch gives
            # up its closing boundary and this batch its first run
            self.adapter_segment_tensors[-1] = self.adapter_segment_tensors[-1][:-1]
            segment_indices = segment_indices[1:]
        self.adapter_segment_tensors.append(adapter_segments)
        self.adapter_segment_indices.extend(segment_indices)

    def build(self) -> Tuple[torch.Tensor, List[int]]:
        return torch.concat(self.adapter_segment_tensors), self.adapter_segment_indices
