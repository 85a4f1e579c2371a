"""Kernel-facing API of the multi-adapter LoRA hot path.

Drop-in for the functions of ``lorax_server/utils/punica.py`` lines 35-255 (constants,
rank padding, weight orientation, the SGMV prefill wrappers, the BGMV decode wrappers,
the scratch-buffer caches and ``segmented_matmul``), with the same names, positional
signatures and error behaviour.  The work is done by hand-written gfx950 HIP kernels
in liblorax_hip.so (see ``_native``); nothing here computes LoRA on the CPU or in
plain PyTorch.

``has_sgmv()`` is true when the shared library loaded and ``DISABLE_SGMV`` is unset
(punica.py:20-27,42-43).  When it is false every kernel wrapper raises.
"""

import os
import warnings
from functools import lru_cache
from typing import List, Optional, Sequence, Tuple

import torch
import torch.nn.functional as F

from lorax_amd import _native

if _native.available():
    _kernels = _native
    HAS_SGMV = not bool(int(os.environ.get("DISABLE_SGMV", "0")))
else:
    warnings.warn(f"Could not load the LoRA HIP kernels: {_native.load_error()}")
    _kernels = None
    HAS_SGMV = False

# The Triton code path of the reference (punica.py:392-793) does not exist here.
LORAX_PUNICA_TRITON_DISABLED = True

MIN_SGMV_RANK = 8
MIN_RANK_CUSTOM = 16
MAX_RANK_CUSTOM = 128
SGMV_BLOCK_SIZE = 16
BGMV_MAX_RANK = 128

_SHRINK_TMP_BYTES = 8 * 1024 * 1024


def has_sgmv() -> bool:
    """punica.py:42-43."""
    return HAS_SGMV


def _native_module():
    if _kernels is None or not HAS_SGMV:
        raise RuntimeError(
            "the LoRA HIP kernels are unavailable (library missing or DISABLE_SGMV set): "
            + str(_native.load_error() or "DISABLE_SGMV=1")
        )
    return _kernels


def pad_to_min_rank(t: torch.Tensor, dim: int, min_rank: int) -> torch.Tensor:
    """Zero-pads dimension `dim` of `t` up to `min_rank`, or, above it, to the next multiple of
    SGMV_BLOCK_SIZE (punica.py:57-76)."""
    rank = t.size(dim)
    if rank <= min_rank:
        target = min_rank
    else:
        target = -(-rank // SGMV_BLOCK_SIZE) * SGMV_BLOCK_SIZE
    if target == rank:
        return t
    # F.pad lists (left, right) pairs starting from the LAST dimension
    spec = [0, 0] * t.dim()
    spec[2 * (t.dim() - 1 - dim) + 1] = target - rank
    return F.pad(t, tuple(spec), mode="constant", value=0.0)


def pad_rank(t: torch.Tensor, dim: int, world_size: int) -> torch.Tensor:
    """punica.py:46-54: a no-op without kernels; the minimum rank grows with the tensor-parallel
    degree because sharding divides the effective rank."""
    if not has_sgmv():
        return t
    return pad_to_min_rank(t, dim, MIN_SGMV_RANK * world_size)


def use_cutlass_shrink(lora_rank: int) -> bool:
    """punica.py:79-80: ranks below 16 keep A as [h_in, r] for the prefill shrink."""
    return lora_rank < MIN_RANK_CUSTOM


def orient_for_rank(t: torch.Tensor, rank: int) -> torch.Tensor:
    """punica.py:83-86: a transposed view for ranks the [r, h_in] shrink kernel handles."""
    return t.transpose(0, 1) if MIN_RANK_CUSTOM <= rank <= MAX_RANK_CUSTOM else t


_tmp_tensors = {}  # device -> the 8 MiB scratch, one per device for the life of the process


def get_tmp_tensor(device: torch.device) -> torch.Tensor:
    """punica.py:145-147 (cached per device: callers that alternate between devices keep both buffers)."""
    device = torch.device(device)
    if device.type == "cuda" and device.index is None:
        device = torch.device("cuda", torch.cuda.current_device())
    tmp = _tmp_tensors.get(device)
    if tmp is None:
        tmp = _tmp_tensors[device] = torch.empty((_SHRINK_TMP_BYTES,), dtype=torch.uint8, device=device)
    return tmp


def get_shrink_scratch(device: torch.device) -> torch.Tensor:
    """Scratch of the resident-layout shrink entries (lora_a_sgmv_resident, lora_a_sgmv_resident_multi): where a
    batch has fewer row tiles than the GPU has CUs, the hidden dimension is cut into parts across workgroups and
    the parts' fp32 sums (parts x rows x summed rank) go here.  It is the reference's 8 MiB buffer: the kernels
    keep their sums inside the first 8 MiB whatever a caller passes, so that the result does not depend on it."""
    return get_tmp_tensor(device)


def get_tmp_expand_size(size: int) -> int:
    """punica.py:156-157."""
    return _native_module().sgmv_cutlass_tmp_size(size)


@lru_cache(maxsize=32)
def get_tmp_tensor_for_size(size: int, device: torch.device) -> torch.Tensor:
    """punica.py:150-153."""
    return torch.empty((get_tmp_expand_size(size),), dtype=torch.uint8, device=device)


def get_tmp_tensors(nsegments: int, lora_rank: int, device: torch.device) -> Tuple[torch.Tensor, torch.Tensor]:
    """(tmp_shrink, tmp_expand) for one rank group, punica.py:160-167."""
    tmp_expand = get_tmp_tensor_for_size(nsegments, device)
    if use_cutlass_shrink(lora_rank):
        return tmp_expand, tmp_expand
    return get_tmp_tensor(device), tmp_expand


def lora_a_sgmv_cutlass(
    x: torch.Tensor,
    tmp: torch.Tensor,
    wa_ptr: torch.Tensor,
    s_start: torch.IntTensor,
    s_end: torch.IntTensor,
    layer_idx: int,
    lora_rank: int,
) -> torch.Tensor:
    """v[s:e] = x[s:e] @ A_i for every segment, zero elsewhere (punica.py:170-184)."""
    k = _native_module()
    v = torch.zeros((x.size(0), lora_rank), dtype=x.dtype, device=x.device)
    if MIN_RANK_CUSTOM <= lora_rank <= MAX_RANK_CUSTOM:
        k.sgmv_shrink(v, x, wa_ptr, s_start, s_end, tmp, layer_idx)
    else:
        k.sgmv_cutlass(v, x, wa_ptr, s_start, s_end, tmp, layer_idx)
    return v


def lora_a_sgmv_resident(
    x: torch.Tensor,
    tmp: torch.Tensor,
    wa_t_ptr: torch.Tensor,
    s_start: torch.IntTensor,
    s_end: torch.IntTensor,
    layer_idx: int,
    lora_rank: int,
    zero_fill: bool = True,
    tiles=None,
) -> torch.Tensor:
    """As lora_a_sgmv_cutlass, reading the [L, r, h_in] stacks of the decode path (weights_a_t) whatever
    the rank.  `tmp` is get_shrink_scratch(device) or the 8 MiB buffer of get_tmp_tensor.
    zero_fill=False skips the zero-fill launch: the kernel overwrites the rows of the segments and the rows
    outside every segment hold garbage - fine for a v that only goes to the expand of the same segments."""
    alloc = torch.zeros if zero_fill else torch.empty
    v = alloc((x.size(0), lora_rank), dtype=x.dtype, device=x.device)
    _native_module().sgmv_shrink_multi([v], x, [wa_t_ptr], s_start, s_end, tmp, layer_idx, 1.0, zero_fill, tiles)
    return v


def lora_a_sgmv_resident_multi(
    x: torch.Tensor,
    tmp: torch.Tensor,
    wa_t_ptrs: Sequence[torch.Tensor],
    s_start: torch.IntTensor,
    s_end: torch.IntTensor,
    layer_idx: int,
    lora_rank: int,
    zero_fill: bool = True,
) -> List[torch.Tensor]:
    """lora_a_sgmv_resident for up to 4 projections that share x, the segments and the rank (q/k/v, gate/up):
    one v per pointer table.  One launch that reads x once when the summed rank is at most 128 and h_in a
    multiple of 128; the reference issues one shrink per projection (layers.py:121-133)."""
    alloc = torch.zeros if zero_fill else torch.empty
    flat = alloc((len(wa_t_ptrs), x.size(0), lora_rank), dtype=x.dtype, device=x.device)
    vs = list(flat.unbind(0))
    _native_module().sgmv_shrink_multi(vs, x, list(wa_t_ptrs), s_start, s_end, tmp, layer_idx, 1.0, zero_fill)
    return vs


def resident_shrink_applies(lora_rank: int, h_in: int, num_tokens: int = 1 << 30) -> bool:
    """Ranks the [L, r, h_in] shrink entry accepts: multiples of 16 always, other multiples of 8 when h_in is
    a multiple of 128 or the batch has at most 512 rows."""
    return 8 <= lora_rank <= MAX_RANK_CUSTOM and lora_rank % 8 == 0 and (
        lora_rank % 16 == 0 or h_in % 128 == 0 or num_tokens <= 512)


def lora_b_sgmv_cutlass(
    y: torch.Tensor,
    v: torch.Tensor,
    tmp: torch.Tensor,
    wb_ptr: torch.Tensor,
    s_start: torch.IntTensor,
    s_end: torch.IntTensor,
    layer_idx: int,
):
    """y[s:e] += v[s:e] @ B_i in place (punica.py:187-196)."""
    _native_module().sgmv_cutlass(y, v, wb_ptr, s_start, s_end, tmp, layer_idx)


def add_lora_sgmv_cutlass(
    y: torch.Tensor,
    x: torch.Tensor,
    wa_ptr: torch.Tensor,
    wb_ptr: torch.Tensor,
    s_start: torch.Tensor,
    s_end: torch.Tensor,
    layer_idx: int,
    lora_rank: int,
):
    """y[s:e] += x[s:e] @ A_i @ B_i with freshly allocated scratch (punica.py:90-142)."""
    k = _native_module()
    nseg = wa_ptr.size(0)
    tmp_expand = torch.empty((k.sgmv_cutlass_tmp_size(nseg),), dtype=torch.uint8, device=x.device)
    if use_cutlass_shrink(lora_rank) or lora_rank > MAX_RANK_CUSTOM:
        tmp_shrink = tmp_expand
    else:
        tmp_shrink = torch.empty((_SHRINK_TMP_BYTES,), dtype=torch.uint8, device=x.device)
    v = lora_a_sgmv_cutlass(x, tmp_shrink, wa_ptr, s_start, s_end, layer_idx, lora_rank)
    lora_b_sgmv_cutlass(y, v, tmp_expand, wb_ptr, s_start, s_end, layer_idx)


def add_lora_a_bgmv(
    v: torch.Tensor,
    x: torch.Tensor,
    wa_T_all: torch.Tensor,
    indicies: torch.LongTensor,
    layer_idx: int,
):
    """v[b] += x[b] @ A[indicies[b]][layer_idx].T for indicies[b] >= 0; A stacks are [L, r, h_in]
    (punica.py:199-227)."""
    _native_module().dispatch_bgmv(v, x, wa_T_all, indicies, layer_idx, 1.0)


def add_lora_b_bgmv(
    y: torch.Tensor,
    v: torch.Tensor,
    wb_T_all: torch.Tensor,
    indicies: torch.LongTensor,
    layer_idx: int,
):
    """y[b] += v[b] @ B[indicies[b]][layer_idx].T for indicies[b] >= 0; B stacks are [L, h_out, r]
    (punica.py:199-217,230-237)."""
    _native_module().dispatch_bgmv(y, v, wb_T_all, indicies, layer_idx, 1.0)


def add_lora_b_bgmv_slice(y, v, wb_T_all, indicies, layer_idx, y_offset: int, y_slice_size: int):
    """As add_lora_b_bgmv, writing columns [y_offset, y_offset + y_slice_size) of a wider y. The reference's
    native side has these parameters but binds them to 0 and h_out (punica_ops.cc:318)."""
    _native_module().bgmv(y, v, wb_T_all, indicies, layer_idx, 1.0, y_offset, y_slice_size)


def lora_b_sgmv_cutlass_slice(y, v, tmp, wb_ptr, s_start, s_end, layer_idx, y_offset: int, y_slice_size: int,
                              transposed: bool = False, tiles=None):
    """As lora_b_sgmv_cutlass, writing columns [y_offset, y_offset + y_slice_size) of a wider y.  With
    `transposed`, wb_ptr addresses the [L, h_out, r] stacks of the decode path (weights_b_t) - same result,
    faster kernel; `tiles` is then an optional row-tile plan of the segment tables (same result again)."""
    _native_module().sgmv_expand(y, v, wb_ptr, s_start, s_end, tmp, layer_idx, y_offset, y_slice_size, transposed,
                                 True, tiles)


def segmented_matmul(
    y: torch.Tensor,
    x: torch.Tensor,
    w: List[torch.Tensor],
    b: List[Optional[torch.Tensor]],
    s_start: torch.IntTensor,
    s_end: torch.IntTensor,
):
    """y[s:e] = linear(x[s:e], w_i, b_i) per non-empty segment (punica.py:240-255). Dense torch ops on
    whatever device the tensors live on; used by the reference's Medusa heads, not by LoRA."""
    starts, ends = s_start.tolist(), s_end.tolist()
    for wi, bi, s, e in zip(w, b, starts, ends):
        if e > s:
            y[s:e] = F.linear(x[s:e], wi, bi)


# The stacked-weight front end of the reference lives in the same module there (punica.py:256-793).
from lorax_amd.punica_wrapper import PunicaWrapper, compute_meta  # noqa: E402,F401
