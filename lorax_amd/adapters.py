"""Adapter-side inputs of the LoRA kernels: per-adapter weight stacks and the per-batch
routing tables (pointer tables, segment bounds, per-token indices) derived from them.

Mirrors, for the LoRA hot path only,
  * ``lorax_server/adapters/weights.py``: ``AdapterBatchMetadata`` (:15-32),
    ``LayerAdapterWeights`` (:66-105), ``AdapterBatchData`` (:108-171);
  * ``lorax_server/adapters/lora.py``: ``LoraWeights`` (:87-140), ``RankSegments``
    (:213-227), ``BatchLoraWeights`` (:230-396), ``get_scaling_factor`` (:399-407).
Attribute and method names are the reference's, so its LoRA layer code and its tests
(server/tests/utils/test_lora.py) read the same against either package.
"""

from abc import ABC, abstractmethod
from collections import defaultdict
from collections.abc import Mapping
from dataclasses import dataclass
from typing import Dict, List, Optional, Set, Tuple, Type

import torch

from lorax_amd.sgmv import (
    BGMV_MAX_RANK,
    MAX_RANK_CUSTOM,
    MIN_RANK_CUSTOM,
    get_tmp_tensors,
    orient_for_rank,
    pad_rank,
    use_cutlass_shrink,
)

LORA = "lora"
LM_HEAD = "lm_head"

# Stands in for "this segment's adapter has no weights for the layer": its address is what
# the pointer tables hold for such segments (adapters/lora.py:26,283). It is never read.
EMPTY_TENSOR = torch.tensor([])


@dataclass
class AdapterBatchMetadata:
    """adapters/weights.py:15-32."""

    adapter_indices: torch.Tensor  # [num_tokens] adapter index of every token
    adapter_list: List[int]  # [batch_size] adapter index of every request
    adapter_set: Set[int]  # distinct adapter indices in the batch
    adapter_segments: torch.Tensor  # [num_segments + 1] token offsets of the runs
    segment_indices: List[int]  # [num_segments] adapter index of every run


class AdapterWeights(ABC):
    @classmethod
    @abstractmethod
    def get_batch_types(cls) -> List[Type["BatchAdapterWeights"]]:
        ...

    @property
    def speculative_tokens(self) -> int:
        return 0


class BatchAdapterWeights(ABC):
    @abstractmethod
    def has_adapter(self, adapter_index: int) -> bool:
        ...

    @classmethod
    @abstractmethod
    def key(cls) -> str:
        ...

    @classmethod
    @abstractmethod
    def load(cls, adapter_weights, meta, layer_name, prefill, prefill_head_indices):
        ...


@dataclass
class LoraConfig:
    """The fields of adapters/lora.py:29-35 that the hot path reads."""

    r: int
    lora_alpha: int = 1
    target_modules: Optional[List[str]] = None
    fan_in_fan_out: bool = False
    use_rslora: bool = False
    base_model_name_or_path: str = ""


def get_scaling_factor(lora_alpha: int, r: int, uses_rslora: bool = False) -> float:
    """adapters/lora.py:399-407."""
    return lora_alpha / (r**0.5) if uses_rslora else lora_alpha / r


class LoraWeights(AdapterWeights):
    """One adapter's A and B for one layer type, stacked over layers (adapters/lora.py:87-140).

    Constructed from per-layer ``A: [h_in, r]`` and ``B: [r, h_out]``.  ONE resident layout serves
    both kernels families here:
      weights_a_t = [L, r, h_in]   read by BGMV shrink and by SGMV shrink (any rank multiple of 8)
      weights_b_t = [L, h_out, r]  read by BGMV expand and by SGMV expand
    The reference keeps one of two layouts at a time - prefill: weights_a = [L, r, h_in] for
    16 <= r <= 128 else [L, h_in, r], weights_b = [L, r, h_out]; decode: the two above - and
    re-transposes the whole stack whenever a batch of the other kind arrives (adapters/lora.py:111-140),
    which also moves the stack to a new address.  weights_a / weights_b are still available for
    callers of the reference-layout entry points; they are materialised on first use and then stay
    resident too, so every pointer handed to the kernels stays valid for the adapter's lifetime.
    """

    def __init__(self, weights_a: List[torch.Tensor], weights_b: List[torch.Tensor], adapter_config: LoraConfig):
        has_layers = len(weights_a) > 0
        self.lora_a_r = weights_a[0].size(1) if has_layers else 1
        self.lora_b_r = weights_b[0].size(0) if has_layers else 1
        self._use_cutlass_shrink = use_cutlass_shrink(self.lora_a_r)
        self._weights_a_t = torch.stack([w.transpose(0, 1).contiguous() for w in weights_a])  # [L, r, h_in]
        self._weights_b_t = torch.stack([w.transpose(0, 1).contiguous() for w in weights_b])  # [L, h_out, r]
        self._weights_a: Optional[torch.Tensor] = None
        self._weights_b: Optional[torch.Tensor] = None
        self._rank_chunks = None
        self.adapter_config = adapter_config

    @property
    def weights_a(self) -> torch.Tensor:
        """The reference's prefill layout of A (orient_for_rank, punica.py:83-86)."""
        if self._weights_a is None:
            # the layouts agree about A for the ranks of the reference's custom shrink (16 to 128) only
            a = self._weights_a_t
            same = MIN_RANK_CUSTOM <= self.lora_a_r <= MAX_RANK_CUSTOM
            self._weights_a = a if same else a.transpose(1, 2).contiguous()
        return self._weights_a

    @property
    def weights_b(self) -> torch.Tensor:
        """The reference's prefill layout of B, [L, r, h_out]."""
        if self._weights_b is None:
            self._weights_b = self._weights_b_t.transpose(1, 2).contiguous()
        return self._weights_b

    @property
    def weights_a_t(self) -> torch.Tensor:
        return self._weights_a_t

    def rank_chunks(self) -> List[Tuple[torch.Tensor, torch.Tensor, int]]:
        """An adapter of a rank above what the kernels take (MAX_RANK_CUSTOM) as several adapters of kernel rank:
        (x A^T) B = sum over chunks c of (x A_c^T) B_c with A_c the rows and B_c the columns [c * 128, ...) of the
        stacks.  Returns [(A_c [L, r_c, h_in], B_c^T [L, h_out, r_c], r_c)], contiguous copies made on first use.
        (The reference runs such adapters through its dense per-adapter loop, utils/layers.py:169-190.)"""
        if self._rank_chunks is None:
            step = MAX_RANK_CUSTOM
            self._rank_chunks = [
                (self._weights_a_t[:, c : c + step, :].contiguous(), self._weights_b_t[:, :, c : c + step].contiguous(),
                 min(step, self.lora_a_r - c))
                for c in range(0, self.lora_a_r, step)
            ]
        return self._rank_chunks

    @property
    def weights_b_t(self) -> torch.Tensor:
        return self._weights_b_t

    @classmethod
    def get_batch_types(cls) -> List[Type[BatchAdapterWeights]]:
        return [BatchLoraWeights]

    @classmethod
    def from_peft(
        cls,
        lora_A: List[torch.Tensor],
        lora_B: List[torch.Tensor],
        config: LoraConfig,
        world_size: int = 1,
    ) -> "LoraWeights":
        """Per-layer PEFT tensors (lora_A.weight [r, h_in], lora_B.weight [h_out, r]) to a stack:
        transpose, fold alpha/r into B, pad the rank (adapters/lora.py:184-210)."""
        scale = get_scaling_factor(config.lora_alpha, config.r, config.use_rslora)
        a_list = [pad_rank(a.transpose(0, 1), dim=1, world_size=world_size) for a in lora_A]
        b_list = [pad_rank(b.transpose(0, 1) * scale, dim=0, world_size=world_size) for b in lora_B]
        if a_list:
            config.r = a_list[0].size(1)
        return cls(a_list, b_list, config)


class RankSegments:
    """Kernel arguments of one rank group (adapters/lora.py:213-227).

    lora_a_ptr / lora_b_ptr are the reference's tables: in decode the addresses of the [L, r, h_in] and
    [L, h_out, r] stacks, in prefill those of the reference's prefill layouts.  The prefill kernels here read
    the decode stacks too (lora_a_t_ptr / lora_b_t_ptr), so the reference-layout tables of a prefill batch -
    and the weight copies behind them - are only built when somebody asks for them."""

    def __init__(self, rank: int, lora_a_ptr, lora_b_ptr, tmp_shrink: Optional[torch.Tensor],
                 tmp_expand: Optional[torch.Tensor], segment_starts: Optional[torch.Tensor],
                 segment_ends: Optional[torch.Tensor], indices: Optional[torch.Tensor],
                 plan: Optional[torch.Tensor] = None, lora_a_t_ptr: Optional[torch.Tensor] = None,
                 lora_b_t_ptr: Optional[torch.Tensor] = None, segments_key=None,
                 num_long_segments: Optional[int] = None, short_plan: Optional[torch.Tensor] = None,
                 shrink_tiles=None, expand_tiles=None):
        self.rank = rank
        self._lora_a_ptr = lora_a_ptr  # a tensor, or a function that builds it
        self._lora_b_ptr = lora_b_ptr
        # prefill (SGMV)
        self.tmp_shrink = tmp_shrink
        self.tmp_expand = tmp_expand
        self.segment_starts = segment_starts
        self.segment_ends = segment_ends
        # decode (BGMV)
        self.indices = indices
        # decode: routing plan for the batched BGMV launches, int64 [num_chunks, 8] on the device; one record
        # per chunk of up to BGMV_PLAN_GROUP tokens of one adapter: [count, tok0..tok3, address of the A stack,
        # address of the B^T stack, 0]. Derived from `indices` and the pointer tables; no counterpart in the
        # reference, whose kernels take one token per thread block.
        self.plan = plan
        # prefill: addresses of the resident stacks, one per segment like lora_a_ptr / lora_b_ptr
        self.lora_a_t_ptr = lora_a_t_ptr
        self.lora_b_t_ptr = lora_b_t_ptr
        # prefill: hashable and equal for rank groups (of different layer types) whose segment_starts /
        # segment_ends hold the same values - their shrinks can share one pass over x; None = unknown
        self.segments_key = segments_key
        # prefill: a batch with many segments of a few rows (decode tokens inside a prefill batch) lists them
        # last in its tables and, besides, as a routing plan over their rows (records as in `plan`).  A caller
        # may then run the segment kernels over the first num_long_segments entries only and the per-token
        # kernels over short_plan; the tables as a whole stay complete.  None / the table's length: no such plan.
        self.short_plan = short_plan
        self.num_long_segments = num_long_segments
        # prefill: row-tile plans (_native.TilePlan) of the first num_long_segments segments for the shrink and
        # the expand kernels, cut on the host from the segment lengths; None = the kernels search their tiles on
        # the device
        self.shrink_tiles = shrink_tiles
        self.expand_tiles = expand_tiles

    @property
    def lora_a_ptr(self) -> Optional[torch.Tensor]:
        if callable(self._lora_a_ptr):
            self._lora_a_ptr = self._lora_a_ptr()
        return self._lora_a_ptr

    @property
    def lora_b_ptr(self) -> Optional[torch.Tensor]:
        if callable(self._lora_b_ptr):
            self._lora_b_ptr = self._lora_b_ptr()
        return self._lora_b_ptr


BGMV_PLAN_GROUP = 4
BGMV_PLAN_WORDS = 8


def build_bgmv_plan(token_slots: List[int], a_addrs: List[int], b_addrs: List[int]) -> List[List[int]]:
    """Cuts the tokens of every adapter slot, in token order, into chunks of at most BGMV_PLAN_GROUP and
    returns one plan record per chunk. token_slots[t] is the token's index into the rank group's pointer
    slice (-1 = not in the group); a_addrs / b_addrs are the addresses in that slice."""
    by_slot: Dict[int, List[int]] = {}
    for t, s in enumerate(token_slots):
        if s >= 0:
            by_slot.setdefault(s, []).append(t)
    records = []
    for s, toks in by_slot.items():
        for i in range(0, len(toks), BGMV_PLAN_GROUP):
            chunk = toks[i : i + BGMV_PLAN_GROUP]
            pad = [chunk[0]] * (BGMV_PLAN_GROUP - len(chunk))
            records.append([len(chunk), *chunk, *pad, a_addrs[s], b_addrs[s], 0])
    return records


SHORT_SEGMENT_ROWS = 4    # segments of at most this many rows may go to the per-token kernels ...
MIN_SHORT_SEGMENTS = 32   # ... when a rank group has at least this many of them


def build_short_plan(segs: List[int], bounds: List[int], a_addrs: List[int], b_addrs: List[int],
                     owners: List[int]) -> List[List[int]]:
    """Plan records over the rows of the segments `segs` (each of at most SHORT_SEGMENT_ROWS rows; the segments
    of one owner next to each other): the rows of one owner, in the order given, in chunks of BGMV_PLAN_GROUP.
    a_addrs / b_addrs / owners are indexed by segment."""
    records = []
    i = 0
    while i < len(segs):
        j, rows = i, []
        while j < len(segs) and owners[segs[j]] == owners[segs[i]]:
            rows += list(range(bounds[segs[j]], bounds[segs[j] + 1]))
            j += 1
        for k in range(0, len(rows), BGMV_PLAN_GROUP):
            chunk = rows[k : k + BGMV_PLAN_GROUP]
            pad = [chunk[0]] * (BGMV_PLAN_GROUP - len(chunk))
            records.append([len(chunk), *chunk, *pad, a_addrs[segs[i]], b_addrs[segs[i]], 0])
        i = j
    return records


def pad_bgmv_plan(plan: torch.Tensor, num_records: int) -> torch.Tensor:
    """`plan` extended with all-zero records to a fixed number of records: the kernels skip them, so a decode
    step captured in a graph can be replayed with the plans of later batches copied into the same tensor
    (the reference pads pointer tables with 0 and indices with -1 for the same purpose, utils/graph.py:71-73)."""
    if plan.size(0) > num_records:
        raise ValueError(f"plan has {plan.size(0)} records, more than the fixed size {num_records}")
    padded = torch.zeros((num_records, BGMV_PLAN_WORDS), dtype=plan.dtype, device=plan.device)
    padded[: plan.size(0)] = plan
    return padded


def _count_short(segs: List[int], bounds: List[int]) -> int:
    return sum(1 for s in segs if bounds[s + 1] - bounds[s] <= SHORT_SEGMENT_ROWS)


def _segment_order(segs: List[int], seg_adapters: List[int], bounds: List[int], split: bool = False):
    """Sort key of a rank group's segments: rows of the segment's adapter inside the group, descending, then the
    adapter index; with `split`, the segments of more than SHORT_SEGMENT_ROWS rows before the others."""
    rows: Dict[int, int] = defaultdict(int)
    for s in segs:
        rows[seg_adapters[s]] += bounds[s + 1] - bounds[s]
    return lambda s: (split and bounds[s + 1] - bounds[s] <= SHORT_SEGMENT_ROWS, -rows[seg_adapters[s]],
                      seg_adapters[s])


def _tile_plans(starts: List[int], ends: List[int], num_long: int, device, rank: int = 0):
    """Row-tile plans (shrink, expand) of the first num_long segments, cut by the library's host routine and
    uploaded; (None, None) where the library is not loaded or the tables live on the CPU."""
    from lorax_amd import _native

    if not _native.available() or torch.device(device).type != "cuda":
        return None, None
    rows = max(ends[:num_long], default=0)
    plans = []
    for kind in (_native.TILES_SHRINK, _native.TILES_EXPAND):
        records, tile_rows = _native.plan_tiles(starts[:num_long], ends[:num_long], rows, kind, rank)
        plans.append(_native.TilePlan(torch.from_numpy(records.copy()).to(device), tile_rows))
    return plans[0], plans[1]


class _LayoutView(Mapping):
    """adapter index -> one layout of its stack (an attribute of LoraWeights), fetched on access."""

    def __init__(self, loras: Dict[int, "LoraWeights"], layout: str):
        self._loras = loras
        self._layout = layout

    def __getitem__(self, idx: int) -> torch.Tensor:
        return getattr(self._loras[idx], self._layout)

    def __iter__(self):
        return iter(self._loras)

    def __len__(self) -> int:
        return len(self._loras)


def _unwrap(weights):
    return weights.lora_weights if hasattr(weights, "lora_weights") else weights


@dataclass
class BatchLoraWeights(BatchAdapterWeights):
    """adapters/lora.py:230-396."""

    lora_a: Mapping  # adapter index -> A stack in the reference's prefill layout (built on access)
    lora_b: Mapping  # adapter index -> B stack [L, r, h_out] (built on access)
    adapter_index_configs: Dict[int, LoraConfig]
    rank_data: Dict[object, RankSegments]  # rank -> group; (rank, chunk) -> group for ranks above 128
    use_sgmv: bool
    layer_name: str
    prefill_head_indices: Optional[torch.Tensor]

    def has_adapter(self, adapter_index: int) -> bool:
        return adapter_index in self.adapter_index_configs

    def can_vectorize(self, pg) -> bool:
        """True when the kernels serve every rank group.  The reference also returns False for the LM head
        (adapters/lora.py:243-247: its BGMV kernels stop at 65 535 output columns) and runs its dense loop
        there; the kernels here take vocabulary-wide outputs, so the LM head is served like any projection."""
        return all(rd.rank // pg.size() <= MAX_RANK_CUSTOM for rd in self.rank_data.values())

    @classmethod
    def key(cls) -> str:
        return LORA

    @classmethod
    def load(
        cls,
        adapter_weights: Dict[int, AdapterWeights],
        meta: AdapterBatchMetadata,
        layer_name: str,
        prefill: bool,
        prefill_head_indices: Optional[torch.Tensor],
    ) -> Optional["BatchLoraWeights"]:
        loras: Dict[int, LoraWeights] = {}
        for idx, w in adapter_weights.items():
            w = _unwrap(w)
            if isinstance(w, LoraWeights):
                loras[idx] = w
        if not loras:
            return None

        seg_adapters = list(meta.segment_indices)
        covered = [s for s, idx in enumerate(seg_adapters) if idx in loras]
        if not covered:
            return None
        device = next(iter(loras.values())).weights_a_t.device

        # adapter -> stack in the reference's prefill layout, read (and materialised) on access only
        lora_a = _LayoutView({seg_adapters[s]: loras[seg_adapters[s]] for s in covered}, "weights_a")
        lora_b = _LayoutView({seg_adapters[s]: loras[seg_adapters[s]] for s in covered}, "weights_b")
        # ranks above the kernels' limit are served as chunks of kernel rank, so decode stays on the BGMV tables
        max_rank = min(max(loras[seg_adapters[s]].lora_a_r for s in covered), MAX_RANK_CUSTOM)
        use_sgmv = bool(prefill or max_rank > BGMV_MAX_RANK)

        # One pointer per segment; segments without weights hold a placeholder address that no
        # rank group refers to.
        null = EMPTY_TENSOR.data_ptr()

        def table(layout: str) -> torch.Tensor:
            addr = [getattr(loras[i], layout).data_ptr() if i in loras else null for i in seg_adapters]
            return torch.tensor(addr, dtype=torch.int64, device=device)

        a_addr = [loras[i].weights_a_t.data_ptr() if i in loras else null for i in seg_adapters]
        b_addr = [loras[i].weights_b_t.data_ptr() if i in loras else null for i in seg_adapters]
        lora_a_t_ptr = torch.tensor(a_addr, dtype=torch.int64, device=device)
        lora_b_t_ptr = torch.tensor(b_addr, dtype=torch.int64, device=device)

        configs = {seg_adapters[s]: loras[seg_adapters[s]].adapter_config for s in covered}

        # A rank group is keyed by its rank, as in the reference; chunk c of the adapters of a rank above 128 forms a
        # group of its own under the key (rank, c), with the chunk's rank and the chunk stacks' addresses.
        by_rank: Dict[object, List[int]] = defaultdict(list)
        for s in covered:
            w = loras[seg_adapters[s]]
            if w.lora_a_r <= MAX_RANK_CUSTOM:
                by_rank[w.lora_a_r].append(s)
            else:
                for c in range(len(w.rank_chunks())):
                    by_rank[(w.lora_a_r, c)].append(s)

        head_starts = head_ends = None
        if prefill_head_indices is not None:
            # LM-head inputs keep one row per request; recount segment bounds in those rows
            head_starts, head_ends = [0], [0]
            bounds = meta.adapter_segments.tolist()
            j = 1
            for head_index in prefill_head_indices.tolist():
                if head_index < bounds[j]:
                    head_ends[-1] += 1
                else:
                    head_starts.append(head_ends[-1])
                    head_ends.append(head_ends[-1] + 1)
                    j += 1

        token_adapters = None if use_sgmv else meta.adapter_indices.tolist()
        rank_data: Dict[object, RankSegments] = {}
        for group_key, segs in by_rank.items():
            chunk = group_key[1] if isinstance(group_key, tuple) else None
            if chunk is None:
                rank = group_key
                group_a, group_b = a_addr, b_addr
            else:  # addresses and rank of chunk `chunk` of every adapter of the group
                rank = loras[seg_adapters[segs[0]]].rank_chunks()[chunk][2]
                group_a, group_b = list(a_addr), list(b_addr)
                for s in segs:
                    a_c, b_c, _ = loras[seg_adapters[s]].rank_chunks()[chunk]
                    group_a[s], group_b[s] = a_c.data_ptr(), b_c.data_ptr()
            group_a_ptr = lora_a_t_ptr if chunk is None else torch.tensor(group_a, dtype=torch.int64, device=device)
            group_b_ptr = lora_b_t_ptr if chunk is None else torch.tensor(group_b, dtype=torch.int64, device=device)
            num_long = short_plan = None
            if use_sgmv:
                # the order of a group's segments is free: keep the segments of one adapter together, so that
                # their tiles run back to back and share the adapter's weights in L2, adapters with the most
                # rows first (the long tiles of a launch start early); many segments of a few rows go last and
                # get a routing plan for the per-token kernels
                seg_bounds = meta.adapter_segments.tolist()
                n_short = _count_short(segs, seg_bounds) if head_starts is None else 0
                split = n_short >= MIN_SHORT_SEGMENTS
                segs.sort(key=_segment_order(segs, seg_adapters, seg_bounds, split))
                if split:
                    num_long = len(segs) - n_short
                    records = build_short_plan(segs[num_long:], seg_bounds, group_a, group_b, seg_adapters)
                    short_plan = torch.tensor(records, dtype=torch.int64, device=device).reshape(-1, BGMV_PLAN_WORDS)
            tmp_shrink = tmp_expand = starts = ends = token_slots = plan = shrink_tiles = expand_tiles = None
            if use_sgmv:
                tmp_shrink, tmp_expand = get_tmp_tensors(len(segs), rank, device)
                starts = meta.adapter_segments[segs]
                ends = meta.adapter_segments[[s + 1 for s in segs]]
                if head_starts is not None:
                    for i, s in enumerate(segs):
                        starts[i] = head_starts[s]
                        ends[i] = head_ends[s]
                shrink_tiles, expand_tiles = _tile_plans(
                    [head_starts[s] if head_starts is not None else seg_bounds[s] for s in segs],
                    [head_ends[s] if head_starts is not None else seg_bounds[s + 1] for s in segs],
                    num_long if num_long is not None else len(segs), device, rank)
            else:
                # slot of an adapter = position of its first segment inside this group's pointer slice
                slot: Dict[int, int] = {}
                for pos, s in enumerate(segs):
                    slot.setdefault(seg_adapters[s], pos)
                in_group = {seg_adapters[s] for s in segs}
                slots = [slot.get(a, -1) if a in in_group else -1 for a in token_adapters]
                token_slots = torch.tensor(slots, dtype=torch.int64, device=device)
                records = build_bgmv_plan(slots, [group_a[s] for s in segs], [group_b[s] for s in segs])
                plan = torch.tensor(records, dtype=torch.int64, device=device).reshape(-1, BGMV_PLAN_WORDS)
            if use_sgmv and chunk is None:
                # the reference's prefill tables, built (with the weight copies behind them) on first access
                ref_a = (lambda segs=segs: table("weights_a")[segs])
                ref_b = (lambda segs=segs: table("weights_b")[segs])
            elif use_sgmv:
                ref_a = ref_b = None  # rank chunks exist in the resident layouts only
            else:
                ref_a, ref_b = group_a_ptr[segs], group_b_ptr[segs]
            rank_data[group_key] = RankSegments(
                rank=rank,
                lora_a_ptr=ref_a,
                lora_b_ptr=ref_b,
                tmp_shrink=tmp_shrink,
                tmp_expand=tmp_expand,
                segment_starts=starts,
                segment_ends=ends,
                indices=token_slots,
                plan=plan,
                lora_a_t_ptr=group_a_ptr[segs] if use_sgmv else None,
                lora_b_t_ptr=group_b_ptr[segs] if use_sgmv else None,
                segments_key=(tuple(segs), head_starts is not None, chunk) if use_sgmv else None,
                num_long_segments=num_long if num_long is not None else (len(segs) if use_sgmv else None),
                short_plan=short_plan,
                shrink_tiles=shrink_tiles,
                expand_tiles=expand_tiles,
            )

        return cls(
            lora_a=lora_a,
            lora_b=lora_b,
            adapter_index_configs=configs,
            rank_data=rank_data,
            use_sgmv=use_sgmv,
            layer_name=layer_name,
            prefill_head_indices=prefill_head_indices,
        )


class LayerAdapterWeights:
    """All adapters loaded for one layer type (adapters/weights.py:66-105)."""

    def __init__(self):
        self.adapter_weights: Dict[int, AdapterWeights] = {}
        self._lora_entries = None  # cached argument of the native table builder
        self._unwrapped = None

    def add_adapter(self, adapter_idx: int, weights: AdapterWeights):
        self.adapter_weights[adapter_idx] = weights
        self._lora_entries = None
        self._unwrapped = None

    def remove_adapter(self, adapter_idx: int):
        self.adapter_weights.pop(adapter_idx, None)
        self._lora_entries = None
        self._unwrapped = None

    def unwrapped(self) -> Dict[int, "AdapterWeights"]:
        """adapter index -> the adapter's weights without their wrapper; rebuilt only when adapters come or go."""
        if self._unwrapped is None:
            self._unwrapped = {idx: _unwrap(w) for idx, w in self.adapter_weights.items()}
        return self._unwrapped

    def lora_entries(self):
        """(adapter, address of the [L, r, h_in] stack, address of the [L, h_out, r] stack, rank) of every LoRA
        adapter of the layer type, sorted by adapter, as a numpy array of _native.ENTRY_DTYPE; None if an adapter
        of another kind, or of a rank above the kernels' 128, is loaded.  Rebuilt only when adapters come or go."""
        if self._lora_entries is None:
            import numpy as np

            from lorax_amd import _native

            rows = []
            for idx in sorted(self.adapter_weights):
                w = _unwrap(self.adapter_weights[idx])
                if not isinstance(w, LoraWeights) or w.get_batch_types() != [BatchLoraWeights]:
                    return None
                if w.lora_a_r > MAX_RANK_CUSTOM:
                    return None  # served in rank chunks, which the per-layer-type Python path builds
                rows.append((idx, w.weights_a_t.data_ptr(), w.weights_b_t.data_ptr(), w.lora_a_r, 0))
            self._lora_entries = np.array(rows, dtype=_native.ENTRY_DTYPE)
        return self._lora_entries

    @property
    def max_speculative_tokens(self) -> int:
        return max(w.speculative_tokens for w in self.adapter_weights.values())

    def is_empty(self) -> bool:
        return not self.adapter_weights

    def get_data(
        self,
        meta: AdapterBatchMetadata,
        layer_name: str,
        prefill: bool,
        prefill_head_indices: Optional[torch.Tensor],
    ) -> Dict[str, BatchAdapterWeights]:
        per_type: Dict[Type[BatchAdapterWeights], Dict[int, AdapterWeights]] = defaultdict(dict)
        for idx, w in self.adapter_weights.items():
            for batch_type in w.get_batch_types():
                per_type[batch_type][idx] = w
        out = {}
        for batch_type, group in per_type.items():
            batched = batch_type.load(group, meta, layer_name, prefill, prefill_head_indices)
            if batched is not None:
                out[batch_type.key()] = batched
        return out


@dataclass
class AdapterBatchData:
    """adapters/weights.py:108-171. ``punica_wrapper`` (lorax_amd.punica_wrapper.PunicaWrapper) and
    ``layer_to_lora_weights`` (stack_preloaded_adapters) select the stacked-weight path of
    LoraLinear.forward_layer_type, as in the reference; both are optional."""

    meta: AdapterBatchMetadata
    data: Dict[str, Dict[str, BatchAdapterWeights]]  # layer type -> adapter type -> batch data
    layer_to_lora_weights: Dict[Tuple[str, int], Tuple[torch.Tensor, torch.Tensor]]
    punica_wrapper: Optional[object]
    prefill: bool

    @staticmethod
    def from_meta(
        meta: AdapterBatchMetadata,
        weights: Dict[str, LayerAdapterWeights],
        layer_to_lora_weights: Optional[Dict] = None,
        punica_wrapper: Optional[object] = None,
        prefill: bool = False,
        prefill_head_indices: Optional[torch.Tensor] = None,
    ) -> "AdapterBatchData":
        # The native builder makes the tables of all layer types in one call; the LM head of a prefill batch,
        # whose input rows are requests rather than tokens, keeps the per-layer-type Python path.
        head_rows = prefill_head_indices is not None
        native_names = {n: w for n, w in weights.items() if not (head_rows and n == LM_HEAD)}
        data = _native_batch_tables(meta, native_names, prefill)
        remaining = weights if data is None else {n: w for n, w in weights.items() if n not in native_names}
        data = {} if data is None else data
        for layer_name, layer_weights in remaining.items():
            if layer_weights.is_empty():
                continue
            head = prefill_head_indices if layer_name == LM_HEAD else None
            batched = layer_weights.get_data(meta, layer_name, prefill, head)
            if batched:
                data[layer_name] = batched
        return AdapterBatchData(
            meta=meta,
            data=data,
            layer_to_lora_weights=layer_to_lora_weights or {},
            punica_wrapper=punica_wrapper,
            prefill=prefill,
        )

    def ranks(self) -> Set[int]:
        found = set()
        for layer_data in self.data.values():
            lora = layer_data.get(LORA)
            if lora is not None:
                found.update(rd.rank for rd in lora.rank_data.values())
        return found

    def layer_names(self) -> Set[str]:
        return set(self.data.keys())

    def adapter_keys(self) -> Set[str]:
        keys = set()
        for layer_data in self.data.values():
            keys.update(layer_data.keys())
        return keys

    @property
    def max_rank(self) -> int:
        return max(self.ranks(), default=0)


def stack_preloaded_adapters(
    layer_to_adapter_weights: Dict[str, LayerAdapterWeights],
    adapter_indices: List[int],
    device=None,
) -> Dict[Tuple[str, int], Tuple[torch.Tensor, torch.Tensor]]:
    """(layer type, layer) -> (lora_a_weights [num_adapters, r, h_in], lora_b_weights [num_adapters, h_out, r]) over
    the given adapters in order, every adapter zero-padded to the largest rank of the stack (models/model.py:289-334).
    Entry i of a stack belongs to adapter_indices[i]; PunicaWrapper.update_metadata maps adapter index k to entry
    k - 1, so the caller numbers its preloaded adapters 1..n as the reference does."""
    from lorax_amd.sgmv import pad_to_min_rank

    out: Dict[Tuple[str, int], Tuple[torch.Tensor, torch.Tensor]] = {}
    for layer_name, layer_adapter_weights in layer_to_adapter_weights.items():
        per_layer_a: Dict[int, List[torch.Tensor]] = defaultdict(list)
        per_layer_b: Dict[int, List[torch.Tensor]] = defaultdict(list)
        for adapter_index in adapter_indices:
            weights = _unwrap(layer_adapter_weights.adapter_weights.get(adapter_index))
            if not isinstance(weights, LoraWeights):
                continue
            lora_a, lora_b = weights.weights_a_t, weights.weights_b_t  # [L, r, h_in], [L, h_out, r]
            for layer_id in range(lora_a.size(0)):
                per_layer_a[layer_id].append(lora_a[layer_id])
                per_layer_b[layer_id].append(lora_b[layer_id])
        for layer_id, a_list in per_layer_a.items():
            b_list = per_layer_b[layer_id]
            r = max(w.size(-1) for w in b_list)
            a_list = [pad_to_min_rank(w, 0, r) for w in a_list]
            b_list = [pad_to_min_rank(w, 1, r) for w in b_list]
            lora_a = torch.stack(a_list).contiguous()
            lora_b = torch.stack(b_list).contiguous()
            if device is not None:
                lora_a, lora_b = lora_a.to(device), lora_b.to(device)
            out[(layer_name, layer_id)] = (lora_a, lora_b)
    return out


def _native_batch_tables(meta: AdapterBatchMetadata, weights: Dict[str, LayerAdapterWeights],
                         prefill: bool) -> Optional[Dict[str, Dict[str, BatchAdapterWeights]]]:
    """The tables of BatchLoraWeights.load for every layer type from one call of the native builder and one
    host-to-device copy.  None (the caller then takes the per-layer-type Python path) when the library is not
    loaded or a layer type holds adapters that are not plain LoRA."""
    from lorax_amd import _native

    if not _native.available():
        return None
    import numpy as np

    names = [n for n, lw in weights.items() if not lw.is_empty()]
    tables = [weights[n].lora_entries() for n in names]
    if not names or any(t is None for t in tables):
        return None
    device = meta.adapter_indices.device
    indices = meta.adapter_indices.detach().cpu().numpy()
    bounds, owners, packed, groups = _native.build_batch_tables(
        indices, np.concatenate(tables), np.array([len(t) for t in tables], dtype=np.int32), prefill
    )
    dev = torch.from_numpy(packed).to(device)
    dev64, dev32 = dev.view(torch.int64), dev.view(torch.int32)
    seg_adapters = owners.tolist()
    batch_adapters = set(seg_adapters)
    T = int(indices.shape[0])

    by_type: Dict[int, List] = defaultdict(list)
    for g in groups:
        by_type[g.layer_type].append(g)
    data: Dict[str, Dict[str, BatchAdapterWeights]] = {}
    for lt, type_groups in by_type.items():
        layer_name = names[lt]
        layer = weights[layer_name]
        every = layer.unwrapped()
        loras = {a: every[a] for a in batch_adapters if a in every}
        use_sgmv = bool(type_groups[0].use_sgmv)
        null = EMPTY_TENSOR.data_ptr()

        def table(layout: str, loras=loras) -> torch.Tensor:
            addr = [getattr(loras[i], layout).data_ptr() if i in loras else null for i in seg_adapters]
            return torch.tensor(addr, dtype=torch.int64, device=device)

        rank_data: Dict[int, RankSegments] = {}
        for g in type_groups:
            n = g.num_segments
            a_ptr = dev64[g.a_ptr_off // 8 : g.a_ptr_off // 8 + n]
            b_ptr = dev64[g.b_ptr_off // 8 : g.b_ptr_off // 8 + n]
            if use_sgmv:
                tmp_shrink, tmp_expand = get_tmp_tensors(n, g.rank, device)

                def ref_table(layout: str, rank=g.rank, loras=loras, table=table) -> torch.Tensor:
                    # the group's segments in the builder's order (only computed if somebody asks for the
                    # reference-layout tables)
                    segs = [s for s, a in enumerate(seg_adapters) if a in loras and loras[a].lora_a_r == rank]
                    seg_bounds = bounds.tolist()
                    split = _count_short(segs, seg_bounds) >= MIN_SHORT_SEGMENTS
                    segs.sort(key=_segment_order(segs, seg_adapters, seg_bounds, split))
                    return table(layout)[segs]

                rank_data[g.rank] = RankSegments(
                    rank=g.rank,
                    lora_a_ptr=(lambda ref_table=ref_table: ref_table("weights_a")),
                    lora_b_ptr=(lambda ref_table=ref_table: ref_table("weights_b")),
                    tmp_shrink=tmp_shrink,
                    tmp_expand=tmp_expand,
                    segment_starts=dev32[g.starts_off // 4 : g.starts_off // 4 + n],
                    segment_ends=dev32[g.ends_off // 4 : g.ends_off // 4 + n],
                    indices=None,
                    lora_a_t_ptr=a_ptr,
                    lora_b_t_ptr=b_ptr,
                    segments_key=(packed[g.starts_off : g.starts_off + 4 * n].tobytes(),
                                  packed[g.ends_off : g.ends_off + 4 * n].tobytes()),
                    num_long_segments=g.num_long_segments,
                    short_plan=dev64[g.plan_off // 8 : g.plan_off // 8 + g.num_chunks * BGMV_PLAN_WORDS].view(
                        g.num_chunks, BGMV_PLAN_WORDS) if g.plan_off >= 0 else None,
                    shrink_tiles=_native.TilePlan(
                        dev32[g.shrink_tiles_off // 4 : g.shrink_tiles_off // 4 + 4 * g.num_shrink_tiles].view(-1, 4),
                        g.shrink_tile_rows) if g.shrink_tiles_off >= 0 else None,
                    expand_tiles=_native.TilePlan(
                        dev32[g.expand_tiles_off // 4 : g.expand_tiles_off // 4 + 4 * g.num_expand_tiles].view(-1, 4),
                        g.expand_tile_rows) if g.expand_tiles_off >= 0 else None,
                )
            else:
                rank_data[g.rank] = RankSegments(
                    rank=g.rank,
                    lora_a_ptr=a_ptr,
                    lora_b_ptr=b_ptr,
                    tmp_shrink=None,
                    tmp_expand=None,
                    segment_starts=None,
                    segment_ends=None,
                    indices=dev64[g.indices_off // 8 : g.indices_off // 8 + T],
                    plan=dev64[g.plan_off // 8 : g.plan_off // 8 + g.num_chunks * BGMV_PLAN_WORDS].view(
                        g.num_chunks, BGMV_PLAN_WORDS),
                )
        data[layer_name] = {
            LORA: BatchLoraWeights(
                lora_a=_LayoutView(loras, "weights_a"),
                lora_b=_LayoutView(loras, "weights_b"),
                adapter_index_configs={a: lw.adapter_config for a, lw in loras.items()},
                rank_data=rank_data,
                use_sgmv=use_sgmv,
                layer_name=layer_name,
                prefill_head_indices=None,
            )
        }
    return data
