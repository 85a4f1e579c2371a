"""Deterministic synthetic workloads: the five benchmark configurations of the multi-adapter
LoRA path (decode batches routed by per-token adapter index, prefill batches routed by
segments), built with the real adapter containers so that a workload exercises the same
routing-table code a server would.

A workload owns, per projection group (e.g. fused q/k/v), the input activations and, per
layer type, a ``LayerAdapterWeights`` with one ``LoraWeights`` per resident adapter.
Weights are N(0, 0.02), activations N(0, 1); everything is derived from one seed.
"""

import math
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Tuple

import torch

from lorax_amd.adapters import (
    AdapterBatchData,
    AdapterBatchMetadata,
    LayerAdapterWeights,
    LoraConfig,
    LoraWeights,
)
from lorax_amd.segments import find_segments


@dataclass
class ProjectionGroup:
    """Projections that share one input and write column slices of one fused output."""

    name: str
    layer_names: List[str]
    h_in: int
    sizes: List[int]  # output width of every layer name

    @property
    def h_out(self) -> int:
        return sum(self.sizes)


@dataclass
class Workload:
    name: str
    dtype: torch.dtype
    device: torch.device
    num_layers: int
    prefill: bool
    groups: List[ProjectionGroup]
    adapter_indices: List[int]  # per token; -1 = no adapter
    rank_of_adapter: Dict[int, int]  # resident adapters with weights
    inputs: Dict[str, torch.Tensor] = field(default_factory=dict)  # group name -> [T, h_in]
    weights: Dict[str, LayerAdapterWeights] = field(default_factory=dict)  # layer name -> adapters
    meta: Optional[AdapterBatchMetadata] = None
    # Segments added to every rank group's tables after they are built: (start, end, adapter) with
    # end <= start, adapter None = a null stack address.  A serving loop produces such entries when it
    # pads its tables to a fixed size (the reference's own SGMV test passes them, server/tests/utils/
    # test_sgmv.py:46-47); the run-length routing of a real batch never does.
    extra_segments: List[Tuple[int, int, Optional[int]]] = field(default_factory=list)

    @property
    def num_tokens(self) -> int:
        return len(self.adapter_indices)

    def routed_tokens(self) -> int:
        return sum(1 for a in self.adapter_indices if a in self.rank_of_adapter)

    def distinct_adapters(self) -> int:
        return len({a for a in self.adapter_indices if a in self.rank_of_adapter})

    def batch_data(self) -> AdapterBatchData:
        batch = AdapterBatchData.from_meta(self.meta, self.weights, {}, None, self.prefill, None)
        if self.extra_segments and self.prefill:
            _inject_segments(self, batch)
        return batch


def _splice_rank_group(rs, layer, rank: int, extra) -> None:
    """Adds the segments `extra` to one rank group's tables: the first one in front of the group's second
    segment, the others at the end - of the long segments, when the group lists its short segments last and
    routes them through a plan (the segment kernels then see the added entries too)."""
    from lorax_amd.sgmv import get_tmp_tensors

    n = rs.segment_starts.numel()
    n_long = rs.num_long_segments if rs.short_plan is not None else n
    at = [min(1, n_long)] + [n_long] * (len(extra) - 1)  # insertion points in the original table

    def spliced(table, values, dtype):
        parts, prev = [], 0
        for pos, val in zip(at, values):
            parts += [table[prev:pos], torch.tensor([val], dtype=dtype, device=table.device)]
            prev = pos
        parts.append(table[prev:])
        return torch.cat(parts)

    def addrs(layout):
        out = []
        for _, _, adapter in extra:
            lw = layer.get(adapter) if adapter is not None else None
            out.append(getattr(lw, layout).data_ptr() if lw is not None and lw.lora_a_r == rank else 0)
        return out

    def later(old, layout):  # the reference-layout tables are built on first access
        return lambda: spliced(old() if callable(old) else old, addrs(layout), torch.int64)

    rs._lora_a_ptr = later(rs._lora_a_ptr, "weights_a")
    rs._lora_b_ptr = later(rs._lora_b_ptr, "weights_b")
    rs.lora_a_t_ptr = spliced(rs.lora_a_t_ptr, addrs("weights_a_t"), torch.int64)
    rs.lora_b_t_ptr = spliced(rs.lora_b_t_ptr, addrs("weights_b_t"), torch.int64)
    rs.segment_starts = spliced(rs.segment_starts, [s for s, _, _ in extra], torch.int32)
    rs.segment_ends = spliced(rs.segment_ends, [e for _, e, _ in extra], torch.int32)
    rs.tmp_shrink, rs.tmp_expand = get_tmp_tensors(n + len(extra), rank, rs.segment_starts.device)
    rs.num_long_segments = n_long + len(extra)
    if rs.segments_key is not None:
        rs.segments_key = (rs.segments_key, tuple(extra))
    # the row-tile plans name segments by their position in the tables: cut them again for the new tables
    from lorax_amd.adapters import _tile_plans

    rs.shrink_tiles, rs.expand_tiles = _tile_plans(rs.segment_starts.tolist(), rs.segment_ends.tolist(),
                                                   rs.num_long_segments, rs.segment_starts.device, rank)


def _inject_segments(w: "Workload", batch: AdapterBatchData) -> None:
    """Adds w.extra_segments to the segment tables of every rank group of a prefill batch."""
    from lorax_amd.adapters import LORA

    for name, per_type in batch.data.items():
        data = per_type.get(LORA)
        if data is None or not data.use_sgmv:
            continue
        for rank, rs in data.rank_data.items():
            _splice_rank_group(rs, w.weights[name].adapter_weights, rank, w.extra_segments)


def _randn(shape, std, gen, dtype, device):
    if gen.device.type == "cpu":
        t = torch.randn(shape, generator=gen, dtype=torch.float32) * std
        return t.to(dtype).to(device)
    return (torch.randn(shape, generator=gen, dtype=torch.float32, device=gen.device) * std).to(dtype)


def _make_generator(seed: int, device: torch.device, on_device: bool) -> torch.Generator:
    gen = torch.Generator(device=device if (on_device and device.type == "cuda") else "cpu")
    gen.manual_seed(seed)
    return gen


def make_meta(adapter_indices: Sequence[int], device: torch.device) -> AdapterBatchMetadata:
    """Batch metadata as the serving loop builds it (flash_causal_lm.py:1012-1021): int64 per-token
    indices and int32 run boundaries on the device, run owners as a host list."""
    bounds, owners = find_segments(list(adapter_indices))
    return AdapterBatchMetadata(
        adapter_indices=torch.tensor(list(adapter_indices), dtype=torch.int64, device=device),
        adapter_list=list(adapter_indices),
        adapter_set=set(int(a) for a in adapter_indices),
        adapter_segments=torch.tensor(bounds, dtype=torch.int32, device=device),
        segment_indices=owners,
    )


def _populate(w: Workload, seed: int, weights_on_device: bool, adapters_with_weights: Optional[Dict[str, set]] = None):
    gen_cpu = _make_generator(seed, w.device, False)
    gen_w = _make_generator(seed + 7919, w.device, weights_on_device)
    T = w.num_tokens
    for g in w.groups:
        w.inputs[g.name] = _randn((T, g.h_in), 1.0, gen_cpu, w.dtype, w.device)
        for name, h_out in zip(g.layer_names, g.sizes):
            layer = LayerAdapterWeights()
            for adapter, rank in w.rank_of_adapter.items():
                if adapters_with_weights is not None and adapter not in adapters_with_weights.get(name, ()):
                    continue
                a = _randn((w.num_layers, g.h_in, rank), 0.02, gen_w, w.dtype, w.device)
                b = _randn((w.num_layers, rank, h_out), 0.02, gen_w, w.dtype, w.device)
                layer.add_adapter(adapter, LoraWeights(list(a.unbind(0)), list(b.unbind(0)), LoraConfig(r=rank)))
            w.weights[name] = layer
    w.meta = make_meta(w.adapter_indices, w.device)


LLAMA7B_Q = [ProjectionGroup("q_proj", ["q_proj"], 4096, [4096])]
GQA_ATTN = [
    ProjectionGroup("qkv", ["q_proj", "k_proj", "v_proj"], 4096, [4096, 1024, 1024]),
    ProjectionGroup("o_proj", ["o_proj"], 4096, [4096]),
]
MISTRAL_MLP = [
    ProjectionGroup("gate_up", ["gate_proj", "up_proj"], 4096, [14336, 14336]),
    ProjectionGroup("down_proj", ["down_proj"], 14336, [4096]),
]
LLAMA70B_LAYER = [
    ProjectionGroup("qkv", ["q_proj", "k_proj", "v_proj"], 8192, [8192, 1024, 1024]),
    ProjectionGroup("o_proj", ["o_proj"], 8192, [8192]),
    ProjectionGroup("gate_up", ["gate_proj", "up_proj"], 8192, [28672, 28672]),
    ProjectionGroup("down_proj", ["down_proj"], 28672, [8192]),
]


def config1(device, num_layers: int = 32, weights_on_device: bool = False) -> Workload:
    """fp16, 64 tokens in 4 runs of 16, adapters 0..3 of rank 16, one 4096 -> 4096 q_proj (prefill)."""
    idx = [t // 16 for t in range(64)]
    w = Workload("cfg1_llama7b_q_prefill", torch.float16, torch.device(device), num_layers, True, LLAMA7B_Q, idx,
                 {a: 16 for a in range(4)})
    _populate(w, 1001, weights_on_device)
    return w


def config2(device, num_layers: int = 32, weights_on_device: bool = False, num_tokens: int = 256,
            num_adapters: int = 128) -> Workload:
    """bf16 decode: 256 tokens, adapter uniform over 128 resident rank-8 adapters, 5 % of tokens with no
    adapter, LoRA on q/k/v/o of a GQA attention block (4096/1024/1024/4096)."""
    gen = torch.Generator(device="cpu").manual_seed(1002)
    idx = torch.randint(0, num_adapters, (num_tokens,), generator=gen)
    drop = torch.rand((num_tokens,), generator=gen) < 0.05
    idx[drop] = -1
    w = Workload("cfg2_bgmv_decode_qkvo", torch.bfloat16, torch.device(device), num_layers, False, GQA_ATTN,
                 idx.tolist(), {a: 8 for a in range(num_adapters)})
    _populate(w, 1002, weights_on_device)
    return w


def config3(device, num_layers: int = 32, weights_on_device: bool = False, num_segments: int = 32,
            min_len: int = 16, max_len: int = 2048) -> Workload:
    """bf16 prefill: 32 runs with log-uniform lengths in [16, 2048], one distinct rank-64 adapter per run,
    LoRA on the Mistral-7B MLP (gate/up 4096 -> 14336, down 14336 -> 4096)."""
    gen = torch.Generator(device="cpu").manual_seed(1003)
    u = torch.rand((num_segments,), generator=gen)
    lens = torch.floor(torch.exp(math.log(min_len) + u * (math.log(max_len) - math.log(min_len)))).long()
    idx: List[int] = []
    for a, n in enumerate(lens.tolist()):
        idx.extend([a] * n)
    w = Workload("cfg3_sgmv_prefill_mlp", torch.bfloat16, torch.device(device), num_layers, True, MISTRAL_MLP, idx,
                 {a: 64 for a in range(num_segments)})
    _populate(w, 1003, weights_on_device)
    return w


def config4(device, num_layers: int = 2, weights_on_device: bool = True, num_tokens: int = 512,
            num_adapters: int = 500, resident_only_active: bool = False) -> Workload:
    """bf16 decode: 512 tokens over 500 adapters with Zipf(1.1) popularity, rank of every adapter drawn
    from {8, 16, 32, 64}, all seven projections of a Mistral-7B decoder block."""
    gen = torch.Generator(device="cpu").manual_seed(1004)
    weights = 1.0 / torch.arange(1, num_adapters + 1, dtype=torch.float64) ** 1.1
    idx = torch.multinomial(weights / weights.sum(), num_tokens, replacement=True, generator=gen)
    ranks = torch.tensor([8, 16, 32, 64])[torch.randint(0, 4, (num_adapters,), generator=gen)]
    rank_of = {a: int(ranks[a]) for a in range(num_adapters)}
    if resident_only_active:
        active = set(idx.tolist())
        rank_of = {a: r for a, r in rank_of.items() if a in active}
    w = Workload("cfg4_bgmv_decode_block_multirank", torch.bfloat16, torch.device(device), num_layers, False,
                 GQA_ATTN + MISTRAL_MLP, idx.tolist(), rank_of)
    _populate(w, 1004, weights_on_device)
    return w


def config5(device, num_layers: int = 1, weights_on_device: bool = True, prefill_tokens: int = 4096,
            decode_tokens: int = 256, num_adapters: int = 256, groups: Optional[List[ProjectionGroup]] = None,
            resident_only_active: bool = False) -> Workload:
    """bf16 mixed batch on a Llama-70B-shaped layer: one chunked-prefill run plus single-token decode runs,
    `num_adapters` resident rank-128 adapters, a run of tokens whose adapter has no weights, tokens with no
    adapter at all, and two empty entries in every rank group's segment tables: one with start == end and a
    valid stack address, one (-1, -1) with a null address.  The whole batch is routed by segments, as the
    reference does for any batch with a prefilling request (flash_causal_lm.py:1594,1617).
    resident_only_active keeps weights only for the adapters the batch uses (for tests on small memory)."""
    gen = torch.Generator(device="cpu").manual_seed(1005)
    dec = torch.randint(0, num_adapters, (decode_tokens,), generator=gen).tolist()
    no_weights_adapter = num_adapters  # resident nowhere: its runs are dropped from every rank group
    idx = [dec[0]] * prefill_tokens  # the long run shares an adapter with the first decode token
    idx += [no_weights_adapter] * 5
    idx += dec[: decode_tokens // 2]
    idx += [-1] * 4
    idx += dec[decode_tokens // 2 :]
    rank_of = {a: 128 for a in range(num_adapters)}
    if resident_only_active:
        active = set(idx)
        rank_of = {a: r for a, r in rank_of.items() if a in active}
    w = Workload("cfg5_llama70b_mixed_prefill_decode", torch.bfloat16, torch.device(device), num_layers, True,
                 groups if groups is not None else LLAMA70B_LAYER, idx, rank_of)
    w.extra_segments = [(prefill_tokens // 2, prefill_tokens // 2, dec[0]), (-1, -1, None)]
    _populate(w, 1005, weights_on_device)
    return w


def config5_decode(device, num_layers: int = 1, weights_on_device: bool = True, decode_tokens: int = 256,
                   num_adapters: int = 256, groups: Optional[List[ProjectionGroup]] = None,
                   resident_only_active: bool = False) -> Workload:
    """The decode tokens of the mixed Llama-70B batch on their own, as a decode batch (per-token routing, BGMV):
    the same adapter draw as config5, `num_adapters` resident rank-128 adapters, four tokens without adapter."""
    gen = torch.Generator(device="cpu").manual_seed(1005)
    dec = torch.randint(0, num_adapters, (decode_tokens,), generator=gen).tolist()
    idx = dec[: decode_tokens // 2] + [-1] * 4 + dec[decode_tokens // 2 :]
    rank_of = {a: 128 for a in range(num_adapters)}
    if resident_only_active:
        active = set(idx)
        rank_of = {a: r for a, r in rank_of.items() if a in active}
    w = Workload("cfg5_llama70b_decode_tokens_bgmv", torch.bfloat16, torch.device(device), num_layers, False,
                 groups if groups is not None else LLAMA70B_LAYER, idx, rank_of)
    _populate(w, 1005, weights_on_device)
    return w


def mid_prefill(device, num_layers: int = 16, weights_on_device: bool = True, num_segments: int = 10) -> Workload:
    """bf16 prefill of about a thousand tokens (10 runs of 32..256 tokens, one rank-64 adapter each) on the
    Mistral-7B MLP: the band between the streaming shrink (a few hundred rows) and batches with enough row tiles
    for every CU; not one of the five benchmark configurations."""
    w = config3(device, num_layers, weights_on_device, num_segments=num_segments, min_len=32, max_len=256)
    w.name = "mid_prefill_1k_mlp"
    return w


CONFIGS = {1: config1, 2: config2, 3: config3, 4: config4, 5: config5}
