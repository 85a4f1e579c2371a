"""End-to-end parity of the LoRA layers on the five benchmark configurations: routing tables built by
BatchLoraWeights, kernels called by LoraLinear.forward_layer_type, result compared with the
reference's per-adapter masked matmul loop (the oracle's fallback_layer_type) on the same inputs.

The oracle loop is dense over all tokens for every adapter, so it runs on reduced layer counts
(the kernels index one layer of the stack; the others only occupy memory) and, for the largest
shapes, on the LoRA delta of a subset of projections; full-size runs are checked through
size-independent properties in test_gpu_properties.py."""

import pytest
import torch

from lorax_amd import synthetic
from lorax_amd.adapters import LORA
from lorax_amd.layers import TensorParallelAdapterRowLinear, TensorParallelMultiAdapterLinear
from oracle import lora_oracle as O
from tests.helpers import assert_close

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


class ZeroBase(torch.nn.Module):
    """Base projection that returns y0 (a fixed tensor) so the test isolates the LoRA path."""

    def __init__(self, y0):
        super().__init__()
        self.y0 = y0

    def forward(self, x):
        return self.y0.clone()


def _oracle_group(w, group, layer_id, y0_cpu):
    x = w.inputs[group.name].cpu()
    idx = torch.tensor(w.adapter_indices)
    result = y0_cpu.clone()
    off = 0
    for name, size in zip(group.layer_names, group.sizes):
        layer = w.weights[name]
        lora_a = {a: lw.weights_a.cpu() for a, lw in layer.adapter_weights.items() if a in set(w.adapter_indices)}
        lora_b = {a: lw.weights_b.cpu() for a, lw in layer.adapter_weights.items() if a in set(w.adapter_indices)}
        O.fallback_layer_type(result, x, idx, set(w.adapter_indices), lora_a, lora_b, layer_id, off, off + size)
        off += size
    return result


def _run_group(w, group, layer_id, y0, batch):
    base = ZeroBase(y0)
    x = w.inputs[group.name]
    if len(group.layer_names) == 1 and group.name in ("o_proj", "down_proj"):
        layer = TensorParallelAdapterRowLinear.load(base, layer_id, group.layer_names[0])
    else:
        sizes = group.sizes if len(group.layer_names) > 1 else None
        layer = TensorParallelMultiAdapterLinear.load(base, layer_id, group.layer_names, sizes)
    return layer(x, batch)


def _check_workload(w, layer_id, y0_std):
    batch = w.batch_data()
    gen = torch.Generator().manual_seed(99)
    untouched = torch.tensor([a not in w.rank_of_adapter for a in w.adapter_indices])
    for group in w.groups:
        print(f"{w.name}: group {group.name} T={w.num_tokens}", flush=True)
        y0 = (torch.randn((w.num_tokens, group.h_out), generator=gen) * y0_std).to(w.dtype)
        out = _run_group(w, group, layer_id, y0.to(DEV), batch)
        torch.cuda.synchronize()
        ref = _oracle_group(w, group, layer_id, y0)
        delta_ref = (ref.float() - y0.float()).to(w.dtype)
        assert_close(out, ref, f"{w.name}/{group.name}", rounded=[delta_ref])
        assert_close(out.float().cpu() - y0.float(), ref.float() - y0.float(), f"{w.name}/{group.name} delta",
                     rounded=[ref, delta_ref])  # fp32 differences of values rounded twice
        assert torch.equal(out.cpu()[untouched], y0[untouched]), "rows without an adapter must be bit-identical"


def assert_has_empty_segments(w, batch):
    """Every rank group of a cfg5 batch carries an empty segment with a valid stack address (start == end) and
    a (-1, -1) segment with a null address, next to its real segments."""
    seen = 0
    for per_type in batch.data.values():
        for rd in per_type[LORA].rank_data.values():
            rows = list(zip(rd.segment_starts.tolist(), rd.segment_ends.tolist(), rd.lora_a_t_ptr.tolist(),
                            rd.lora_b_t_ptr.tolist()))
            assert any(s == e and s >= 0 and a != 0 and b != 0 for s, e, a, b in rows), rows
            assert any(s == -1 and e == -1 and a == 0 and b == 0 for s, e, a, b in rows), rows
            assert rd.tmp_expand.numel() == 60 * len(rows)
            seen += 1
    assert seen > 0


def test_config1_llama7b_q_proj_prefill():
    w = synthetic.config1(DEV, num_layers=2)
    assert w.meta.adapter_segments.tolist() == [0, 16, 32, 48, 64] and w.meta.segment_indices == [0, 1, 2, 3]
    data = w.batch_data().data["q_proj"][LORA]
    assert data.use_sgmv and list(data.rank_data) == [16]
    _check_workload(w, 1, 0.5)
    _check_workload(w, 0, 0.0)


def test_config2_bgmv_decode_qkvo():
    w = synthetic.config2(DEV, num_layers=2)
    assert w.num_tokens == 256 and 0 < w.num_tokens - w.routed_tokens() < 40
    data = w.batch_data().data["q_proj"][LORA]
    assert not data.use_sgmv and list(data.rank_data) == [8]
    _check_workload(w, 1, 0.25)
    _check_workload(w, 0, 0.0)


def test_config3_sgmv_prefill_mlp_reduced():
    # same generator as the full configuration with shorter runs: 12 runs, lengths in [16, 300]
    w = synthetic.config3(DEV, num_layers=2, num_segments=12, max_len=300)
    assert all(rd.rank == 64 for rd in w.batch_data().data["gate_proj"][LORA].rank_data.values())
    _check_workload(w, 1, 0.5)


def test_config4_bgmv_multirank_decode_block():
    w = synthetic.config4(DEV, num_layers=2, weights_on_device=False, num_tokens=512, resident_only_active=True)
    batch = w.batch_data()
    ranks = set(batch.data["q_proj"][LORA].rank_data)
    assert ranks == {8, 16, 32, 64}
    for rd in batch.data["down_proj"][LORA].rank_data.values():
        members = (rd.indices >= 0).sum().item()
        assert 0 < members < w.num_tokens  # every rank group leaves the others' tokens at -1
    _check_workload(w, 1, 0.25)


def test_config5_llama70b_mixed_batch_reduced():
    # the real hidden sizes with a shorter prefill run and fewer decode tokens; attention projections
    groups = [g for g in synthetic.LLAMA70B_LAYER if g.name in ("qkv", "o_proj")]
    w = synthetic.config5(DEV, num_layers=1, weights_on_device=False, prefill_tokens=300, decode_tokens=24,
                          num_adapters=16, groups=groups)
    batch = w.batch_data()
    data = batch.data["q_proj"][LORA]
    assert data.use_sgmv and list(data.rank_data) == [128]
    rd = data.rank_data[128]
    lens = (rd.segment_ends - rd.segment_starts).tolist()
    assert max(lens) >= 300 and lens.count(1) >= 10
    # the run whose adapter has no weights and the run with no adapter are in no rank group; two empty
    # entries were added to the tables
    assert len(lens) - 2 < len(w.meta.segment_indices)
    assert_has_empty_segments(w, batch)
    assert len(w.rank_of_adapter) == 16  # every adapter resident, not only the batch's
    _check_workload(w, 0, 0.25)


def test_config5_mlp_projections_reduced():
    groups = [g for g in synthetic.LLAMA70B_LAYER if g.name in ("gate_up", "down_proj")]
    w = synthetic.config5(DEV, num_layers=1, weights_on_device=False, prefill_tokens=130, decode_tokens=8,
                          num_adapters=6, groups=groups)
    assert_has_empty_segments(w, w.batch_data())
    _check_workload(w, 0, 0.25)


def test_config5_many_decode_tokens_take_the_per_token_kernels():
    # enough one-row segments for the tables to list them last with a routing plan: the segment kernels then run
    # the long segments (the added empty ones among them) and the per-token kernels the decode rows
    groups = [g for g in synthetic.LLAMA70B_LAYER if g.name in ("qkv", "down_proj")]
    w = synthetic.config5(DEV, num_layers=1, weights_on_device=False, prefill_tokens=200, decode_tokens=44,
                          num_adapters=12, groups=groups)
    batch = w.batch_data()
    for name in ("q_proj", "down_proj"):
        rd = batch.data[name][LORA].rank_data[128]
        lens = (rd.segment_ends - rd.segment_starts).tolist()
        assert rd.short_plan is not None and 0 < rd.num_long_segments < len(lens)
        assert all(n > 4 or n <= 0 for n in lens[: rd.num_long_segments])  # long runs and the two empty entries
        assert all(1 <= n <= 4 for n in lens[rd.num_long_segments :])
        assert int(rd.short_plan[:, 0].sum()) == sum(lens[rd.num_long_segments :])
    assert_has_empty_segments(w, batch)
    _check_workload(w, 0, 0.25)


def test_prefill_batch_of_short_segments_only():
    """A prefill batch whose segments all have one to four rows (many requests with tiny prompts): the tables hold
    no long segment at all and the per-token kernels do the whole update."""
    gen = torch.Generator().manual_seed(21)
    idx = []
    for _ in range(40):
        a = int(torch.randint(0, 6, (1,), generator=gen))
        idx += [a] * int(torch.randint(1, 5, (1,), generator=gen)) + [-1]
    groups = [synthetic.ProjectionGroup("qkv", ["q_proj", "k_proj", "v_proj"], 1024, [1024, 256, 256]),
              synthetic.ProjectionGroup("o_proj", ["o_proj"], 1024, [1024])]
    w = synthetic.Workload("short_segments_only", torch.bfloat16, torch.device(DEV), 1, True, groups, idx,
                           {a: 32 for a in range(6)})
    synthetic._populate(w, 21, False)
    batch = w.batch_data()
    rd = batch.data["q_proj"][LORA].rank_data[32]
    assert rd.short_plan is not None and rd.num_long_segments == 0
    _check_workload(w, 0, 0.25)


def test_config5_decode_tokens_alone_as_bgmv_reduced():
    # the decode share of the mixed batch as a decode batch: rank 128, the real hidden sizes, fewer tokens
    for names in (("qkv", "o_proj"), ("gate_up", "down_proj")):
        groups = [g for g in synthetic.LLAMA70B_LAYER if g.name in names]
        w = synthetic.config5_decode(DEV, num_layers=1, weights_on_device=False, decode_tokens=20, num_adapters=8,
                                     groups=groups)
        batch = w.batch_data()
        data = batch.data[groups[0].layer_names[0]][LORA]
        assert not data.use_sgmv and list(data.rank_data) == [128]
        assert (data.rank_data[128].indices < 0).sum().item() == 4
        _check_workload(w, 0, 0.25)


@pytest.mark.parametrize("prefill", [True, False])
def test_lm_head_with_a_large_vocabulary(prefill):
    """The LM head through MultiAdapterHead: 70 000 output columns (more than the reference's BGMV kernels take),
    adapters of rank 8 and 16 and requests without adapter.  In prefill the head sees one row per request, picked
    by prefill_head_indices, and the segment bounds are recounted in those rows."""
    from lorax_amd.adapters import LM_HEAD, AdapterBatchData, LayerAdapterWeights, LoraConfig, LoraWeights
    from lorax_amd.layers import MultiAdapterHead
    from lorax_amd.synthetic import make_meta

    dtype, hidden, vocab = torch.bfloat16, 1024, 70000
    gen = torch.Generator().manual_seed(5)
    request_adapters = [0, 0, 1, 7, 1, 2, 2, 2, 7, 0]      # 7 has no weights
    lens = [5, 1, 9, 3, 2, 6, 1, 4, 2, 8] if prefill else [1] * len(request_adapters)
    tokens = [a for a, n in zip(request_adapters, lens) for _ in range(n)]
    meta = make_meta(tokens, torch.device(DEV))
    head_idx = None
    if prefill:
        ends = torch.tensor(lens).cumsum(0)
        head_idx = (ends - 1).to(torch.int64).to(DEV)  # last token of every request
    layer = LayerAdapterWeights()
    ranks = {0: 8, 1: 16, 2: 16}
    for a, r in ranks.items():
        wa = (torch.randn((1, hidden, r), generator=gen) * 0.05).to(dtype).to(DEV)
        wb = (torch.randn((1, r, vocab), generator=gen) * 0.05).to(dtype).to(DEV)
        layer.add_adapter(a, LoraWeights(list(wa.unbind(0)), list(wb.unbind(0)), LoraConfig(r=r)))
    batch = AdapterBatchData.from_meta(meta, {LM_HEAD: layer}, prefill=prefill, prefill_head_indices=head_idx)
    rows = len(request_adapters)
    x = (torch.randn((rows, hidden), generator=gen)).to(dtype)
    y0 = (torch.randn((rows, vocab), generator=gen) * 0.25).to(dtype)
    head = MultiAdapterHead.load(ZeroBase(y0.to(DEV)), 0, LM_HEAD)
    logits, speculative = head(x.to(DEV), batch)
    torch.cuda.synchronize()
    assert speculative is None
    ref = y0.clone()
    idx = torch.tensor(request_adapters)
    lora_a = {a: lw.weights_a.cpu() for a, lw in layer.adapter_weights.items()}
    lora_b = {a: lw.weights_b.cpu() for a, lw in layer.adapter_weights.items()}
    O.fallback_layer_type(ref, x, idx, set(request_adapters), lora_a, lora_b, 0, 0, vocab)
    delta = (ref.float() - y0.float()).to(dtype)
    assert_close(logits, ref, "lm_head logits", rounded=[delta])
    untouched = torch.tensor([a not in ranks for a in request_adapters])
    assert torch.equal(logits.cpu()[untouched], y0[untouched])
    assert torch.count_nonzero(logits.cpu()[~untouched] != y0[~untouched]) > 0


@pytest.mark.parametrize("mode,lens", [
    ("decode", [1] * 12),
    ("prefill", [40, 3, 9, 1, 17, 5, 30, 2, 8, 1, 6, 11]),          # a short batch
    ("prefill", [300, 3, 90, 1, 170, 50, 30, 2, 80, 1, 60, 110]),   # past the streaming kernels' range
])
def test_ranks_above_the_kernel_limit_run_as_rank_chunks(mode, lens):
    """Adapters of rank 192 and 256 next to one of rank 16 and requests without adapter, on a fused q/k/v
    projection: the kernels take ranks up to 128, so such an adapter is served as chunks of its rank (128 + 64,
    128 + 128), each a rank group of its own.  The oracle multiplies with the whole rank at once."""
    _check_rank_chunks(mode, [0, 1, 2, 9, 1, 0, 2, 2, 9, 0, 1, 1], lens)      # 9 has no weights


def test_rank_chunks_with_many_short_segments():
    """The same in a prefill batch with dozens of one- to three-row segments per chunked adapter: every chunk's
    rank group lists them last and routes them through the per-token kernels, chunk after chunk."""
    adapters, lens = [0, 1], [60, 20]
    for i in range(40):
        adapters += [0, 9, 1, 9]
        lens += [1 + i % 3, 1, 1 + (i + 1) % 3, 2]
    batch = _check_rank_chunks("prefill", adapters, lens)
    for key, rs in batch.data["q_proj"][LORA].rank_data.items():
        assert (rs.short_plan is not None) == isinstance(key, tuple), key  # adapter 2 (rank 16) is not in the batch


def _check_rank_chunks(mode, request_adapters, lens):
    from lorax_amd.adapters import AdapterBatchData, LayerAdapterWeights, LoraConfig, LoraWeights
    from lorax_amd.synthetic import make_meta

    prefill = mode == "prefill"
    dtype, hidden, layers, layer_id = torch.bfloat16, 1024, 2, 1
    names, sizes = ["q_proj", "k_proj", "v_proj"], [1024, 256, 256]
    gen = torch.Generator().manual_seed(len(lens) + sum(lens))
    ranks = {0: 192, 1: 256, 2: 16}
    tokens = [a for a, n in zip(request_adapters, lens) for _ in range(n)]
    meta = make_meta(tokens, torch.device(DEV))
    weights = {}
    for name, size in zip(names, sizes):
        layer = LayerAdapterWeights()
        for a, r in ranks.items():
            wa = (torch.randn((layers, hidden, r), generator=gen) * 0.05).to(dtype).to(DEV)
            wb = (torch.randn((layers, r, size), generator=gen) * 0.05).to(dtype).to(DEV)
            layer.add_adapter(a, LoraWeights(list(wa.unbind(0)), list(wb.unbind(0)), LoraConfig(r=r)))
        weights[name] = layer
    batch = AdapterBatchData.from_meta(meta, weights, prefill=prefill)
    groups = batch.data["q_proj"][LORA].rank_data
    expect = [(192, 0), (192, 1), (256, 0), (256, 1)] + ([16] if 2 in request_adapters else [])
    assert sorted(map(str, groups)) == sorted(map(str, expect))
    assert sorted(rs.rank for rs in groups.values()) == ([16] if 2 in request_adapters else []) + [64, 128, 128, 128]
    assert batch.data["q_proj"][LORA].use_sgmv == prefill

    T = len(tokens)
    x = torch.randn((T, hidden), generator=gen).to(dtype)
    y0 = (torch.randn((T, sum(sizes)), generator=gen) * 0.25).to(dtype)
    proj = TensorParallelMultiAdapterLinear.load(ZeroBase(y0.to(DEV)), layer_id, names, sizes)
    out = proj(x.to(DEV), batch)
    torch.cuda.synchronize()
    ref, off, idx = y0.clone(), 0, torch.tensor(tokens)
    for name, size in zip(names, sizes):
        lora_a = {a: lw.weights_a.cpu() for a, lw in weights[name].adapter_weights.items()}
        lora_b = {a: lw.weights_b.cpu() for a, lw in weights[name].adapter_weights.items()}
        O.fallback_layer_type(ref, x, idx, set(tokens), lora_a, lora_b, layer_id, off, off + size)
        off += size
    delta = (ref.float() - y0.float()).to(dtype)
    # a chunked adapter's update reaches y in two roundings (one per chunk) instead of one
    assert_close(out, ref, f"rank chunks, {mode}", rounded=[delta, delta])
    untouched = torch.tensor([a not in ranks for a in tokens])
    assert torch.equal(out.cpu()[untouched], y0[untouched])
    return batch
