"""Host-side mirror of the reference API (no GPU): routing tables, padding, orientation, the
scratch-size contract - against the reference tests' golden vectors and against the oracle."""

import json
from pathlib import Path
from unittest import mock

import pytest
import torch

from lorax_amd import punica, sgmv
from lorax_amd.adapters import (
    LORA,
    LM_HEAD,
    AdapterBatchData,
    AdapterBatchMetadata,
    AdapterWeights,
    BatchAdapterWeights,
    LayerAdapterWeights,
    LoraConfig,
    LoraWeights,
    get_scaling_factor,
)
from lorax_amd.layers import SingleProcessGroup
from lorax_amd.segments import SegmentConcatBuilder, find_segments
from oracle import lora_oracle as O

GOLDEN = Path(__file__).resolve().parent / "golden"


def _golden(name):
    return json.loads((GOLDEN / f"{name}.json").read_text())


def test_surface_matches_reference_names():
    for name in ["MIN_SGMV_RANK", "MIN_RANK_CUSTOM", "MAX_RANK_CUSTOM", "SGMV_BLOCK_SIZE", "BGMV_MAX_RANK",
                 "LORAX_PUNICA_TRITON_DISABLED", "has_sgmv", "pad_rank", "pad_to_min_rank", "use_cutlass_shrink",
                 "orient_for_rank", "add_lora_sgmv_cutlass", "lora_a_sgmv_cutlass", "lora_b_sgmv_cutlass",
                 "add_lora_a_bgmv", "add_lora_b_bgmv", "get_tmp_tensor", "get_tmp_tensors",
                 "get_tmp_tensor_for_size", "get_tmp_expand_size", "segmented_matmul"]:
        assert hasattr(sgmv, name), name
        assert getattr(punica, name) is getattr(sgmv, name), name
    assert (sgmv.MIN_SGMV_RANK, sgmv.MIN_RANK_CUSTOM, sgmv.MAX_RANK_CUSTOM, sgmv.SGMV_BLOCK_SIZE,
            sgmv.BGMV_MAX_RANK) == (8, 16, 128, 16, 128)


@pytest.mark.parametrize("case", _golden("segments")["find_segments"])
@pytest.mark.parametrize("as_tensor", [True, False])
def test_find_segments_golden(case, as_tensor):
    arg = torch.tensor(case["adapter_indices"]) if as_tensor else case["adapter_indices"]
    assert find_segments(arg) == (case["segments"], case["segment_indices"])


def test_find_segments_matches_oracle_on_random_runs():
    g = torch.Generator().manual_seed(5)
    for n in [1, 2, 7, 64, 513]:
        idx = torch.randint(-1, 4, (n,), generator=g)
        assert find_segments(idx) == O.find_segments_ref(idx.tolist())


@pytest.mark.parametrize("case", _golden("segments")["concat_segments"])
def test_concat_segments_golden(case):
    builder = SegmentConcatBuilder()
    for seg, idx in case["batches"]:
        builder.concat(torch.tensor(seg), idx)
    segments, owners = builder.build()
    assert segments.tolist() == case["segments"]
    assert owners == case["segment_indices"]
    assert O.concat_segments_ref(case["batches"]) == (case["segments"], case["segment_indices"])


@pytest.mark.parametrize("world_size", _golden("sgmv_kat")["pad_rank"]["world_sizes"])
@pytest.mark.parametrize("lora_rank", _golden("sgmv_kat")["pad_rank"]["lora_ranks"])
def test_pad_rank(lora_rank, world_size):
    assert sgmv.has_sgmv(), "the shared library must load on a machine without a GPU too"
    kat = _golden("sgmv_kat")["pad_rank"]
    x = torch.randn((kat["bs"], kat["h"]), dtype=torch.float16)
    a = torch.randn((kat["h"], lora_rank), dtype=torch.float16)
    b = torch.randn((lora_rank, kat["h"]), dtype=torch.float16)
    ap = sgmv.pad_rank(a, dim=1, world_size=world_size)
    bp = sgmv.pad_rank(b, dim=0, world_size=world_size)
    assert ap.size(1) == bp.size(0) >= lora_rank
    assert torch.equal(ap, O.pad_to_min_rank_ref(a, 1, 8 * world_size))
    assert torch.equal(bp, O.pad_to_min_rank_ref(b, 0, 8 * world_size))
    assert torch.allclose(x @ a @ b, x @ ap @ bp)


def test_orient_and_cutlass_shrink_rules():
    t = torch.zeros(6, 4)
    for r in [1, 8, 15, 16, 64, 128, 129, 256]:
        assert sgmv.use_cutlass_shrink(r) == (r < 16)
        assert sgmv.orient_for_rank(t, r).shape == O.orient_for_rank_ref(t, r).shape
    assert sgmv.orient_for_rank(t, 16).data_ptr() == t.data_ptr()  # a view, not a copy


def test_scaling_factor():
    assert get_scaling_factor(16, 8) == 2.0
    assert get_scaling_factor(16, 64, uses_rslora=True) == 2.0


def test_tmp_size_contract():
    for n in [0, 1, 2, 32, 257]:
        assert sgmv.get_tmp_expand_size(n) == O.sgmv_tmp_size_ref(n)


def _meta(adapter_indices, segments=None, segment_indices=None, adapter_list=None):
    if segments is None:
        segments, segment_indices = find_segments(adapter_indices)
    return AdapterBatchMetadata(
        adapter_indices=torch.tensor(adapter_indices, dtype=torch.int64),
        adapter_list=adapter_list if adapter_list is not None else adapter_indices,
        adapter_set=set(adapter_indices),
        adapter_segments=torch.tensor(segments, dtype=torch.int64),
        segment_indices=segment_indices,
    )


def _layer(ranks, h=1024):
    layer = LayerAdapterWeights()
    assert layer.is_empty()
    for idx, r in enumerate(ranks):
        w = LoraWeights([torch.randn((h, r), dtype=torch.float16)], [torch.randn((r, h), dtype=torch.float16)],
                        LoraConfig(r=r))
        assert w.lora_a_r == r and w.lora_b_r == r
        layer.add_adapter(idx, w)
    assert not layer.is_empty()
    return layer


@pytest.mark.parametrize("lora_ranks", _golden("lora_batch")["prefill"]["rank_sets"])
def test_batched_lora_weights_prefill(lora_ranks):
    gp = _golden("lora_batch")["prefill"]
    h = gp["h"]
    layer = _layer(lora_ranks, h)
    meta = _meta(gp["adapter_indices"], gp["adapter_segments"], gp["segment_indices"], gp["adapter_list"])
    with mock.patch("lorax_amd.adapters.get_tmp_tensors", return_value=(torch.empty(0), torch.empty(0))):
        data = layer.get_data(meta, LM_HEAD, prefill=True, prefill_head_indices=None).get(LORA)
    assert data.use_sgmv
    assert data.lora_a.keys() == meta.adapter_set and data.lora_b.keys() == meta.adapter_set
    for i, r in enumerate(lora_ranks):
        assert data.lora_a[i].shape == ((1, h, r) if r < gp["min_rank_custom"] else (1, r, h))
        assert data.lora_b[i].shape == (1, r, h)
    assert data.rank_data.keys() == set(lora_ranks)
    n = gp["entries_per_rank_group"]
    for r, rd in data.rank_data.items():
        assert rd.rank == r
        assert rd.lora_a_ptr.shape == rd.lora_b_ptr.shape == rd.segment_starts.shape == rd.segment_ends.shape == (n,)
        assert rd.indices is None
    # rank group of adapter 0 owns runs 0 and 2
    rd0 = data.rank_data[lora_ranks[0]]
    assert rd0.segment_starts.tolist() == [0, 4] and rd0.segment_ends.tolist() == [2, 6]
    assert rd0.lora_a_ptr.tolist() == [layer.adapter_weights[0].weights_a.data_ptr()] * 2
    assert rd0.lora_b_ptr.tolist() == [layer.adapter_weights[0].weights_b.data_ptr()] * 2


@pytest.mark.parametrize("case", _golden("lora_batch")["decode"])
def test_batched_lora_weights_decode(case):
    layer = _layer(case["lora_ranks"])
    meta = _meta(case["adapter_indices"])
    data = layer.get_data(meta, LM_HEAD, prefill=False, prefill_head_indices=None).get(LORA)
    assert not data.use_sgmv
    assert {str(r) for r in data.rank_data} == set(case["expected"])
    oracle = O.rank_groups_ref(meta.segment_indices, case["adapter_indices"],
                               {i: r for i, r in enumerate(case["lora_ranks"])})
    for r, rd in data.rank_data.items():
        exp = case["expected"][str(r)]
        assert rd.lora_a_ptr.shape == rd.lora_b_ptr.shape == (exp["num_ptrs"],)
        assert rd.indices.dtype == torch.int64 and rd.indices.tolist() == exp["indices"] == oracle[r][1]
        assert rd.segment_starts is None and rd.segment_ends is None
        assert rd.tmp_shrink is None and rd.tmp_expand is None
        # decode pointers address the [L, r, h_in] / [L, h_out, r] stacks of the run owners
        owners = [meta.segment_indices[p] for p in oracle[r][0]]
        assert rd.lora_a_ptr.tolist() == [layer.adapter_weights[a].weights_a_t.data_ptr() for a in owners]
        assert rd.lora_b_ptr.tolist() == [layer.adapter_weights[a].weights_b_t.data_ptr() for a in owners]


class _OtherWeights(AdapterWeights):
    @classmethod
    def get_batch_types(cls):
        return [_OtherBatch]


class _OtherBatch(BatchAdapterWeights):
    def has_adapter(self, adapter_index):
        return False

    @classmethod
    def key(cls):
        return "other"

    @classmethod
    def load(cls, adapter_weights, meta, layer_name, prefill, prefill_head_indices):
        return None


def test_batch_with_no_lora_segment_yields_nothing():
    g = _golden("lora_batch")["no_lora_segments"]
    layer = LayerAdapterWeights()
    layer.add_adapter(0, _OtherWeights())
    r = g["lora_rank"]
    layer.add_adapter(g["lora_adapter"], LoraWeights([torch.randn(64, r)], [torch.randn(r, 64)], LoraConfig(r=r)))
    meta = _meta(g["adapter_indices"], g["adapter_segments"], g["segment_indices"], g["adapter_list"])
    assert layer.get_data(meta, LM_HEAD, prefill=True, prefill_head_indices=None) == {}
    batch = AdapterBatchData.from_meta(meta, {"q_proj": layer}, {}, None, True, None)
    assert batch.data == {} and batch.max_rank == 0 and batch.ranks() == set()


def test_lora_weights_layouts_stay_resident():
    h_in, h_out = 64, 48
    for r in [8, 16]:
        a = [torch.randn(h_in, r) for _ in range(3)]
        b = [torch.randn(r, h_out) for _ in range(3)]
        w = LoraWeights(a, b, LoraConfig(r=r))
        assert w.weights_a.shape == ((3, h_in, r) if r < 16 else (3, r, h_in))
        assert w.weights_b.shape == (3, r, h_out)
        assert w.weights_a_t.shape == (3, r, h_in) and w.weights_b_t.shape == (3, h_out, r)
        ptrs = (w.weights_a.data_ptr(), w.weights_b.data_ptr(), w.weights_a_t.data_ptr(), w.weights_b_t.data_ptr())
        for _ in range(2):  # alternating prefill / decode accesses never move a stack
            assert ptrs == (w.weights_a.data_ptr(), w.weights_b.data_ptr(), w.weights_a_t.data_ptr(),
                            w.weights_b_t.data_ptr())
        assert torch.equal(w.weights_a_t[1], a[1].t()) and torch.equal(w.weights_b_t[2], b[2].t())


def test_ranks_above_128_become_rank_chunks():
    """An adapter of rank 192 is split into chunks of kernel rank (128 + 64); every chunk is a rank group of its
    own whose tables hold the chunk stacks' addresses.  The reference's layouts of the whole stack stay available
    ([L, h_in, r] for A above rank 128, orient_for_rank, punica.py:83-86)."""
    h_in, h_out, r = 64, 48, 192
    a = [torch.randn(h_in, r) for _ in range(2)]
    b = [torch.randn(r, h_out) for _ in range(2)]
    big = LoraWeights(a, b, LoraConfig(r=r))
    small = LoraWeights([torch.randn(h_in, 16)] * 2, [torch.randn(16, h_out)] * 2, LoraConfig(r=16))
    assert big.weights_a.shape == (2, h_in, r) and big.weights_b.shape == (2, r, h_out)
    chunks = big.rank_chunks()
    assert [c[2] for c in chunks] == [128, 64] and big.rank_chunks() is chunks
    assert torch.equal(chunks[1][0][1], a[1].t()[128:]) and torch.equal(chunks[1][1][0], b[0].t()[:, 128:])
    x = torch.randn(5, h_in)
    whole = x @ a[0] @ b[0]
    parts = sum((x @ ca[0].t()) @ cb[0].t() for ca, cb, _ in chunks)
    assert torch.allclose(parts, whole, atol=1e-3)

    layer = LayerAdapterWeights()
    layer.add_adapter(0, big)
    layer.add_adapter(1, small)
    assert layer.lora_entries() is None  # the native table builder leaves such a layer type to the Python path
    tokens = [0, 0, 1, 0, 1]
    for prefill in (False, True):
        meta = _meta(tokens)
        data = layer.get_data(meta, "q_proj", prefill, None)[LORA]
        assert data.use_sgmv == prefill and data.can_vectorize(SingleProcessGroup())
        assert set(data.rank_data) == {16, (192, 0), (192, 1)}
        for c, (ca, cb, rc) in enumerate(chunks):
            rs = data.rank_data[(192, c)]
            assert rs.rank == rc
            a_tab = rs.lora_a_t_ptr if prefill else rs.lora_a_ptr
            b_tab = rs.lora_b_t_ptr if prefill else rs.lora_b_ptr
            assert set(a_tab.tolist()) == {ca.data_ptr()} and set(b_tab.tolist()) == {cb.data_ptr()}
            if prefill:
                assert rs.lora_a_ptr is None and rs.segment_starts.tolist() == [0, 3] and rs.segment_ends.tolist() == [2, 4]
            else:
                assert rs.indices.tolist() == [0, 0, -1, 0, -1]
                assert sorted(rec[0] for rec in rs.plan.tolist()) == [3]


def test_from_peft_folds_scale_and_pads():
    r, h_in, h_out = 4, 32, 24
    A = [torch.randn(r, h_in)]
    B = [torch.randn(h_out, r)]
    cfg = LoraConfig(r=r, lora_alpha=8)
    w = LoraWeights.from_peft(A, B, cfg)
    assert cfg.r == 8 and w.lora_a_r == 8
    x = torch.randn(5, h_in)
    expect = (x @ A[0].t() @ B[0].t()) * 2.0
    assert torch.allclose(x @ w.weights_a[0] @ w.weights_b[0], expect, atol=1e-5)


def test_segmented_matmul():
    x = torch.randn(6, 8)
    w = [torch.randn(4, 8), torch.randn(4, 8), torch.randn(4, 8)]
    b = [torch.randn(4), None, torch.randn(4)]
    y = torch.zeros(6, 4)
    sgmv.segmented_matmul(y, x, w, b, torch.tensor([0, 3, 2], dtype=torch.int32), torch.tensor([2, 6, 2], dtype=torch.int32))
    assert torch.allclose(y[0:2], x[0:2] @ w[0].t() + b[0])
    assert torch.allclose(y[3:6], x[3:6] @ w[1].t())
    assert torch.count_nonzero(y[2]) == 0


def test_bgmv_plan_covers_every_routed_token_once():
    from lorax_amd.adapters import BGMV_PLAN_GROUP, build_bgmv_plan

    g = torch.Generator().manual_seed(3)
    slots = torch.randint(-1, 7, (203,), generator=g).tolist()
    a_addrs = [1000 + 16 * s for s in range(7)]
    b_addrs = [9000 + 16 * s for s in range(7)]
    records = build_bgmv_plan(slots, a_addrs, b_addrs)
    seen = []
    for rec in records:
        n, toks, a, b, pad = rec[0], rec[1:5], rec[5], rec[6], rec[7]
        assert 1 <= n <= BGMV_PLAN_GROUP and pad == 0 and len(rec) == 8
        s = slots[toks[0]]
        assert s >= 0 and (a, b) == (a_addrs[s], b_addrs[s])
        assert all(slots[t] == s for t in toks[:n])
        assert toks[:n] == sorted(toks[:n]) and all(t == toks[0] for t in toks[n:])
        seen.extend(toks[:n])
    assert sorted(seen) == [t for t, s in enumerate(slots) if s >= 0]
    assert build_bgmv_plan([-1, -1], a_addrs, b_addrs) == []


@pytest.mark.parametrize("case", _golden("lora_batch")["decode"])
def test_decode_rank_groups_carry_a_plan(case):
    layer = _layer(case["lora_ranks"])
    meta = _meta(case["adapter_indices"])
    data = layer.get_data(meta, LM_HEAD, prefill=False, prefill_head_indices=None).get(LORA)
    for r, rd in data.rank_data.items():
        idx = rd.indices.tolist()
        assert rd.plan.dtype == torch.int64 and rd.plan.shape[1] == 8
        covered = sorted(t for rec in rd.plan.tolist() for t in rec[1:1 + rec[0]])
        assert covered == [t for t, s in enumerate(idx) if s >= 0]
        for rec in rd.plan.tolist():
            s = idx[rec[1]]
            assert rec[5] == rd.lora_a_ptr[s].item() and rec[6] == rd.lora_b_ptr[s].item()


def test_prefill_tables_touch_only_resident_layouts():
    """Building the tables of a prefill batch must not materialise the reference's prefill layouts: the kernels
    read the resident [L, r, h_in] / [L, h_out, r] stacks; the reference-layout tables appear on first access."""
    from lorax_amd.adapters import BatchLoraWeights, LayerAdapterWeights, LoraConfig, LoraWeights
    from lorax_amd.synthetic import make_meta

    h, L = 32, 2
    layer = LayerAdapterWeights()
    for idx, r in ((0, 8), (1, 16)):
        a = [torch.randn(h, r) for _ in range(L)]
        b = [torch.randn(r, h) for _ in range(L)]
        layer.add_adapter(idx, LoraWeights(a, b, LoraConfig(r=r)))
    meta = make_meta([0, 0, 1, 1, 1, 0], torch.device("cpu"))
    data = BatchLoraWeights.load(layer.adapter_weights, meta, "q_proj", prefill=True, prefill_head_indices=None)
    lws = [layer.adapter_weights[i] for i in (0, 1)]
    assert all(lw._weights_a is None and lw._weights_b is None for lw in lws)
    for r, rd in data.rank_data.items():
        owner = lws[0] if r == 8 else lws[1]
        assert set(rd.lora_a_t_ptr.tolist()) == {owner.weights_a_t.data_ptr()}
        assert set(rd.lora_b_t_ptr.tolist()) == {owner.weights_b_t.data_ptr()}
    assert all(lw._weights_a is None and lw._weights_b is None for lw in lws)
    rd8 = data.rank_data[8]
    assert set(rd8.lora_a_ptr.tolist()) == {lws[0].weights_a.data_ptr()}  # now the [L, h_in, 8] copy exists
    assert lws[0].weights_a.shape == (L, h, 8) and lws[0].weights_a_t.shape == (L, 8, h)
    assert data.lora_b[1].shape == (L, 16, h) and lws[1]._weights_b is not None
    assert torch.equal(lws[0].weights_a.transpose(1, 2), lws[0].weights_a_t)


@pytest.mark.parametrize("config", [1, 2, 3, 4, 5, "5 with many decode tokens"])
def test_native_table_builder_matches_python_tables(config):
    """lorax_build_batch_tables (one call, one packed buffer for all layer types) against the per-layer-type Python
    restatement of BatchLoraWeights.load, which the golden vectors of the reference's test_lora.py pin."""
    from lorax_amd import synthetic
    from lorax_amd.adapters import LORA, AdapterBatchData
    from lorax_amd.segments import find_segments

    kwargs = {"num_layers": 1}
    if config in (3,):
        kwargs.update(num_segments=12, max_len=40)
    if config == 4:
        kwargs.update(num_tokens=96, num_adapters=40)
    if config == 5:
        kwargs.update(prefill_tokens=50, decode_tokens=24, num_adapters=12)
    many_short = config == "5 with many decode tokens"
    if many_short:  # enough one-row segments for the tables to list them last and to carry a plan for them
        config = 5
        kwargs.update(prefill_tokens=50, decode_tokens=70, num_adapters=12)
    w = synthetic.CONFIGS[config]("cpu", **kwargs)
    fast = AdapterBatchData.from_meta(w.meta, w.weights, prefill=w.prefill)
    assert set(fast.data) == {n for n, lw in w.weights.items() if not lw.is_empty()}
    for name, layer in w.weights.items():
        slow = layer.get_data(w.meta, name, w.prefill, None)
        if not slow:
            assert name not in fast.data
            continue
        a, b = fast.data[name][LORA], slow[LORA]
        assert a.use_sgmv == b.use_sgmv and a.layer_name == b.layer_name
        assert list(a.rank_data) == list(b.rank_data)  # ranks in order of first appearance
        assert a.adapter_index_configs.keys() == b.adapter_index_configs.keys()
        for rank in a.rank_data:
            ra, rb = a.rank_data[rank], b.rank_data[rank]
            assert ra.num_long_segments == rb.num_long_segments
            assert (ra.short_plan is not None) == many_short
            for field in ("lora_a_t_ptr", "lora_b_t_ptr", "segment_starts", "segment_ends", "indices", "plan",
                          "short_plan"):
                ta, tb = getattr(ra, field), getattr(rb, field)
                assert (ta is None) == (tb is None), field
                if ta is not None:
                    assert ta.dtype == tb.dtype and torch.equal(ta, tb), (name, rank, field)
            assert torch.equal(ra.lora_a_ptr, rb.lora_a_ptr) and torch.equal(ra.lora_b_ptr, rb.lora_b_ptr)
    bounds, owners = find_segments(w.meta.adapter_indices)
    assert w.meta.adapter_segments.tolist() == bounds and w.meta.segment_indices == owners


def test_short_segments_of_a_prefill_batch_get_a_plan():
    """A prefill batch with at least 32 segments of at most 4 rows lists them after the long segments and carries
    a routing plan over exactly their rows: every such row once, under its own adapter's stack addresses, at most
    four rows per record, the rows of one adapter together; the tables as a whole still hold every segment."""
    from lorax_amd.adapters import BatchLoraWeights, LayerAdapterWeights, LoraConfig, LoraWeights
    from lorax_amd.synthetic import make_meta

    h, L, r = 32, 1, 16
    layer = LayerAdapterWeights()
    for idx in range(6):
        layer.add_adapter(idx, LoraWeights([torch.randn(h, r)] * L, [torch.randn(r, h)] * L, LoraConfig(r=r)))
    gen = torch.Generator().manual_seed(5)
    idx = [0] * 40 + [1] * 7  # two long runs
    for _ in range(40):       # then runs of 1 to 4 rows
        a = int(torch.randint(0, 6, (1,), generator=gen))
        idx += [a] * int(torch.randint(1, 5, (1,), generator=gen))
        idx += [-1]           # separated by a row without adapter, so that equal neighbours do not merge
    meta = make_meta(idx, torch.device("cpu"))
    rd = BatchLoraWeights.load(layer.adapter_weights, meta, "q_proj", True, None).rank_data[r]
    starts, ends = rd.segment_starts.tolist(), rd.segment_ends.tolist()
    lens = [e - s for s, e in zip(starts, ends)]
    n_long = rd.num_long_segments
    assert 0 < n_long < len(lens) and rd.short_plan is not None
    assert all(n > 4 for n in lens[:n_long]) and all(1 <= n <= 4 for n in lens[n_long:])
    routed = sorted(t for s, e in zip(starts, ends) for t in range(s, e))
    assert routed == [t for t, a in enumerate(idx) if a >= 0]  # the tables as a whole are complete
    short_rows = sorted(t for s, e in zip(starts[n_long:], ends[n_long:]) for t in range(s, e))
    plan = rd.short_plan.tolist()
    seen, owners_in_order = [], []
    for n, t0, t1, t2, t3, a_addr, b_addr, zero in plan:
        assert 1 <= n <= 4 and zero == 0
        rows = [t0, t1, t2, t3][:n]
        assert [t0, t1, t2, t3][n:] == [t0] * (4 - n)  # unused slots repeat the first row
        owner = {idx[t] for t in rows}
        assert len(owner) == 1
        lw = layer.adapter_weights[owner.pop()]
        assert (a_addr, b_addr) == (lw.weights_a_t.data_ptr(), lw.weights_b_t.data_ptr())
        seen += rows
        owners_in_order.append(idx[rows[0]])
    assert sorted(seen) == short_rows and len(seen) == len(set(seen))
    runs = [a for i, a in enumerate(owners_in_order) if i == 0 or owners_in_order[i - 1] != a]
    assert len(runs) == len(set(runs))  # the records of one adapter are neighbours
    # fewer short segments than the threshold: no plan, every segment "long"
    meta = make_meta([0] * 9 + [1, -1, 2, 2, -1, 3], torch.device("cpu"))
    rd = BatchLoraWeights.load(layer.adapter_weights, meta, "q_proj", True, None).rank_data[r]
    assert rd.short_plan is None and rd.num_long_segments == rd.segment_starts.numel() == 4


@pytest.mark.parametrize("short_segments,rows,expect_plan", [(31, 4, False), (32, 4, True), (40, 5, False), (32, 1, True)])
def test_short_segment_thresholds_agree_between_the_two_builders(short_segments, rows, expect_plan):
    """The native builder and its Python restatement keep their own copies of the two thresholds (at least 32
    segments of at most 4 rows): both sides of both boundaries, compared field by field."""
    from lorax_amd.adapters import BatchLoraWeights, LayerAdapterWeights, LoraConfig, LoraWeights
    from lorax_amd.synthetic import make_meta

    h, r = 32, 8
    layer = LayerAdapterWeights()
    for idx in range(3):
        layer.add_adapter(idx, LoraWeights([torch.randn(h, r)], [torch.randn(r, h)], LoraConfig(r=r)))
    idx = [0] * 20
    for i in range(short_segments):
        idx += [1 + i % 2] * rows + [-1]
    meta = make_meta(idx, torch.device("cpu"))
    slow = BatchLoraWeights.load(layer.adapter_weights, meta, "q_proj", True, None).rank_data[r]
    fast = AdapterBatchData.from_meta(meta, {"q_proj": layer}, prefill=True).data["q_proj"][LORA].rank_data[r]
    assert (slow.short_plan is not None) == expect_plan
    assert slow.num_long_segments == fast.num_long_segments == (1 if expect_plan else short_segments + 1)
    for field in ("segment_starts", "segment_ends", "lora_a_t_ptr", "lora_b_t_ptr", "short_plan"):
        a, b = getattr(slow, field), getattr(fast, field)
        assert (a is None) == (b is None), field
        if a is not None:
            assert torch.equal(a, b), field


def test_native_table_builder_reports_the_space_it_needs():
    import ctypes

    import numpy as np

    from lorax_amd import _native

    idx = np.array([3, 3, 7, -1, 3], dtype=np.int64)
    entries = np.array([(3, 1000, 2000, 8, 0), (7, 3000, 4000, 16, 0)], dtype=_native.ENTRY_DTYPE)
    counts = np.array([2], dtype=np.int32)
    bounds, owners = np.zeros(6, dtype=np.int32), np.zeros(5, dtype=np.int64)
    nseg, ngroups, nbytes = ctypes.c_int32(), ctypes.c_int32(), ctypes.c_int64()
    f = _native.lib().lorax_build_batch_tables
    rc = f(idx.ctypes.data, 5, entries.ctypes.data, counts.ctypes.data, 1, 0, bounds.ctypes.data, owners.ctypes.data,
           ctypes.byref(nseg), None, 0, ctypes.byref(nbytes), None, 0, ctypes.byref(ngroups))
    assert rc == _native.ESPACE and ngroups.value == 2 and nbytes.value > 0
    assert bounds[: nseg.value + 1].tolist() == [0, 2, 3, 4, 5] and owners[: nseg.value].tolist() == [3, 7, -1, 3]
    b, o, packed, groups = _native.build_batch_tables(idx, entries, counts, prefill=False)
    assert packed.nbytes == nbytes.value and [g.rank for g in groups] == [8, 16]
    g8 = groups[0]
    plan = packed.view(np.int64)[g8.plan_off // 8 : g8.plan_off // 8 + 8 * g8.num_chunks].reshape(-1, 8)
    assert plan.tolist() == [[3, 0, 1, 4, 0, 1000, 2000, 0]]  # adapter 3's tokens, both runs in one chunk
    indices = packed.view(np.int64)[g8.indices_off // 8 : g8.indices_off // 8 + 5]
    assert indices.tolist() == [0, 0, -1, -1, 0]
    # prefill: segment tables instead
    _, _, packed, groups = _native.build_batch_tables(idx, entries, counts, prefill=True)
    g8 = groups[0]
    assert g8.use_sgmv == 1 and g8.num_segments == 2 and g8.plan_off == -1
    assert packed.view(np.int32)[g8.starts_off // 4 : g8.starts_off // 4 + 2].tolist() == [0, 4]
    assert packed.view(np.int32)[g8.ends_off // 4 : g8.ends_off // 4 + 2].tolist() == [2, 5]


def test_prefill_batches_beyond_the_per_token_kernels_range_stay_on_the_segment_kernels(monkeypatch):
    """The per-token kernels number rows and plan records with 16 bits.  A prefill batch whose short segments have
    a routing plan goes to them only inside that range; beyond it the segment kernels take the complete tables,
    which still list every segment (the limit is lowered here so that a small batch crosses it)."""
    from lorax_amd import _native, layers
    from lorax_amd.adapters import LORA, AdapterBatchData, BatchLoraWeights, LayerAdapterWeights, LoraConfig, LoraWeights
    from lorax_amd.synthetic import make_meta

    h, L, r = 128, 1, 32  # rank 32: outside the single-launch prefill update
    layer = LayerAdapterWeights()
    for idx in range(6):
        layer.add_adapter(idx, LoraWeights([torch.randn(h, r)] * L, [torch.randn(r, h)] * L, LoraConfig(r=r)))
    idx = [0] * 40
    for i in range(40):
        idx += [1 + i % 5] * (1 + i % 3) + [-1]
    meta = make_meta(idx, torch.device("cpu"))
    batch = BatchLoraWeights.load(layer.adapter_weights, meta, "q_proj", True, None)
    rd = batch.rank_data[r]
    assert rd.short_plan is not None and rd.num_long_segments == 1
    data = AdapterBatchData(meta=meta, data={"q_proj": {LORA: batch}}, layer_to_lora_weights={}, punica_wrapper=None,
                            prefill=True)
    calls = []
    monkeypatch.setattr(layers, "has_sgmv", lambda: True)
    monkeypatch.setattr(layers, "get_shrink_scratch", lambda device: None)
    monkeypatch.setattr(layers, "get_tmp_expand_size", lambda n: 60 * n)
    monkeypatch.setattr(_native, "sgmv_shrink_multi", lambda vs, x, tables, s, e, *a, **k: calls.append(("shrink", s.numel())))
    monkeypatch.setattr(_native, "bgmv_multi", lambda *a, **k: calls.append(("bgmv", None)))
    monkeypatch.setattr(layers, "lora_b_sgmv_cutlass_slice",
                        lambda y, v, tmp, table, s, e, *a, **k: calls.append(("expand", s.numel())))
    lin = layers.LoraLinear(None, 0)
    x = torch.zeros((len(idx), h), dtype=torch.bfloat16)
    y = torch.zeros((len(idx), h), dtype=torch.bfloat16)
    lin.forward_layer_type(y, x, data, "q_proj", 0, h)
    assert calls == [("shrink", 1), ("bgmv", None), ("expand", 1), ("bgmv", None)]  # inside the range: split
    calls.clear()
    monkeypatch.setattr(_native, "MAX_BGMV_TOKENS", len(idx) - 1)
    lin.forward_layer_type(y, x, data, "q_proj", 0, h)
    n_all = rd.segment_starts.numel()
    assert calls == [("shrink", n_all), ("expand", n_all)]  # beyond it: every segment on the segment kernels
