"""Parity at the full sizes of the benchmark configurations, where the dense oracle loop over all tokens is too
slow: (1) a random sample of rows against the fallback oracle run on just those rows; (2) rows without an
adapter bit-identical; (3) properties that hold exactly whatever the size - a token's result does not depend on
its position in the batch or on how its neighbours are grouped (permutation of a decode batch, splitting of
prefill segments), and doubling B (a power of two, exact in fp16/bf16) doubles the update exactly."""

import pytest
import torch

from lorax_amd import sgmv, synthetic
from lorax_amd.adapters import AdapterBatchData
from lorax_amd.synthetic import make_meta
from oracle import lora_oracle as O
from tests.helpers import _ulp, assert_close, ptr_table
from tests.test_gpu_layers import _run_group, assert_has_empty_segments

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _sample_rows(w, n, seed):
    gen = torch.Generator().manual_seed(seed)
    routed = [t for t, a in enumerate(w.adapter_indices) if a in w.rank_of_adapter]
    other = [t for t, a in enumerate(w.adapter_indices) if a not in w.rank_of_adapter]
    pick = [routed[i] for i in torch.randperm(len(routed), generator=gen)[:n].tolist()]
    pick += other[:8]
    return sorted(pick)


def _oracle_rows(w, group, layer_id, y0_rows, rows):
    """The fallback loop of the reference on the sampled rows only (each row's result depends on no other row)."""
    x = w.inputs[group.name][rows].cpu()
    idx = torch.tensor([w.adapter_indices[t] for t in rows])
    result = y0_rows.clone()
    off = 0
    for name, size in zip(group.layer_names, group.sizes):
        layer = w.weights[name]
        used = set(idx.tolist())
        lora_a = {a: lw.weights_a.cpu() for a, lw in layer.adapter_weights.items() if a in used}
        lora_b = {a: lw.weights_b.cpu() for a, lw in layer.adapter_weights.items() if a in used}
        O.fallback_layer_type(result, x, idx, used, lora_a, lora_b, layer_id, off, off + size)
        off += size
    return result


def _check_sampled(w, layer_id, sample=96):
    batch = w.batch_data()
    gen = torch.Generator().manual_seed(7)
    untouched = torch.tensor([a not in w.rank_of_adapter for a in w.adapter_indices])
    for group in w.groups:
        print(f"{w.name}: group {group.name} T={w.num_tokens} h_out={group.h_out}", flush=True)
        y0 = (torch.randn((w.num_tokens, group.h_out), generator=gen) * 0.25).to(w.dtype)
        out = _run_group(w, group, layer_id, y0.to(DEV), batch).cpu()
        rows = _sample_rows(w, sample, seed=len(group.name))
        ref = _oracle_rows(w, group, layer_id, y0[rows], rows)
        delta = (ref.float() - y0[rows].float()).to(w.dtype)
        assert_close(out[rows], ref, f"{w.name}/{group.name} sampled rows", rounded=[delta])
        assert torch.equal(out[untouched], y0[untouched]), "rows without an adapter must be bit-identical"
        assert torch.isfinite(out.float()).all()


def test_cfg2_full_size_sampled_rows():
    _check_sampled(synthetic.config2(DEV, num_layers=2, weights_on_device=True), 1)


def test_cfg3_full_size_sampled_rows():
    _check_sampled(synthetic.config3(DEV, num_layers=1, weights_on_device=True), 0)


def test_cfg4_full_size_sampled_rows():
    _check_sampled(synthetic.config4(DEV, num_layers=1, weights_on_device=True), 0)


def test_cfg5_full_size_sampled_rows():
    w = synthetic.config5(DEV, num_layers=1, weights_on_device=True)
    assert len(w.rank_of_adapter) == 256 and w.distinct_adapters() < 256  # all 256 adapters are resident
    assert_has_empty_segments(w, w.batch_data())
    _check_sampled(w, 0, sample=64)


@pytest.mark.parametrize("config", [2, 4])
def test_decode_result_does_not_depend_on_token_order(config):
    """Permuting the tokens of a decode batch permutes the result, bit for bit: chunks of tokens that share an
    adapter are formed differently, every token's sums are not."""
    w = synthetic.CONFIGS[config](DEV, num_layers=1, weights_on_device=True)
    gen = torch.Generator().manual_seed(3)
    perm = torch.randperm(w.num_tokens, generator=gen)
    meta_p = make_meta([w.adapter_indices[i] for i in perm.tolist()], torch.device(DEV))
    batch = w.batch_data()
    batch_p = AdapterBatchData.from_meta(meta_p, w.weights, prefill=False)
    for group in w.groups:
        print(f"{w.name}: group {group.name}", flush=True)
        y0 = (torch.randn((w.num_tokens, group.h_out), generator=gen) * 0.25).to(w.dtype).to(DEV)
        out = _run_group(w, group, 0, y0, batch)
        x_saved = w.inputs[group.name]
        w.inputs[group.name] = x_saved[perm.to(DEV)]
        try:
            out_p = _run_group(w, group, 0, y0[perm.to(DEV)], batch_p)
        finally:
            w.inputs[group.name] = x_saved
        assert torch.equal(out_p, out[perm.to(DEV)])


def test_prefill_result_does_not_depend_on_segment_cuts():
    """Cutting every segment of a prefill batch into pieces (same adapter, same rows) changes tiles and workgroups
    but not what a row is multiplied with.  The expand's sums for a row do not depend on the tile at all: with
    the same v its output is bit-identical.  The shrink adds a row's 128-element partial sums in an order that
    depends on the tile (every tile starts its walk over the hidden dimension somewhere else), so v may differ
    by the last rounding: every element equal or on neighbouring values of the output type, and few of them.
    Both runs pass tables of the same size (the uncut one padded with empty segments), because the number of K
    parts of a launch is chosen from the table size."""
    w = synthetic.config3(DEV, num_layers=1, weights_on_device=True, num_segments=16, max_len=1200)
    group = w.groups[0]  # gate_up: 4096 -> 2 x 14336
    name = group.layer_names[0]
    rd = w.batch_data().data[name]["lora"].rank_data[64]
    x = w.inputs[group.name]
    starts, ends = rd.segment_starts.tolist(), rd.segment_ends.tolist()
    a_ptr, b_ptr = rd.lora_a_t_ptr.tolist(), rd.lora_b_t_ptr.tolist()
    cut_s, cut_e, cut_a, cut_b = [], [], [], []
    for s, e, a, b in zip(starts, ends, a_ptr, b_ptr):
        pieces = sorted({s, e, s + (e - s) // 3, s + 1 if e - s > 1 else s, e - 5 if e - s > 5 else s})
        for p, q in zip(pieces[:-1], pieces[1:]):
            cut_s.append(p), cut_e.append(q), cut_a.append(a), cut_b.append(b)
    assert len(cut_s) > 2 * len(starts)

    def run(s_list, e_list, a_list, b_list, v=None):
        s_t = torch.tensor(s_list, dtype=torch.int32, device=DEV)
        e_t = torch.tensor(e_list, dtype=torch.int32, device=DEV)
        a_t = torch.tensor(a_list, dtype=torch.int64, device=DEV)
        b_t = torch.tensor(b_list, dtype=torch.int64, device=DEV)
        if v is None:
            v = sgmv.lora_a_sgmv_resident(x, sgmv.get_tmp_tensor(torch.device(DEV)), a_t, s_t, e_t, 0, 64)
        y = torch.zeros((x.size(0), group.sizes[0]), dtype=x.dtype, device=DEV)
        tmp = sgmv.get_tmp_tensor_for_size(len(s_list), torch.device(DEV))
        sgmv.lora_b_sgmv_cutlass_slice(y, v, tmp, b_t, s_t, e_t, 0, 0, group.sizes[0], transposed=True)
        return v, y

    pad = len(cut_s) - len(starts)
    v1, y1 = run(starts + [0] * pad, ends + [0] * pad, a_ptr + [0] * pad, b_ptr + [0] * pad)
    v2, _ = run(cut_s, cut_e, cut_a, cut_b)
    _, y2 = run(cut_s, cut_e, cut_a, cut_b, v=v1)
    assert torch.equal(y1, y2)
    assert torch.count_nonzero(y1) > 0
    differ = v1 != v2
    assert differ.float().mean().item() < 0.02, differ.float().mean().item()
    # the two fp32 sums of an element differ by summation order only (a few 1e-6 for sums of this size), so the
    # rounded values are equal or one spacing of the output type apart; next to zero, where the spacing is
    # finer than that, the fp32 difference itself shows
    gap = (v1.double() - v2.double()).abs().cpu()
    assert torch.all(gap <= _ulp(v1.double().cpu(), v1.dtype) * 1.0001 + 2e-5), gap.max().item()


@pytest.mark.parametrize("config", [2, 3])
def test_doubling_b_doubles_the_update(config):
    """B -> 2B is exact in bf16, so the update (y0 = 0) doubles bit for bit, in decode and in prefill."""
    kwargs = {"num_layers": 1, "weights_on_device": True}
    if config == 3:
        kwargs.update(num_segments=12, max_len=600)
    w = synthetic.CONFIGS[config](DEV, **kwargs)
    group = w.groups[-1]
    zeros = torch.zeros((w.num_tokens, group.h_out), dtype=w.dtype, device=DEV)
    out1 = _run_group(w, group, 0, zeros, w.batch_data())
    for name in group.layer_names:
        for lw in w.weights[name].adapter_weights.values():
            lw.weights_b_t.mul_(2.0)
            if lw._weights_b is not None:
                lw._weights_b.mul_(2.0)
    out2 = _run_group(w, group, 0, zeros, w.batch_data())
    assert torch.count_nonzero(out1) > 0
    assert torch.equal(out2, out1 * 2)
