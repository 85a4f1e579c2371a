"""The stacked-weight operators (lorax_amd.ops) and PunicaWrapper.add_lora on the GPU against the oracle.

The reference has no numerics test for this path; what is checked is its documented semantics
(lorax_server/utils/punica.py:710-718: y[i] += x[i] @ A[idx[i]].T @ B[idx[i]].T * scale) through the same
oracle functions that pin the pointer-table path, with the intermediate rounded to the weight type where
the reference's expand operators round it (CAST_TYPE)."""

import pytest
import torch

from lorax_amd import ops
from lorax_amd.adapters import AdapterBatchData, LayerAdapterWeights, LoraConfig, LoraWeights, stack_preloaded_adapters
from lorax_amd.layers import TensorParallelMultiAdapterLinear
from lorax_amd.punica_wrapper import PunicaWrapper, compute_meta
from lorax_amd.synthetic import make_meta
from oracle import lora_oracle as O
from tests.helpers import assert_close, randn

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _stacks(n, r, h_in, h_out, gen, dtype):
    a = randn((n, r, h_in), 0.03, gen, dtype, DEV)
    b = randn((n, 1, h_out, r), 0.03, gen, dtype, DEV)  # the optional singleton dimension
    return a, b


def _ref_lora(y0, x, a, b, token_idx, scale, off, width, dtype):
    """y[t, off:off+width] += T(T(scale * x[t] @ A[i].T) @ B[i].T), fp32 sums, i = token_idx[t] >= 0."""
    y = y0.clone()
    a, b = a.cpu(), b.cpu().squeeze(1)
    for t, i in enumerate(token_idx):
        if i < 0:
            continue
        v = ((x[t].float() @ a[i].float().t()) * scale).to(dtype)
        delta = (v.float() @ b[i].float().t()).to(dtype)
        y[t, off:off + width] = (y[t, off:off + width].float() + delta.float()).to(dtype)
    return y


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("r", [8, 16, 64])
@pytest.mark.parametrize("buffer_dtype", ["input", "fp32"])
def test_bgmv_operators(dtype, r, buffer_dtype):
    print(f"case dtype={dtype} r={r} buffer={buffer_dtype}", flush=True)
    gen = torch.Generator().manual_seed(r)
    T, h_in, h_out, n = 37, 1024, 1160, 5
    a, b = _stacks(n, r, h_in, h_out, gen, dtype)
    x = randn((T, h_in), 1.0, gen, dtype, DEV)
    y0 = randn((T, h_out + 64), 0.5, gen, dtype, DEV)
    idx = torch.randint(-1, n, (T,), generator=gen)
    buf = torch.zeros((T, r), dtype=dtype if buffer_dtype == "input" else torch.float32, device=DEV)
    ops.bgmv_shrink(x, a, buf, idx.to(DEV), 0.5)
    v_ref = torch.zeros((T, r), dtype=dtype)
    for t, i in enumerate(idx.tolist()):
        if i >= 0:
            v_ref[t] = ((x[t].cpu().float() @ a[i].cpu().float().t()) * 0.5).to(dtype)
    assert_close(buf.to(dtype), v_ref, "bgmv_shrink")
    y = y0.clone()
    ops.bgmv_expand_slice(buf, b, y, idx.to(DEV), 64, h_out, add_inputs=True)
    y_ref = _ref_lora(y0.cpu(), x.cpu(), a, b, idx.tolist(), 0.5, 64, h_out, dtype)
    assert_close(y, y_ref, "bgmv_expand_slice", rounded=[(y_ref.float() - y0.cpu().float()).to(dtype)])
    assert torch.equal(y.cpu()[:, :64], y0.cpu()[:, :64])
    # add_inputs=False: rows with an adapter are overwritten, the others untouched
    y2 = y0[:, 64:].contiguous()
    ops.bgmv_expand(buf, b, y2, idx.to(DEV), add_inputs=False)
    delta_ref = _ref_lora(torch.zeros((T, h_out), dtype=dtype), x.cpu(), a, b, idx.tolist(), 0.5, 0, h_out, dtype)
    routed = idx >= 0
    assert_close(y2.cpu()[routed], delta_ref[routed], "bgmv_expand overwrite")
    assert torch.equal(y2.cpu()[~routed], y0.cpu()[:, 64:][~routed])


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("r", [8, 16, 64])
@pytest.mark.parametrize("buffer_dtype", ["input", "fp32"])
def test_sgmv_operators(dtype, r, buffer_dtype):
    print(f"case dtype={dtype} r={r} buffer={buffer_dtype}", flush=True)
    gen = torch.Generator().manual_seed(100 + r)
    h_in, h_out, n = 1024, 1160, 4
    token_idx = [-1] * 3 + [0] * 70 + [2] * 1 + [-1] * 2 + [1] * 300 + [2] * 17 + [3] * 5
    T = len(token_idx)
    a, b = _stacks(n, r, h_in, h_out, gen, dtype)
    x = randn((T, h_in), 1.0, gen, dtype, DEV)
    y0 = randn((T, h_out + 64), 0.5, gen, dtype, DEV)
    starts, lengths, seq_idx, batches, longest, _ = compute_meta(torch.tensor(token_idx, device=DEV))
    buf = torch.zeros((T, r), dtype=dtype if buffer_dtype == "input" else torch.float32, device=DEV)
    ops.sgmv_shrink(x, a, buf, starts, lengths, seq_idx, batches, longest, 2.0)
    y = y0.clone()
    ops.sgmv_expand_slice(buf, b, y, starts, lengths, seq_idx, batches, longest, 64, h_out, add_inputs=True)
    y_ref = _ref_lora(y0.cpu(), x.cpu(), a, b, token_idx, 2.0, 64, h_out, dtype)
    assert_close(y, y_ref, "sgmv shrink + expand_slice", rounded=[(y_ref.float() - y0.cpu().float()).to(dtype)])
    assert torch.equal(y.cpu()[:, :64], y0.cpu()[:, :64])
    y2 = y0[:, 64:].contiguous()
    ops.sgmv_expand(buf, b, y2, starts, lengths, seq_idx, batches, longest)  # add_inputs defaults to False
    delta_ref = _ref_lora(torch.zeros((T, h_out), dtype=dtype), x.cpu(), a, b, token_idx, 2.0, 0, h_out, dtype)
    routed = torch.tensor(token_idx) >= 0
    assert_close(y2.cpu()[routed], delta_ref[routed], "sgmv_expand overwrite")
    assert torch.equal(y2.cpu()[~routed], y0.cpu()[:, 64:][~routed])


def _layer_with_adapters(ranks, h_in, sizes, L, gen, dtype):
    layers = {}
    names = ["q_proj", "k_proj", "v_proj"][: len(sizes)]
    for name, h_out in zip(names, sizes):
        layer = LayerAdapterWeights()
        for idx, r in ranks.items():
            a = [randn((h_in, r), 0.03, gen, dtype, DEV) for _ in range(L)]
            b = [randn((r, h_out), 0.03, gen, dtype, DEV) for _ in range(L)]
            layer.add_adapter(idx, LoraWeights(a, b, LoraConfig(r=r)))
        layers[name] = layer
    return names, layers


@pytest.mark.parametrize("prefill", [False, True])
def test_add_lora_through_the_layer_matches_the_pointer_table_path(prefill):
    """LoraLinear with a PunicaWrapper and stacked weights of preloaded adapters (ranks 8 and 16 padded to 16)
    against the fallback oracle and against the same layer without the wrapper."""
    print(f"case prefill={prefill}", flush=True)
    dtype, h_in, sizes, L = torch.bfloat16, 1024, [1024, 256, 256], 2
    gen = torch.Generator().manual_seed(5)
    ranks = {1: 8, 2: 16, 3: 8}  # adapter index 0 is the base model
    names, layers = _layer_with_adapters(ranks, h_in, sizes, L, gen, dtype)
    token_adapters = [0, 0, 1, 1, 1, 2, 0, 3, 3, 2, 2, 2] * 3
    meta = make_meta(token_adapters, torch.device(DEV))
    T = len(token_adapters)
    x = randn((T, h_in), 1.0, gen, dtype, DEV)
    y0 = randn((T, sum(sizes)), 0.5, gen, dtype, DEV)
    stacks = stack_preloaded_adapters(layers, [1, 2, 3], DEV)
    wrapper = PunicaWrapper(max_num_batched_tokens=64, max_batches=64, device=DEV, enabled=True)
    wrapper.update_metadata(meta, prefill)

    class Base(torch.nn.Module):
        def forward(self, inp):
            return y0.clone()

    layer_id = 1
    layer = TensorParallelMultiAdapterLinear.load(Base(), layer_id, names, sizes)
    with_wrapper = AdapterBatchData.from_meta(meta, layers, stacks, wrapper, prefill=prefill)
    plain = AdapterBatchData.from_meta(meta, layers, prefill=prefill)
    out_wrapper = layer(x, with_wrapper)
    out_plain = layer(x, plain)
    torch.cuda.synchronize()
    ref = y0.cpu().clone()
    idx = torch.tensor(token_adapters)
    off = 0
    for name, size in zip(names, sizes):
        lora_a = {a: lw.weights_a.cpu() for a, lw in layers[name].adapter_weights.items()}
        lora_b = {a: lw.weights_b.cpu() for a, lw in layers[name].adapter_weights.items()}
        O.fallback_layer_type(ref, x.cpu(), idx, set(token_adapters), lora_a, lora_b, layer_id, off, off + size)
        off += size
    delta = (ref.float() - y0.cpu().float()).to(dtype)
    assert_close(out_wrapper, ref, "stacked-weight path", rounded=[delta])
    assert_close(out_plain, ref, "pointer-table path", rounded=[delta])
    base_rows = idx == 0
    assert torch.equal(out_wrapper.cpu()[base_rows], y0.cpu()[base_rows])


@pytest.mark.parametrize("prefill", [False, True])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("ranks,repeat", [((8, 16, 64), 1), ((16, 16, 16), 1), ((32, 32, 32), 16)])
def test_add_lora_packed_nslice(prefill, dtype, ranks, repeat):
    """PunicaWrapper.add_lora_packed_nslice (punica.py:750-773) over three slices: in decode the shrinks are one
    launch and the expands another; in prefill slices of one rank shrink together (one launch over the stacked
    A matrices once the batch has more than 512 rows); the result is add_lora slice by slice."""
    print(f"case prefill={prefill} dtype={dtype} ranks={ranks} repeat={repeat}", flush=True)
    gen = torch.Generator().manual_seed(17)
    h_in, sizes, n = 1024, (1024, 264, 256), 4
    token_idx = ([-1] * 2 + [0] * 9 + [2] * 1 + [-1] * 1 + [1] * 20 + [2] * 3 + [3] * 5) * repeat
    T = len(token_idx)
    stacks = [_stacks(n, r, h_in, h_out, gen, dtype) for r, h_out in zip(ranks, sizes)]
    x = randn((T, h_in), 1.0, gen, dtype, DEV)
    y0 = randn((T, sum(sizes)), 0.5, gen, dtype, DEV)
    wrapper = PunicaWrapper(max_num_batched_tokens=1024, max_batches=256, device=DEV, enabled=True)
    # token_adapters of the batch: adapter index i + 1 is stack entry i, index 0 is the base model
    wrapper.update_metadata(make_meta([i + 1 for i in token_idx], torch.device(DEV)), prefill)
    assert wrapper.token_lora_indices.tolist() == token_idx
    y = y0.clone()
    wrapper.add_lora_packed_nslice(y, x, tuple(a for a, _ in stacks), tuple(b for _, b in stacks), 0.5, sizes)
    y_each = y0.clone()
    off = 0
    for (a, b), size in zip(stacks, sizes):
        wrapper.add_lora(y_each, x, a, b, 0.5, off, size)
        off += size
    torch.cuda.synchronize()
    y_ref, off = y0.cpu(), 0
    for (a, b), size in zip(stacks, sizes):
        y_ref = _ref_lora(y_ref, x.cpu(), a, b, token_idx, 0.5, off, size, dtype)
        off += size
    assert_close(y, y_ref, "add_lora_packed_nslice", rounded=[(y_ref.float() - y0.cpu().float()).to(dtype)])
    if prefill:  # the grouped shrink sums in another order than a projection's own launch
        assert_close(y, y_each.cpu(), "grouped against slice by slice", rounded=[(y_ref.float() - y0.cpu().float()).to(dtype)])
    else:
        assert torch.equal(y.cpu(), y_each.cpu())  # same kernels, same arithmetic, one launch or three
    routed = torch.tensor(token_idx) >= 0
    assert torch.equal(y.cpu()[~routed], y0.cpu()[~routed])


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("ranks,widths", [
    ((8, 8, 8), (4096, 1024, 1024)),   # q/k/v at rank 8: shrink and expand in one launch
    ((16, 16), (2048, 2048)),          # rank 16
    ((8, 16, 8), (1024, 512, 512)),    # mixed 8 and 16: one launch per rank
    ((32, 64, 8), (1024, 1024, 1024)),  # ranks beyond the single launch: two planned launches
])
def test_decode_with_a_slot_plan_equals_the_scanning_launches(dtype, ranks, widths):
    """ops.bgmv_lora_slices with the batch's routing plan over stack entries (ops.build_slot_plan) against the same
    call without it, bit for bit, and against the documented formula; PunicaWrapper.update_metadata builds the
    plan and add_lora_slices uses it."""
    print(f"case dtype={dtype} ranks={ranks} widths={widths}", flush=True)
    gen = torch.Generator().manual_seed(sum(ranks))
    T, h_in, n = 61, 4096, 7
    x = randn((T, h_in), 1.0, gen, dtype, DEV)
    total = sum(widths)
    y0 = randn((T, total), 0.5, gen, dtype, DEV)
    idx = torch.randint(-1, n, (T,), generator=gen)
    idx[:9] = 3  # more than two chunks of one adapter
    slices, off = [], 0
    for r, w in zip(ranks, widths):
        a, b = _stacks(n, r, h_in, w, gen, dtype)
        slices.append((a, b, off, w))
        off += w
    plan_host = ops.build_slot_plan(idx.numpy())
    # every routed token once, at most four per record, one entry per record
    seen = []
    for count, t0, t1, t2, t3, ea, eb, zero in plan_host.tolist():
        rows = [t0, t1, t2, t3][:count]
        assert 1 <= count <= 4 and ea == eb and zero == 0 and {int(idx[t]) for t in rows} == {ea}
        seen += rows
    assert sorted(seen) == [t for t in range(T) if idx[t] >= 0]
    plan = plan_host.to(DEV)
    y_scan, y_plan = y0.clone(), y0.clone()
    ops.bgmv_lora_slices(x, slices, y_scan, idx.to(DEV), 1.0)
    ops.bgmv_lora_slices(x, slices, y_plan, idx.to(DEV), 1.0, plan=plan)
    torch.cuda.synchronize()
    assert torch.equal(y_scan, y_plan)
    y_ref = y0.cpu()
    for a, b, first, w in slices:
        y_ref = _ref_lora(y_ref, x.cpu(), a, b, idx.tolist(), 1.0, first, w, dtype)
    assert_close(y_plan, y_ref, "planned decode", rounded=[(y_ref.float() - y0.cpu().float()).to(dtype)])
    untouched = idx < 0
    assert torch.equal(y_plan.cpu()[untouched], y0.cpu()[untouched])
    # a scale other than 1 keeps the two-launch arithmetic (planned launches, same bits as the scanning ones)
    y_a, y_b = y0.clone(), y0.clone()
    ops.bgmv_lora_slices(x, slices, y_a, idx.to(DEV), 0.5)
    ops.bgmv_lora_slices(x, slices, y_b, idx.to(DEV), 0.5, plan=plan)
    assert torch.equal(y_a, y_b)
    # through the wrapper: adapter 0 is the base model, entry i belongs to adapter i + 1
    wrapper = PunicaWrapper(256, 64, DEV, enabled=True)
    wrapper.update_metadata(make_meta((idx + 1).tolist(), torch.device(DEV)), prefill=False)
    assert wrapper._plan_records == plan_host.size(0)
    y_w = y0.clone()
    wrapper.add_lora_slices(y_w, x, slices, 1.0)
    torch.cuda.synchronize()
    assert torch.equal(y_w, y_plan)


def test_slot_plan_buffer_is_padded_with_skipped_records():
    """The wrapper keeps its routing plan in one fixed buffer: after a smaller batch the records of the batch
    before are zeroed, so a launch that reads a fixed number of records (a captured step) sees padding, which the
    kernels skip, and gives the smaller batch's result."""
    dtype, h_in, w, r, n = torch.bfloat16, 1024, 1024, 8, 5
    gen = torch.Generator().manual_seed(3)
    a, b = _stacks(n, r, h_in, w, gen, dtype)
    wrapper = PunicaWrapper(128, 128, DEV, enabled=True)
    big = torch.randint(0, n, (90,), generator=gen)
    wrapper.update_metadata(make_meta((big + 1).tolist(), torch.device(DEV)), prefill=False)
    first = wrapper._plan_records
    small = torch.randint(-1, n, (23,), generator=gen)
    wrapper.update_metadata(make_meta((small + 1).tolist(), torch.device(DEV)), prefill=False)
    assert wrapper._plan_records < first
    assert torch.count_nonzero(wrapper._plan[wrapper._plan_records:first]) == 0
    x = randn((23, h_in), 1.0, gen, dtype, DEV)
    y_fixed = torch.zeros((23, w), dtype=dtype, device=DEV)
    ops.bgmv_lora_slices(x, [(a, b, 0, w)], y_fixed, small.to(DEV), 1.0, plan=wrapper._plan[:first])  # with the padding
    y_ref = torch.zeros((23, w), dtype=dtype, device=DEV)
    ops.bgmv_lora_slices(x, [(a, b, 0, w)], y_ref, small.to(DEV), 1.0)
    torch.cuda.synchronize()
    assert torch.equal(y_fixed, y_ref) and torch.count_nonzero(y_ref) > 0
