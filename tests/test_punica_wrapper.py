"""Host logic of the stacked-weight path: run-length metadata, index shifting, segment bounds and the
stacking of preloaded adapters.  No kernel runs here.

The reference holds no test or fixture for this path (lorax_server/utils/punica.py:256-793, utils/ops/*):
the expected values below are worked out by hand from its code, and the GPU tests check the operators
against the same oracle functions as the pointer-table path (tests/test_gpu_punica_wrapper.py)."""

import torch

from lorax_amd import ops
from lorax_amd.adapters import LayerAdapterWeights, LoraConfig, LoraWeights, stack_preloaded_adapters
from lorax_amd.punica_wrapper import PunicaWrapper, compute_meta
from lorax_amd.synthetic import make_meta


def test_compute_meta_merges_neighbours_with_the_same_adapter():
    tokens = torch.tensor([-1, -1, 0, 0, 0, 2, -1, 2, 2])
    starts, lengths, idx, batches, longest, no_lora = compute_meta(tokens)
    assert starts.tolist() == [0, 2, 5, 6, 7]
    assert lengths.tolist() == [2, 3, 1, 1, 2]
    assert idx.tolist() == [-1, 0, 2, -1, 2]
    assert (batches, longest, no_lora) == (5, 3, False)
    assert compute_meta(torch.tensor([-1, -1, -1]))[3:] == (1, 3, True)
    assert compute_meta(torch.tensor([4, 4]))[3:] == (1, 2, False)


def test_segment_bounds_empty_for_sequences_without_adapter():
    starts, lengths, idx, *_ = compute_meta(torch.tensor([-1, -1, 0, 0, 0, 2, -1, 2, 2]))
    s, e = ops.segment_bounds(starts, lengths, idx)
    assert s.dtype == e.dtype == torch.int32
    assert s.tolist() == [0, 2, 5, 6, 7] and e.tolist() == [0, 5, 6, 6, 9]


def test_update_metadata_shifts_adapter_indices_by_the_base_model_slot():
    wrapper = PunicaWrapper(max_num_batched_tokens=16, max_batches=8, device="cpu", enabled=True)
    meta = make_meta([0, 0, 1, 1, 3, 0], torch.device("cpu"))  # adapter index 0 = base model
    wrapper.update_metadata(meta, prefill=True)
    assert wrapper.is_prefill and not wrapper.no_lora
    assert wrapper.token_lora_indices.tolist() == [-1, -1, 0, 0, 2, -1]
    starts, lengths, idx, batches, longest = wrapper.prefill_metadata
    assert (starts.tolist(), lengths.tolist(), idx.tolist(), batches, longest) == ([0, 2, 4, 5], [2, 2, 1, 1],
                                                                                   [-1, 0, 2, -1], 4, 2)
    s, e = wrapper._kernel_bounds
    assert s.tolist() == [0, 2, 4, 5] and e.tolist() == [0, 4, 5, 5]
    wrapper.update_metadata(make_meta([2, 0, 1], torch.device("cpu")), prefill=False)
    assert not wrapper.is_prefill and wrapper.token_lora_indices.tolist() == [1, -1, 0]
    wrapper.update_metadata(make_meta([0, 0], torch.device("cpu")), prefill=True)
    assert wrapper.no_lora and wrapper.batch_size == 1


def test_stack_preloaded_adapters_pads_to_the_largest_rank():
    h_in, h_out, L = 32, 48, 2
    layer = LayerAdapterWeights()
    gen = torch.Generator().manual_seed(0)
    for idx, r in ((1, 8), (2, 16), (3, 8)):
        a = [torch.randn((h_in, r), generator=gen) for _ in range(L)]
        b = [torch.randn((r, h_out), generator=gen) for _ in range(L)]
        layer.add_adapter(idx, LoraWeights(a, b, LoraConfig(r=r)))
    stacks = stack_preloaded_adapters({"q_proj": layer}, [1, 2, 3])
    assert set(stacks) == {("q_proj", 0), ("q_proj", 1)}
    lora_a, lora_b = stacks[("q_proj", 1)]
    assert lora_a.shape == (3, 16, h_in) and lora_b.shape == (3, h_out, 16)
    assert lora_a.is_contiguous() and lora_b.is_contiguous()
    w1 = layer.adapter_weights[1]
    assert torch.equal(lora_a[0, :8], w1.weights_a_t[1]) and torch.count_nonzero(lora_a[0, 8:]) == 0
    assert torch.equal(lora_b[0, :, :8], w1.weights_b_t[1]) and torch.count_nonzero(lora_b[0, :, 8:]) == 0
    assert torch.equal(lora_a[1], layer.adapter_weights[2].weights_a_t[1])
    # zero padding leaves the product unchanged
    x = torch.randn((5, h_in), generator=gen)
    assert torch.allclose(x @ lora_a[0].t() @ lora_b[0].t(), x @ w1.weights_a_t[1].t() @ w1.weights_b_t[1].t(), atol=1e-5)


def test_stack_table_addresses_every_entry():
    w = torch.zeros((5, 8, 32), dtype=torch.bfloat16)
    table = ops.stack_table(w)
    assert table.dtype == torch.int64
    assert table.tolist() == [w.data_ptr() + i * 8 * 32 * 2 for i in range(5)]
    assert ops.stack_table(w) is table  # cached per weight tensor


def test_run_table_taken_from_the_batch_equals_the_one_computed_from_the_tokens():
    """update_metadata reuses adapter_segments / segment_indices when the metadata carries them; a metadata object
    with only per-token indices goes through _update_prefill_metada.  Both give the same state."""
    from types import SimpleNamespace

    tokens = [2, 2, 0, 0, 0, 5, 2, 2, 0]
    full = make_meta(tokens, torch.device("cpu"))
    bare = SimpleNamespace(adapter_indices=full.adapter_indices)
    a = PunicaWrapper(max_num_batched_tokens=16, max_batches=8, device="cpu", enabled=True)
    b = PunicaWrapper(max_num_batched_tokens=16, max_batches=8, device="cpu", enabled=True)
    a.update_metadata(full, prefill=True)
    b.update_metadata(bare, prefill=True)
    for x, y in zip(a.prefill_metadata, b.prefill_metadata):
        assert (x.tolist() == y.tolist()) if isinstance(x, torch.Tensor) else x == y
    assert a.prefill_metadata[3:] == (5, 3) and a.no_lora == b.no_lora is False
    assert [t.tolist() for t in a._kernel_bounds] == [t.tolist() for t in b._kernel_bounds] == [[0, 2, 5, 6, 8],
                                                                                               [2, 2, 6, 8, 8]]
    # a batch of base-model tokens only: nothing is routed
    for w, m in ((a, make_meta([0, 0, 0], torch.device("cpu"))),
                 (b, SimpleNamespace(adapter_indices=torch.tensor([0, 0, 0])))):
        w.update_metadata(m, prefill=True)
        assert w.no_lora and w.batch_size == 1
