"""Row-tile plans built on the host (lorax_sgmv_plan_tiles, lorax_build_batch_tables) against the kernels' own
search of the segment tables on the device: the same launches with and without a plan.

The expand's result does not depend on the tiling at all (every element of the update is one dot product over r),
so planned and unplanned launches agree bit for bit.  The shrink adds its sums over the hidden dimension in an
order that depends on the tile, so the two agree bit for bit in fixed-order mode (lorax_set_fixed_order_shrink) and
to one spacing of the output type on a few percent of the elements otherwise (sums that cancel to nearly zero
differ by the fp32 reordering error instead); both are checked against the oracle
formula (per segment x[s:e] @ A_i^T, test_sgmv.py:16-39)."""

import pytest
import torch

from lorax_amd import _native, sgmv
from tests.helpers import assert_close, ptr_table, randn

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _tables(lens, gap):
    starts, ends, pos = [], [], 1
    for n in lens:
        starts.append(pos)
        ends.append(pos + max(n, 0))
        pos += max(n, 0) + gap
    return starts, ends, pos + 2


def _plan(starts, ends, T, kind):
    records, tile_rows = _native.plan_tiles(starts, ends, T, kind)
    return _native.TilePlan(torch.from_numpy(records.copy()).to(DEV), tile_rows)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("r,h_out,lens", [
    (64, 1536, [700, 0, 41, 269, 1, 256, 3]),   # remainders that merge and that do not, an empty segment
    (128, 1024, [1500]),                        # one long run
    (16, 4096, [5] * 40 + [300]),               # many short segments
    (24, 2752, [513, 17]),                      # a rank and a width that are not powers of two
    (32, 512, [9, 300] * 50),                   # a hundred segments: table entries past the first 64
])
def test_expand_with_a_plan_is_bit_identical(dtype, r, h_out, lens):
    print(f"case dtype={dtype} r={r} h_out={h_out} lens={lens}", flush=True)
    gen = torch.Generator().manual_seed(r + h_out)
    starts, ends, T = _tables(lens, gap=1)
    layer = 1
    v = randn((T, r), 1.0, gen, dtype, DEV)
    y0 = randn((T, h_out + 64), 0.5, gen, dtype, DEV)
    bt = [randn((2, h_out, r), 0.05, gen, dtype, DEV) if n > 0 else None for n in lens]
    table = ptr_table(bt, DEV)
    s_start = torch.tensor(starts, dtype=torch.int32, device=DEV)
    s_end = torch.tensor(ends, dtype=torch.int32, device=DEV)
    tmp = sgmv.get_tmp_tensor_for_size(len(lens), torch.device(DEV))
    plan = _plan(starts, ends, T, _native.TILES_EXPAND)
    assert plan.num_tiles >= sum(1 for n in lens if n > 0)
    for accumulate in (True, False):
        y_a, y_b = y0.clone(), y0.clone()
        _native.sgmv_expand(y_a, v, table, s_start, s_end, tmp, layer, 64, h_out, True, accumulate)
        _native.sgmv_expand(y_b, v, table, s_start, s_end, tmp, layer, 64, h_out, True, accumulate, plan)
        torch.cuda.synchronize()
        assert torch.equal(y_a, y_b), f"accumulate={accumulate}"
    want = y0.cpu().clone()
    for i, (s, e) in enumerate(zip(starts, ends)):
        if e > s:
            delta = v.cpu()[s:e] @ bt[i][layer].cpu().t()
            want[s:e, 64:] = delta  # the last call overwrote
    assert_close(y_b, want, "planned expand")
    assert torch.equal(y_b[:, :64], y0[:, :64])


@pytest.mark.parametrize("count,r,h_in,lens", [
    (1, 64, 2048, [700, 0, 41, 269, 1, 256, 3]),   # about 1300 rows: low tiles, K cut into parts
    (2, 64, 1024, [3000, 900, 2500, 77]),          # stacked rank 128, several thousand rows: 48- or 64-row tiles
    (1, 128, 4096, [4096]),                        # one long run at rank 128
    (1, 40, 1536, [33] * 30),                      # a rank that is not a multiple of 16
    (3, 16, 512, [9000]),                          # many tiles: more than one round over the CUs
    (2, 32, 1024, [70, 7] * 50),                   # a hundred segments: table entries past the first 64
])
def test_shrink_with_a_plan(count, r, h_in, lens):
    print(f"case count={count} r={r} h_in={h_in} lens={lens}", flush=True)
    dtype = torch.bfloat16
    gen = torch.Generator().manual_seed(count + r + h_in)
    starts, ends, T = _tables(lens, gap=2)
    layer = 1
    x = randn((T, h_in), 1.0, gen, dtype, DEV)
    stacks = [[randn((2, r, h_in), 0.05, gen, dtype, DEV) if n > 0 else None for n in lens] for _ in range(count)]
    tables = [ptr_table(ws, DEV) for ws in stacks]
    s_start = torch.tensor(starts, dtype=torch.int32, device=DEV)
    s_end = torch.tensor(ends, dtype=torch.int32, device=DEV)
    tmp = sgmv.get_tmp_tensor(torch.device(DEV))
    plan = _plan(starts, ends, T, _native.TILES_SHRINK)
    covered = torch.zeros(T, dtype=torch.bool)
    for s, e in zip(starts, ends):
        covered[s:e] = True

    def run(tiles):
        vs = [torch.full((T, r), 7.0, dtype=dtype, device=DEV) for _ in range(count)]
        _native.sgmv_shrink_multi(vs, x, tables, s_start, s_end, tmp, layer, 1.0, False, tiles)
        torch.cuda.synchronize()
        return vs

    searched, planned = run(None), run(plan)
    previous = _native.set_fixed_order_shrink(True)
    try:
        searched_fixed, planned_fixed = run(None), run(plan)
    finally:
        _native.set_fixed_order_shrink(previous)
    for p in range(count):
        want = torch.full((T, r), 7.0, dtype=dtype)
        for i, (s, e) in enumerate(zip(starts, ends)):
            if e > s:
                want[s:e] = x.cpu()[s:e] @ stacks[p][i][layer].cpu().t()
        for name, got in (("searched", searched), ("planned", planned), ("planned, fixed order", planned_fixed)):
            assert_close(got[p], want, f"{name}, projection {p}", rounded=[want])
            assert torch.all(got[p].cpu()[~covered] == 7.0), f"{name}: rows outside the segments were written"
        assert torch.equal(searched_fixed[p], planned_fixed[p]), f"fixed order, projection {p}"
        # default mode: the same sums in another order - neighbouring values of the output type on a few elements
        a, b = searched[p].float().cpu(), planned[p].float().cpu()
        differ = a != b
        assert differ.float().mean().item() <= 0.05, f"projection {p}: {differ.float().mean().item():.3%} of v differ"
        spacing = torch.exp2(torch.floor(torch.log2(torch.maximum(a.abs(), b.abs()).clamp_min(2.0 ** -14))) - 7)
        # (values near zero - cancelled sums - carry the fp32 sums' own reordering error, far below the spacing of
        # the terms: an absolute floor for those)
        assert torch.all((a - b).abs()[differ] <= torch.clamp(1.0001 * spacing[differ], min=1e-4))


def test_batch_tables_carry_tile_plans_that_the_layer_uses():
    """The native table builder emits both plans for every prefill rank group; a layer run with them equals a run
    without (expand bit for bit; the shrink's v to one spacing, so y within the parity tolerance)."""
    from lorax_amd import synthetic
    from lorax_amd.adapters import LORA
    from lorax_amd.layers import TensorParallelMultiAdapterLinear

    w = synthetic.config3(DEV, num_layers=1, weights_on_device=True, num_segments=12, min_len=16, max_len=600)
    batch = w.batch_data()
    group = next(g for g in w.groups if len(g.layer_names) == 2)  # gate/up
    x = w.inputs[group.name]
    rd = batch.data[group.layer_names[0]][LORA].rank_data[64]
    assert rd.shrink_tiles is not None and rd.expand_tiles is not None
    lens = (rd.segment_ends - rd.segment_starts).tolist()
    assert rd.expand_tiles.num_tiles >= len(lens) and rd.shrink_tiles.tile_rows in (16, 32, 48, 64)
    rows = sorted(r for _, a, b, _ in rd.shrink_tiles.records.tolist() for r in range(a, b))
    assert rows == list(range(w.num_tokens))

    class Base(torch.nn.Module):
        def forward(self, inp):
            return torch.zeros((inp.size(0), group.h_out), dtype=inp.dtype, device=inp.device)

    layer = TensorParallelMultiAdapterLinear.load(Base(), 0, group.layer_names, group.sizes)
    with_plans = layer(x, batch)
    for name in group.layer_names:
        for rs in batch.data[name][LORA].rank_data.values():
            rs.shrink_tiles = rs.expand_tiles = None
    without = layer(x, batch)
    torch.cuda.synchronize()
    assert_close(with_plans, without.cpu(), "layer output with plans against without")
    assert torch.count_nonzero(with_plans) > 0


def test_a_tile_that_names_a_segment_without_a_stack_is_skipped():
    """A caller's plan may be wrong about a segment: a tile whose segment has a null table entry is dropped by both
    kernels (and records are clamped to the call's sizes), the other tiles give the usual result."""
    dtype, r, h_in, h_out, layer = torch.bfloat16, 32, 1024, 768, 0
    gen = torch.Generator().manual_seed(9)
    starts, ends, T = [0, 700, 700], [700, 700, 1300], 1300  # the middle segment is empty and has no stack
    x = randn((T, h_in), 1.0, gen, dtype, DEV)
    a = [randn((1, r, h_in), 0.05, gen, dtype, DEV), None, randn((1, r, h_in), 0.05, gen, dtype, DEV)]
    bt = [randn((1, h_out, r), 0.05, gen, dtype, DEV), None, randn((1, h_out, r), 0.05, gen, dtype, DEV)]
    s_start = torch.tensor(starts, dtype=torch.int32, device=DEV)
    s_end = torch.tensor(ends, dtype=torch.int32, device=DEV)
    tmp = sgmv.get_tmp_tensor(torch.device(DEV))
    tmp_e = sgmv.get_tmp_tensor_for_size(3, torch.device(DEV))
    for kind, rows in ((_native.TILES_SHRINK, 48), (_native.TILES_EXPAND, 256)):
        records, tile_rows = _native.plan_tiles(starts, ends, T, kind, r)
        stray = torch.tensor([[1, 100, 100 + min(rows, tile_rows), 0], [2, 1290, 5000, 99]], dtype=torch.int32)
        wrong = _native.TilePlan(torch.cat([torch.from_numpy(records.copy()), stray]).to(DEV), tile_rows)
        good = _native.TilePlan(torch.from_numpy(records.copy()).to(DEV), tile_rows)
        if kind == _native.TILES_SHRINK:
            outs = []
            previous = _native.set_fixed_order_shrink(True)  # two more tiles change the grid, and with it the order
            try:                                             # of the sums, unless that order is fixed
                for plan in (good, wrong):
                    v = torch.zeros((T, r), dtype=dtype, device=DEV)
                    _native.sgmv_shrink_multi([v], x, [ptr_table(a, DEV)], s_start, s_end, tmp, layer, 1.0, False, plan)
                    outs.append(v)
            finally:
                _native.set_fixed_order_shrink(previous)
        else:
            vin = randn((T, r), 1.0, gen, dtype, DEV)
            outs = []
            for plan in (good, wrong):
                y = torch.zeros((T, h_out), dtype=dtype, device=DEV)
                _native.sgmv_expand(y, vin, ptr_table(bt, DEV), s_start, s_end, tmp_e, layer, 0, h_out, True, False, plan)
                outs.append(y)
        torch.cuda.synchronize()
        # the stray tile over rows 1290.. of segment 2 is clamped to the batch and rewrites what its own tile wrote
        differ = (outs[0] != outs[1]).nonzero()
        assert differ.numel() == 0, f"kind {kind}: {differ.size(0)} elements differ, first {differ[:8].tolist()}"
        assert torch.count_nonzero(outs[0]) > 0
