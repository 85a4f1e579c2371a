"""SGMV parity on the GPU: shrink and expand HIP kernels through the C ABI (via the
reference-shaped wrappers lora_a_sgmv_cutlass / lora_b_sgmv_cutlass) against the CPU oracle.
Tolerance: max-abs <= 2e-2, relative L2 <= 5e-3; rows outside every segment stay bit-identical."""

import json
from pathlib import Path

import pytest
import torch

from lorax_amd import _native, sgmv
from oracle import lora_oracle as O
from tests.helpers import assert_close, ptr_table, randn, stored_sgmv_a

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
KAT = json.loads((Path(__file__).resolve().parent / "golden" / "sgmv_kat.json").read_text())


def _run_pair(x, y, wa_list, wb_list, starts, ends, layer, r):
    s_start = torch.tensor(starts, dtype=torch.int32, device=DEV)
    s_end = torch.tensor(ends, dtype=torch.int32, device=DEV)
    wa_ptr = ptr_table(wa_list, DEV)
    wb_ptr = ptr_table(wb_list, DEV)
    tmp_shrink, tmp_expand = sgmv.get_tmp_tensors(len(starts), r, x.device)
    v = sgmv.lora_a_sgmv_cutlass(x, tmp_shrink, wa_ptr, s_start, s_end, layer, r)
    sgmv.lora_b_sgmv_cutlass(y, v, tmp_expand, wb_ptr, s_start, s_end, layer)
    return v


@pytest.mark.parametrize("segments", KAT["segments"])
@pytest.mark.parametrize("lora_rank", KAT["lora_ranks"])
def test_add_lora_sgmv_reference_kat(lora_rank, segments):
    """The reference's own known-answer test (server/tests/utils/test_sgmv.py:42-105): same shapes,
    seed, segment lists (the second has an empty segment behind a null pointer), tolerances and the
    requirement that a graph-captured replay gives the same answer."""
    print(f"case r={lora_rank} segments={segments}", flush=True)
    torch.manual_seed(KAT["seed"])
    B, H, r, L = KAT["B"], KAT["H"], lora_rank, KAT["nlayers"]
    y = torch.zeros((B, H), dtype=torch.float16, device=DEV)
    x = torch.randn((B, H), dtype=torch.float16, device=DEV)
    wa = torch.randn(L, r, H, dtype=torch.float16, device=DEV)
    if sgmv.use_cutlass_shrink(r):
        wa = wa.transpose(1, 2).contiguous()
    wb = torch.randn(L, r, H, dtype=torch.float16, device=DEV)
    starts, ends = segments
    wa_list = [wa if e - s > 0 else None for s, e in zip(starts, ends)]
    wb_list = [wb if e - s > 0 else None for s, e in zip(starts, ends)]
    layer = KAT["layer_idx"]

    y_ref = O.sgmv_ref(y.clone(), x, wa_list, wb_list, starts, ends, layer, r)

    y_ours = torch.zeros((B, H), dtype=torch.float16, device=DEV)
    _run_pair(x, y_ours, wa_list, wb_list, starts, ends, layer, r)
    assert torch.allclose(y_ref, y_ours, rtol=KAT["rtol"], atol=KAT["atol"]), (y_ref - y_ours).abs().max()

    s_start = torch.tensor(starts, dtype=torch.int32, device=DEV)
    s_end = torch.tensor(ends, dtype=torch.int32, device=DEV)
    wa_ptr, wb_ptr = ptr_table(wa_list, DEV), ptr_table(wb_list, DEV)
    tmp_shrink, tmp_expand = sgmv.get_tmp_tensors(len(starts), r, x.device)
    y_graph = torch.zeros((B, H), dtype=torch.float16, device=DEV)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, pool=None):
        v = sgmv.lora_a_sgmv_cutlass(x, tmp_shrink, wa_ptr, s_start, s_end, layer, r)
        sgmv.lora_b_sgmv_cutlass(y_graph, v, tmp_expand, wb_ptr, s_start, s_end, layer)
    torch.cuda.synchronize()
    graph.replay()
    torch.cuda.synchronize()
    assert torch.allclose(y_ours, y_graph, rtol=KAT["rtol"], atol=KAT["atol"])
    for _ in range(2):  # further replays accumulate the same delta again
        y_graph.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y_ours, y_graph)


def _ragged_case(dtype, r, h_in, h_out, lens, gen, L=2, gaps=True):
    """Segments of the given lengths laid out in order with a few uncovered rows between them."""
    starts, ends, pos = [], [], 0
    for i, n in enumerate(lens):
        if gaps and i % 3 == 1:
            pos += 2  # rows that belong to no segment
        starts.append(pos)
        ends.append(pos + n)
        pos += n
    T = pos + (3 if gaps else 0)
    x = randn((T, h_in), 1.0, gen, dtype, DEV)
    y0 = randn((T, h_out), 0.5, gen, dtype, DEV)
    a = [randn((L, h_in, r), 0.02, gen, dtype, DEV) if n > 0 else None for n in lens]
    wa = [stored_sgmv_a(t, r) if t is not None else None for t in a]
    wb = [randn((L, r, h_out), 0.02, gen, dtype, DEV) if n > 0 else None for n in lens]
    return T, x, y0, wa, wb, starts, ends


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("r", [8, 16, 32, 64, 128])
@pytest.mark.parametrize("h_in,h_out,lens", [
    (4096, 4096, [16, 16, 16, 16]),
    (1024, 2048, [1, 0, 3, 17, 1, 64, 5, 0, 130]),
    (4096, 14336, [300, 2, 31, 257]),
    (14336, 4096, [70, 1, 1, 200]),
])
def test_sgmv_shrink_expand_vs_oracle(dtype, r, h_in, h_out, lens):
    print(f"case dtype={dtype} r={r} h_in={h_in} h_out={h_out} lens={lens}", flush=True)
    gen = torch.Generator().manual_seed(r * 7 + len(lens))
    layer = 1
    T, x, y0, wa, wb, starts, ends = _ragged_case(dtype, r, h_in, h_out, lens, gen)
    y = y0.clone()
    v = _run_pair(x, y, wa, wb, starts, ends, layer, r)
    torch.cuda.synchronize()

    cpu = lambda ts: [t.cpu() if t is not None else None for t in ts]  # noqa: E731
    v_ref = O.sgmv_ref(torch.zeros((T, r), dtype=dtype), x.cpu(), cpu(wa),
                       [torch.eye(r, dtype=dtype).expand(2, r, r) if w is not None else None for w in wb],
                       starts, ends, layer, r)
    y_ref = O.sgmv_ref(y0.cpu().clone(), x.cpu(), cpu(wa), cpu(wb), starts, ends, layer, r)
    assert_close(v, v_ref, "shrink output v")  # where |v| reaches 4..8 the limit is the spacing of the type there
    assert_close(y, y_ref, "expand output y")
    covered = torch.zeros(T, dtype=torch.bool)
    for s, e in zip(starts, ends):
        covered[s:e] = True
    assert torch.equal(y.cpu()[~covered], y0.cpu()[~covered])
    assert torch.count_nonzero(v.cpu()[~covered]) == 0


@pytest.mark.parametrize("r,h_in,lens", [
    # the shrink launcher picks its tile height from the row and segment counts and its kernel family from
    # the rank and from h_in % 128; these shapes reach every combination it has
    (16, 256, [3000, 1, 2500, 2691]),         # 64-row tiles
    (64, 384, [4096, 4096]),                  # 64-row tiles, four rank blocks
    (128, 256, [2048, 2048, 2048, 2048]),     # 64-row tiles, rank 128
    (96, 128, [2100, 2100, 2100, 2100]),      # 64-row tiles, odd number of rank blocks above four
    (32, 512, [500] * 8 + [5]),               # 32-row tiles
    (48, 256, [600, 700, 800, 900, 1000]),    # 32-row tiles, odd number of rank blocks
    (128, 256, [40] * 100 + [1] * 60),        # 32-row tiles, rank 128, many short segments
    (16, 128, [1] * 600),                     # 16-row tiles, one row each
    (64, 4096, [200, 300, 7, 400, 100]),      # a thousand rows: hidden dimension in 3 parts, second pass adds them
    (128, 2048, [600, 1, 50]),                # the same at rank 128, 2 parts
    (40, 3072, [513]),                        # the same with an odd number of rank blocks, one segment
    (64, 192, [3000, 2000, 3000]),            # h_in not a multiple of 128: register-operand kernel
    (16, 4160, [330, 290]),                   # the same with K split across workgroups
    (24, 1000, [100, 28, 1]),                 # a few rows: streaming kernel, any rank and h_in multiple of 8
])
def test_sgmv_shrink_tile_variants(r, h_in, lens):
    print(f"case r={r} h_in={h_in} segments={len(lens)} rows={sum(lens)}", flush=True)
    dtype = torch.bfloat16
    gen = torch.Generator().manual_seed(r + h_in + len(lens))
    T, x, y0, wa, wb, starts, ends = _ragged_case(dtype, r, h_in, 128, lens, gen, L=2)
    y = y0.clone()
    v = _run_pair(x, y, wa, wb, starts, ends, 1, r)
    torch.cuda.synchronize()
    cpu = lambda ts: [t.cpu() if t is not None else None for t in ts]  # noqa: E731
    v_ref = O.sgmv_ref(torch.zeros((T, r), dtype=dtype), x.cpu(), cpu(wa),
                       [torch.eye(r, dtype=dtype).expand(2, r, r) for _ in wb], starts, ends, 1, r)
    y_ref = O.sgmv_ref(y0.cpu().clone(), x.cpu(), cpu(wa), cpu(wb), starts, ends, 1, r)
    assert_close(v, v_ref, "shrink output v")
    assert_close(y, y_ref, "expand output y")
    covered = torch.zeros(T, dtype=torch.bool)
    for s, e in zip(starts, ends):
        covered[s:e] = True
    assert torch.count_nonzero(v.cpu()[~covered]) == 0


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("r", [8, 16, 24, 32, 64, 96, 128])
@pytest.mark.parametrize("h_out,lens,window", [
    (4096, [16, 16, 16, 16], None),
    (2048, [1, 0, 3, 17, 1, 64, 5, 0, 130], None),
    (1160, [300, 2, 31, 257], None),             # 18 panels of 64 columns and one of 8
    (1024, [70, 1, 1, 600], (512, 384)),         # a column window of a wider y
    (512, [288, 289, 545, 16], None),            # remainders that are merged into the other tiles, and one that is not
    (8, [5, 40], None),
])
def test_sgmv_expand_transposed_b(dtype, r, h_out, lens, window):
    """lorax_sgmv_expand with b_layout = LORAX_B_HR ([L, h_out, r] stacks) against the oracle on the
    reference layout, and against the kernel for the reference layout."""
    print(f"case dtype={dtype} r={r} h_out={h_out} lens={lens} window={window}", flush=True)
    gen = torch.Generator().manual_seed(r * 11 + h_out)
    layer = 1
    T, _, y0, _, wb, starts, ends = _ragged_case(dtype, r, 64, h_out, lens, gen)
    v = randn((T, r), 1.0, gen, dtype, DEV)
    off, width = window if window is not None else (0, h_out)
    if window is not None:
        wb = [w[:, :, :width].contiguous() if w is not None else None for w in wb]
    wbt = [w.transpose(1, 2).contiguous() if w is not None else None for w in wb]
    s_start = torch.tensor(starts, dtype=torch.int32, device=DEV)
    s_end = torch.tensor(ends, dtype=torch.int32, device=DEV)
    tmp = sgmv.get_tmp_expand_size(len(starts))
    tmp = torch.empty((tmp,), dtype=torch.uint8, device=DEV)
    y_t, y_n = y0.clone(), y0.clone()
    sgmv.lora_b_sgmv_cutlass_slice(y_t, v, tmp, ptr_table(wbt, DEV), s_start, s_end, layer, off, width, transposed=True)
    sgmv.lora_b_sgmv_cutlass_slice(y_n, v, tmp, ptr_table(wb, DEV), s_start, s_end, layer, off, width)
    torch.cuda.synchronize()
    y_ref = y0.cpu().clone()
    for i, (s, e) in enumerate(zip(starts, ends)):
        if e > s:
            delta = v.cpu()[s:e] @ wb[i][layer].cpu()
            y_ref[s:e, off:off + width] = y_ref[s:e, off:off + width] + delta
    assert_close(y_t, y_ref, "transposed-B expand", rounded=[(y_ref.float() - y0.cpu().float()).to(dtype)])
    # Segments of more than 4 rows run the same MFMA arithmetic in the same order for both layouts (the
    # reference-layout kernel sums shorter ones on the vector ALU; a remainder of a few rows is merged into the
    # segment's other tiles, so only segments of up to 4 rows make such tiles).
    long_rows = torch.zeros(T, dtype=torch.bool)
    for s, e in zip(starts, ends):
        if e - s > 4:
            long_rows[s:e] = True
    assert torch.equal(y_t.cpu()[long_rows], y_n.cpu()[long_rows])
    assert_close(y_n, y_ref, "reference-layout expand", rounded=[(y_ref.float() - y0.cpu().float()).to(dtype)])
    outside = torch.ones_like(y0, dtype=torch.bool).cpu()
    for s, e in zip(starts, ends):
        outside[s:e, off:off + width] = False
    assert torch.equal(y_t.cpu()[outside], y0.cpu()[outside])


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("r", [8, 24, 40, 72, 120])
@pytest.mark.parametrize("h_in,lens", [(1024, [1, 0, 3, 17, 1, 64, 5, 0, 130]), (256, [700, 650, 3, 900])])
def test_sgmv_shrink_resident_layout_any_rank(dtype, r, h_in, lens):
    """lorax_sgmv_shrink with LORAX_A_RH stacks ([L, r, h_in]) takes every rank that is a multiple of 8 when
    h_in is a multiple of 128 - the layout decode keeps resident, so prefill needs no second copy of A."""
    print(f"case dtype={dtype} r={r} h_in={h_in} lens={lens}", flush=True)
    from lorax_amd import _native

    gen = torch.Generator().manual_seed(r + h_in)
    starts, ends, pos = [], [], 0
    for n in lens:
        starts.append(pos)
        ends.append(pos + n)
        pos += n + 1  # one uncovered row after every segment
    T = pos
    x = randn((T, h_in), 1.0, gen, dtype, DEV)
    wa_t = [randn((2, r, h_in), 0.05, gen, dtype, DEV) if n > 0 else None for n in lens]
    v = torch.zeros((T, r), dtype=dtype, device=DEV)
    _native.sgmv_shrink(v, x, ptr_table(wa_t, DEV), torch.tensor(starts, dtype=torch.int32, device=DEV),
                        torch.tensor(ends, dtype=torch.int32, device=DEV), sgmv.get_tmp_tensor(torch.device(DEV)), 1)
    torch.cuda.synchronize()
    v_ref = torch.zeros((T, r), dtype=dtype)
    for i, (s, e) in enumerate(zip(starts, ends)):
        if e > s:
            v_ref[s:e] = x.cpu()[s:e] @ wa_t[i][1].cpu().t()
    assert_close(v, v_ref, "shrink output v")
    covered = torch.zeros(T, dtype=torch.bool)
    for s, e in zip(starts, ends):
        covered[s:e] = True
    assert torch.count_nonzero(v.cpu()[~covered]) == 0
    if r % 16 != 0 and T > 512:
        with pytest.raises(RuntimeError, match="No suitable kernel"):
            _native.sgmv_shrink(torch.zeros((T, r), dtype=dtype, device=DEV), x[:, :h_in - 64].contiguous(),
                                ptr_table(wa_t, DEV), torch.tensor(starts, dtype=torch.int32, device=DEV),
                                torch.tensor(ends, dtype=torch.int32, device=DEV),
                                sgmv.get_tmp_tensor(torch.device(DEV)), 1)


@pytest.mark.parametrize("r", [48, 80, 96, 112])
def test_sgmv_other_multiples_of_16(r):
    """pad_to_min_rank can produce these ranks (punica.py:57-65); the reference's shrink has no
    instantiation for 48, 80 and 112 (sgmv_config.h:10-15)."""
    gen = torch.Generator().manual_seed(r)
    dtype = torch.bfloat16
    T, x, y0, wa, wb, starts, ends = _ragged_case(dtype, r, 2752, 1152, [40, 3, 129], gen)
    y = y0.clone()
    _run_pair(x, y, wa, wb, starts, ends, 0, r)
    cpu = lambda ts: [t.cpu() if t is not None else None for t in ts]  # noqa: E731
    y_ref = O.sgmv_ref(y0.cpu().clone(), x.cpu(), cpu(wa), cpu(wb), starts, ends, 0, r)
    assert_close(y, y_ref, "y")


def test_sgmv_empty_negative_and_null_segments_touch_nothing():
    dtype, r, h = torch.bfloat16, 64, 1024
    gen = torch.Generator().manual_seed(2)
    T = 40
    x = randn((T, h), 1.0, gen, dtype, DEV)
    y0 = randn((T, h), 0.5, gen, dtype, DEV)
    wa = stored_sgmv_a(randn((1, h, r), 0.02, gen, dtype, DEV), r)
    wb = randn((1, r, h), 0.02, gen, dtype, DEV)
    starts = [0, 10, -1, 20, 30]
    ends = [10, 10, -1, 15, 40]  # empty, (-1, -1), negative length
    wa_list = [wa, None, None, None, wa]
    wb_list = [wb, None, None, None, wb]
    y = y0.clone()
    v = _run_pair(x, y, wa_list, wb_list, starts, ends, 0, r)
    y_ref = O.sgmv_ref(y0.cpu().clone(), x.cpu(), [wa.cpu(), None, None, None, wa.cpu()],
                       [wb.cpu(), None, None, None, wb.cpu()], starts, ends, 0, r)
    assert_close(y, y_ref, "y")
    assert torch.equal(y.cpu()[10:30], y0.cpu()[10:30])
    assert torch.count_nonzero(v.cpu()[10:30]) == 0
    # no segment at all
    y2 = y0.clone()
    _run_pair(x, y2, [None], [None], [5], [5], 0, r)
    assert torch.equal(y2, y0)


def test_sgmv_routing_is_bit_exact():
    """Every segment's A picks x[:, 0] = 1 and its B writes (i + 1) / 128 + j / 32 into column j."""
    dtype, r, h_in, h_out = torch.float16, 16, 512, 128
    lens = [5, 1, 40, 16, 300, 2]
    starts, ends, pos = [], [], 3
    for n in lens:
        starts.append(pos)
        ends.append(pos + n)
        pos += n + 1
    T = pos
    x = torch.randn(T, h_in, generator=torch.Generator().manual_seed(0))
    x[:, 0] = 1.0
    x = x.to(dtype).to(DEV)
    wa, wb = [], []
    for i in range(len(lens)):
        a = torch.zeros(1, r, h_in)
        a[0, 0, 0] = 1.0
        b = torch.zeros(1, r, h_out)
        b[0, 0, :] = (i + 1) / 128.0 + torch.arange(h_out) / 32.0
        wa.append(a.to(dtype).to(DEV))
        wb.append(b.to(dtype).to(DEV))
    y = torch.full((T, h_out), 0.5, dtype=dtype, device=DEV)
    _run_pair(x, y, wa, wb, starts, ends, 0, r)
    expect = torch.full((T, h_out), 0.5)
    for i, (s, e) in enumerate(zip(starts, ends)):
        expect[s:e] += (i + 1) / 128.0 + torch.arange(h_out) / 32.0
    assert torch.equal(y.cpu(), expect.to(dtype))


def test_sgmv_expand_column_window():
    dtype, r, h_in = torch.bfloat16, 32, 4096
    sizes = [14336, 14336]
    gen = torch.Generator().manual_seed(4)
    lens = [33, 100, 7]
    T, x, _, _, _, starts, ends = _ragged_case(dtype, r, h_in, 8, lens, gen, gaps=False)
    y0 = randn((T, sum(sizes)), 0.5, gen, dtype, DEV)
    y = y0.clone()
    y_ref = y0.cpu().clone()
    s_start = torch.tensor(starts, dtype=torch.int32, device=DEV)
    s_end = torch.tensor(ends, dtype=torch.int32, device=DEV)
    off = 0
    for h_out in sizes:
        wa = [stored_sgmv_a(randn((1, h_in, r), 0.02, gen, dtype, DEV), r) for _ in lens]
        wb = [randn((1, r, h_out), 0.02, gen, dtype, DEV) for _ in lens]
        tmp_shrink, tmp_expand = sgmv.get_tmp_tensors(len(lens), r, x.device)
        v = sgmv.lora_a_sgmv_cutlass(x, tmp_shrink, ptr_table(wa, DEV), s_start, s_end, 0, r)
        sgmv.lora_b_sgmv_cutlass_slice(y, v, tmp_expand, ptr_table(wb, DEV), s_start, s_end, 0, off, h_out)
        part = O.sgmv_ref(y_ref[:, off:off + h_out].clone(), x.cpu(), [w.cpu() for w in wa], [w.cpu() for w in wb],
                          starts, ends, 0, r)
        y_ref[:, off:off + h_out] = part
        off += h_out
    assert_close(y, y_ref, "fused gate/up output")


@pytest.mark.parametrize("r,h_in,lens", [(16, 4160, [300, 7, 313]), (64, 2080, [520, 1, 40]), (128, 1056, [700])])
def test_sgmv_split_k_is_deterministic_and_cleans_its_counters(r, h_in, lens):
    """More than 512 rows, h_in not a multiple of 128 and few row tiles: the register-operand kernel with K split
    across workgroups, partial sums and arrival counters in the caller's tmp.  The tmp buffer is filled with
    garbage before every call (nothing may be expected in it), and repeated calls must give bit-identical results
    (fixed summation order)."""
    dtype = torch.bfloat16
    gen = torch.Generator().manual_seed(9 + r)
    T, x, _, wa, _, starts, ends = _ragged_case(dtype, r, h_in, 8, lens, gen, gaps=True)
    assert T > 512
    s_start = torch.tensor(starts, dtype=torch.int32, device=DEV)
    s_end = torch.tensor(ends, dtype=torch.int32, device=DEV)
    tmp = sgmv.get_tmp_tensor(x.device)
    outs = []
    for i in range(4):
        tmp.fill_(0xA5 + i)
        outs.append(sgmv.lora_a_sgmv_cutlass(x, tmp, ptr_table(wa, DEV), s_start, s_end, 1, r))
    torch.cuda.synchronize()
    for o in outs[1:]:
        assert torch.equal(o, outs[0])
    v_ref = O.sgmv_ref(torch.zeros((T, r), dtype=dtype), x.cpu(), [w.cpu() for w in wa],
                       [torch.eye(r, dtype=dtype).expand(2, r, r)] * len(lens), starts, ends, 1, r)
    assert_close(outs[0], v_ref, "v")


def test_sgmv_errors_raise_runtime_error():
    x = torch.zeros((4, 1024), dtype=torch.bfloat16, device=DEV)
    ptr = torch.zeros(1, dtype=torch.int64, device=DEV)
    s = torch.zeros(1, dtype=torch.int32, device=DEV)
    good_shrink, good_expand = sgmv.get_tmp_tensors(1, 16, x.device)
    with pytest.raises(RuntimeError, match="CHECK_EQ"):
        sgmv.lora_a_sgmv_cutlass(x, good_expand, ptr, s, s, 0, 16)  # 60-byte tmp where 8 MiB is required
    with pytest.raises(RuntimeError, match="CHECK_EQ"):
        sgmv.lora_b_sgmv_cutlass(torch.zeros((4, 1024), dtype=torch.bfloat16, device=DEV),
                                 torch.zeros((4, 16), dtype=torch.bfloat16, device=DEV), good_shrink, ptr, s, s, 0)
    with pytest.raises(RuntimeError, match="No suitable kernel"):
        sgmv.lora_a_sgmv_cutlass(x.float(), good_shrink, ptr, s, s, 0, 16)
    with pytest.raises(RuntimeError, match="int32"):
        sgmv.lora_a_sgmv_cutlass(x, good_shrink, ptr, s.long(), s.long(), 0, 16)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("count,r,h_in,lens", [
    (2, 64, 1024, [700, 1, 0, 33, 1, 300]),   # gate/up at rank 64: one launch of summed rank 128
    (2, 64, 4096, [500, 1, 0, 33, 1, 300]),   # the same with the hidden dimension cut into parts (two passes)
    (3, 16, 512, [520, 17, 64]),              # q/k/v at rank 16
    (3, 40, 256, [1, 600, 5]),                # summed rank 120, not a multiple of 16 per projection
    (4, 8, 384, [256, 257, 3]),               # four projections of rank 8
    (4, 32, 1024, [900]),                     # summed rank 128
    (3, 64, 512, [600, 40]),                  # summed rank 192: one launch per projection
    (2, 16, 1000, [600, 40]),                 # h_in not a multiple of 128: one launch per projection
    (2, 64, 1024, [100, 1, 30]),              # a small batch: the streaming kernel, one launch per projection
])
def test_sgmv_shrink_multi(dtype, count, r, h_in, lens):
    """lorax_sgmv_shrink_multi: every projection's v as from lorax_sgmv_shrink on its own, whether the call
    runs as one launch over the stacked A matrices or falls back to one launch per projection."""
    print(f"case dtype={dtype} count={count} r={r} h_in={h_in} lens={lens}", flush=True)
    gen = torch.Generator().manual_seed(count * 1000 + r + h_in)
    starts, ends, pos = [], [], 2
    for n in lens:
        starts.append(pos)
        ends.append(pos + n)
        pos += n + 1  # one uncovered row after every segment
    T, layer = pos, 1
    x = randn((T, h_in), 1.0, gen, dtype, DEV)
    stacks = [[randn((2, r, h_in), 0.05, gen, dtype, DEV) if n > 0 else None for n in lens] for _ in range(count)]
    s_start = torch.tensor(starts, dtype=torch.int32, device=DEV)
    s_end = torch.tensor(ends, dtype=torch.int32, device=DEV)
    tmp = sgmv.get_tmp_tensor(torch.device(DEV))
    tables = [ptr_table(ws, DEV) for ws in stacks]
    vs = sgmv.lora_a_sgmv_resident_multi(x, tmp, tables, s_start, s_end, layer, r)
    singles = [sgmv.lora_a_sgmv_resident(x, tmp, t, s_start, s_end, layer, r) for t in tables]
    # overwrite mode: same values in the rows of the segments whatever v held, other rows untouched
    dirty = [torch.full((T, r), 7.0, dtype=dtype, device=DEV) for _ in tables]
    _native.sgmv_shrink_multi(dirty, x, tables, s_start, s_end, sgmv.get_shrink_scratch(torch.device(DEV)), layer, 1.0,
                              accumulate=False)
    torch.cuda.synchronize()
    covered = torch.zeros(T, dtype=torch.bool)
    for s, e in zip(starts, ends):
        covered[s:e] = True
    for p in range(count):
        assert torch.equal(dirty[p].cpu()[covered], vs[p].cpu()[covered])
        assert torch.all(dirty[p].cpu()[~covered] == 7.0)
    for p in range(count):
        v_ref = torch.zeros((T, r), dtype=dtype)
        for i, (s, e) in enumerate(zip(starts, ends)):
            if e > s:
                v_ref[s:e] = x.cpu()[s:e] @ stacks[p][i][layer].cpu().t()
        assert_close(vs[p], v_ref, f"projection {p}")
        assert_close(vs[p], singles[p].cpu(), f"projection {p} against its own launch")
        assert torch.count_nonzero(vs[p].cpu()[~covered]) == 0


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("r,h_in,widths,lens", [
    (16, 4096, [4096], [16, 16, 16, 16]),          # the 64-token q_proj prefill
    (8, 4096, [4096, 1024, 1024], [5, 0, 1, 33]),  # q/k/v slices of one fused output, an empty segment
    (16, 1024, [520, 2048], [1, 1, 1, 1, 1, 1, 1]),  # ragged width, single-row segments
    (8, 2048, [256], [130, 3, 200]),                # a few hundred rows
])
def test_sgmv_lora_single_launch(dtype, r, h_in, widths, lens):
    """lorax_sgmv_lora_multi: shrink and expand of a short prefill batch in one launch - the values of the
    overwrite-mode shrink followed by the transposed-B expand (the two paths add in different orders, so not
    always the same bits) and the oracle's values."""
    print(f"case dtype={dtype} r={r} h_in={h_in} widths={widths} lens={lens}", flush=True)
    gen = torch.Generator().manual_seed(r + h_in + len(lens))
    starts, ends, pos = [], [], 1
    for n in lens:
        starts.append(pos)
        ends.append(pos + n)
        pos += n + 1  # one uncovered row after every segment
    T, layer = pos, 1
    x = randn((T, h_in), 1.0, gen, dtype, DEV)
    y0 = randn((T, sum(widths)), 0.5, gen, dtype, DEV)
    s_start = torch.tensor(starts, dtype=torch.int32, device=DEV)
    s_end = torch.tensor(ends, dtype=torch.int32, device=DEV)
    a_stacks = [[randn((2, r, h_in), 0.05, gen, dtype, DEV) if n > 0 else None for n in lens] for _ in widths]
    b_stacks = [[randn((2, w, r), 0.05, gen, dtype, DEV) if n > 0 else None for n in lens] for w in widths]
    a_tabs = [ptr_table(s, DEV) for s in a_stacks]
    b_tabs = [ptr_table(s, DEV) for s in b_stacks]
    offs = [sum(widths[:i]) for i in range(len(widths))]
    y = y0.clone()
    _native.sgmv_lora_multi([(y, a, b, off, w) for a, b, off, w in zip(a_tabs, b_tabs, offs, widths)], x, s_start, s_end,
                            r, layer)
    y2 = y0.clone()
    scratch = sgmv.get_shrink_scratch(torch.device(DEV))
    tmp = sgmv.get_tmp_tensor_for_size(len(lens), torch.device(DEV))
    for a, b, off, w in zip(a_tabs, b_tabs, offs, widths):
        v = sgmv.lora_a_sgmv_resident(x, scratch, a, s_start, s_end, layer, r, zero_fill=False)
        sgmv.lora_b_sgmv_cutlass_slice(y2, v, tmp, b, s_start, s_end, layer, off, w, transposed=True)
    torch.cuda.synchronize()
    assert_close(y, y2.cpu(), "single launch against shrink + expand")
    y_ref = y0.cpu().clone()
    for p, (off, w) in enumerate(zip(offs, widths)):
        for i, (s, e) in enumerate(zip(starts, ends)):
            if e > s:
                v_ref = (x.cpu()[s:e] @ a_stacks[p][i][layer].cpu().t())
                y_ref[s:e, off:off + w] += (v_ref @ b_stacks[p][i][layer].cpu().t())
    assert_close(y, y_ref, "y")
    covered = torch.zeros(T, dtype=torch.bool)
    for s, e in zip(starts, ends):
        covered[s:e] = True
    assert torch.equal(y.cpu()[~covered], y0.cpu()[~covered])
