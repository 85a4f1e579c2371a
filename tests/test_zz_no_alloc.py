"""lorax_sgmv_shrink_static, the entry point that allocates nothing: its output against lorax_sgmv_shrink's on the
same arguments, bit for bit, on two calls in a row (the second with a smaller batch), on shapes that use the
split-K scratch and on shapes that do not; the size limit; and that the call allocates no device memory."""

import pytest
import torch

from lorax_amd import _native, sgmv
from tests.helpers import assert_close, ptr_table, randn

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _case(r, h_in, lens, seed, dtype=torch.bfloat16):
    gen = torch.Generator().manual_seed(seed)
    starts, ends, pos = [], [], 1
    for n in lens:
        starts.append(pos)
        ends.append(pos + n)
        pos += n + 2  # uncovered rows between the segments
    x = randn((pos, h_in), 1.0, gen, dtype, DEV)
    stacks = [randn((2, r, h_in), 0.05, gen, dtype, DEV) if n > 0 else None for n in lens]
    s_start = torch.tensor(starts, dtype=torch.int32, device=DEV)
    s_end = torch.tensor(ends, dtype=torch.int32, device=DEV)
    return x, stacks, ptr_table(stacks, DEV), s_start, s_end, starts, ends


def _both(r, h_in, lens, seed, layer=1):
    x, stacks, table, s_start, s_end, starts, ends = _case(r, h_in, lens, seed)
    tmp = sgmv.get_tmp_tensor(torch.device(DEV))
    v_ref = torch.zeros((x.size(0), r), dtype=x.dtype, device=DEV)
    _native.sgmv_shrink(v_ref, x, table, s_start, s_end, tmp, layer)
    v = torch.zeros_like(v_ref)
    _native.init(torch.device(DEV))  # the per-device set-up; after it the entry point has nothing left to set up
    torch.cuda.synchronize()
    # free device memory as the driver reports it: a hipMalloc inside the library would show here, whoever made it
    # (torch's own counter only sees torch's allocator)
    free_before, allocated_before = torch.cuda.mem_get_info()[0], torch.cuda.memory_allocated()
    _native.sgmv_shrink_static(v, x, table, s_start, s_end, layer)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before
    assert torch.cuda.memory_allocated() == allocated_before
    want = torch.zeros((x.size(0), r), dtype=x.dtype)
    for i, (s, e) in enumerate(zip(starts, ends)):
        if e > s:
            want[s:e] = x.cpu()[s:e] @ stacks[i][layer].cpu().t()
    return v, v_ref, want


@pytest.mark.parametrize("r,h_in,first,second", [
    (16, 4160, [300, 7, 313], [520, 30]),     # split-K kernel both times: partial tiles and counters in the scratch
    (64, 2080, [700, 0, 90], [513]),
    (128, 1056, [1200], [600, 1, 1]),
    (32, 4096, [900, 40], [64, 3]),           # LDS-staged kernel, then the streaming kernel: no scratch
])
def test_static_shrink_matches_the_tmp_entry_point(r, h_in, first, second):
    print(f"case r={r} h_in={h_in} first={first} second={second}", flush=True)
    for lens, seed in ((first, 11), (second, 12)):
        v, v_ref, want = _both(r, h_in, lens, seed + r)
        assert torch.equal(v, v_ref), f"lens={lens}"
        assert torch.count_nonzero(v) > 0
        assert_close(v, want, f"v lens={lens}")




def test_static_shrink_refuses_a_split_that_does_not_fit_its_scratch():
    """12 000 rows at rank 64 over h_in = 4160 are 189 row tiles of the register-operand kernel, which would split
    the hidden dimension three ways: three fp32 copies of v (9.2 MB) exceed the 8 MiB array, so the call is refused
    and nothing is launched; the entry point with a caller's tmp runs it with two."""
    r, h_in, T = 64, 4160, 12000
    x = torch.zeros((T, h_in), dtype=torch.bfloat16, device=DEV)
    v = torch.full((T, r), 3.0, dtype=torch.bfloat16, device=DEV)
    w = torch.zeros((1, r, h_in), dtype=torch.bfloat16, device=DEV)
    s_start = torch.tensor([0], dtype=torch.int32, device=DEV)
    s_end = torch.tensor([T], dtype=torch.int32, device=DEV)
    with pytest.raises(RuntimeError, match="static scratch"):
        _native.sgmv_shrink_static(v, x, ptr_table([w], DEV), s_start, s_end, 0)
    torch.cuda.synchronize()
    assert torch.all(v == 3.0)
    # a batch that does not split (more row tiles) has no limit: 20 000 rows use no scratch at all
    T2 = 20000
    x2 = torch.ones((T2, 1056), dtype=torch.bfloat16, device=DEV)
    w2 = torch.ones((1, 128, 1056), dtype=torch.bfloat16, device=DEV)
    v2 = torch.zeros((T2, 128), dtype=torch.bfloat16, device=DEV)
    _native.sgmv_shrink_static(v2, x2, ptr_table([w2], DEV), s_start, torch.tensor([T2], dtype=torch.int32, device=DEV), 0)
    torch.cuda.synchronize()
    assert torch.all(v2 == 1056)


def test_static_shrink_inside_a_graph_capture():
    """The entry point exists for callers under stream capture: after lorax_init a call is captured, the graph is
    replayed three times with an eager call of lorax_sgmv_shrink in between, and every replay leaves the bits the
    eager entry point computes (overwrite semantics are not offered here, so v is cleared inside the graph)."""
    r, h_in, lens = 48, 2048, [700, 0, 41, 600]   # LDS-staged kernel, hidden dimension in parts: the scratch is used
    x, stacks, table, s_start, s_end, starts, ends = _case(r, h_in, lens, 31)
    _native.init(torch.device(DEV))
    tmp = sgmv.get_tmp_tensor(torch.device(DEV))
    v_ref = torch.zeros((x.size(0), r), dtype=x.dtype, device=DEV)
    _native.sgmv_shrink(v_ref, x, table, s_start, s_end, tmp, 1)
    v = torch.zeros_like(v_ref)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        v.zero_()  # a fill kernel, not a memset node
        _native.sgmv_shrink_static(v, x, table, s_start, s_end, 1)
    for replay in range(3):
        v.fill_(5.0)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(v, v_ref), f"replay {replay}"
        other = torch.zeros_like(v_ref)
        _native.sgmv_shrink(other, x, table, s_start, s_end, tmp, 1)  # eager work between the replays
        torch.cuda.synchronize()
        assert torch.equal(other, v_ref)
    assert torch.count_nonzero(v) > 0
