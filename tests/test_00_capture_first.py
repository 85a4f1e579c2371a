"""The first call of an entry point may already be under stream capture.

This file is collected first, so nothing of the library has run in the process yet: after lorax_init (the
documented per-device set-up, which may not be captured) the first-ever launch of one LDS-staged shrink shape and
of one expand shape happens inside a graph capture; the graph is then replayed several times, with eager work in
between, and every replay is checked against the oracle.  A call the runtime refused under capture would return
an error code (RuntimeError here); nothing in this test can fault."""

import pytest
import torch

from lorax_amd import _native, sgmv
from oracle import lora_oracle as O
from tests.helpers import assert_close, ptr_table, randn

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def test_first_ever_shrink_and_expand_inside_a_capture():
    dev = torch.device(DEV)
    gen = torch.Generator().manual_seed(5)
    dtype, r, h_in, h_out, L, layer = torch.bfloat16, 48, 2048, 1536, 2, 1
    lens = [700, 0, 41, 600]  # more than 512 rows, h_in a multiple of 128: the LDS-staged kernel, K cut into parts
    starts, ends, pos = [], [], 0
    for n in lens:
        starts.append(pos)
        ends.append(pos + n)
        pos += n
    T = pos
    x = randn((T, h_in), 1.0, gen, dtype, DEV)
    a_t = [randn((L, r, h_in), 0.02, gen, dtype, DEV) for _ in lens]
    b_t = [randn((L, h_out, r), 0.02, gen, dtype, DEV) for _ in lens]
    a_ptr, b_ptr = ptr_table(a_t, DEV, null_at=[1]), ptr_table(b_t, DEV, null_at=[1])
    s_start = torch.tensor(starts, dtype=torch.int32, device=DEV)
    s_end = torch.tensor(ends, dtype=torch.int32, device=DEV)
    y0 = randn((T, h_out), 0.5, gen, dtype, DEV)
    y = y0.clone()
    v = torch.zeros((T, r), dtype=dtype, device=DEV)
    tmp = sgmv.get_tmp_tensor(dev)
    tmp_e = sgmv.get_tmp_tensor_for_size(len(lens), dev)
    _native.init(dev)
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        _native.sgmv_shrink_multi([v], x, [a_ptr], s_start, s_end, tmp, layer, 1.0, False)
        sgmv.lora_b_sgmv_cutlass_slice(y, v, tmp_e, b_ptr, s_start, s_end, layer, 0, h_out, transposed=True)

    xc = x.cpu()
    v_ref = torch.zeros((T, r), dtype=dtype)
    delta = torch.zeros((T, h_out), dtype=dtype)
    for i, (s, e) in enumerate(zip(starts, ends)):
        if e > s:
            v_ref[s:e] = xc[s:e] @ a_t[i][layer].cpu().t()
            delta[s:e] = v_ref[s:e] @ b_t[i][layer].cpu().t()
    for replay in range(3):
        before = y.cpu()  # every replay adds the update once more to what the last one left
        graph.replay()
        torch.cuda.synchronize()
        want = (before.float() + delta.float()).to(dtype)
        assert_close(v, v_ref, f"v, replay {replay}")
        assert_close(y, want, f"y, replay {replay}", rounded=[delta])
        # eager work between the replays: the same launches outside the graph give the same v bit for bit
        v2 = torch.zeros_like(v)
        _native.sgmv_shrink_multi([v2], x, [a_ptr], s_start, s_end, tmp, layer, 1.0, False)
        torch.cuda.synchronize()
        assert torch.equal(v2, v)
    O.sgmv_ref  # the oracle module is the checker's home; the per-segment products above restate sgmv_ref
