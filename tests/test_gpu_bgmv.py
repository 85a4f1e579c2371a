"""BGMV parity on the GPU: the HIP kernels, called through the C ABI by the reference-shaped
wrappers (add_lora_a_bgmv / add_lora_b_bgmv), against the CPU oracle on the same seeded inputs.
Tolerance: max-abs <= 2e-2 and relative L2 <= 5e-3; routing (which rows change) is bit-exact."""

import pytest
import torch

from lorax_amd import _native, sgmv
from oracle import lora_oracle as O
from tests.helpers import assert_close, ptr_table, randn

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _stacks(n, L, rows, cols, gen, dtype, std=0.02):
    return [randn((L, rows, cols), std, gen, dtype, DEV) for _ in range(n)]


def _indices(T, n_adapters, gen, drop=0.1):
    idx = torch.randint(0, n_adapters, (T,), generator=gen)
    idx[torch.rand((T,), generator=gen) < drop] = -1
    return idx


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("r", [8, 16, 32, 64, 128])
@pytest.mark.parametrize("T,h_in,h_out,n_adapters", [(1, 1024, 1024, 1), (7, 4096, 1024, 3), (256, 4096, 4096, 24),
                                                     (33, 14336, 4096, 12)])
def test_bgmv_shrink_expand_vs_oracle(dtype, r, T, h_in, h_out, n_adapters):
    print(f"case dtype={dtype} r={r} T={T} h_in={h_in} h_out={h_out}", flush=True)
    gen = torch.Generator().manual_seed(100 + r + T)
    L, layer = 3, 2
    wa_t = _stacks(n_adapters, L, r, h_in, gen, dtype)   # [L, r, h_in]
    wb_t = _stacks(n_adapters, L, h_out, r, gen, dtype)  # [L, h_out, r]
    x = randn((T, h_in), 1.0, gen, dtype, DEV)
    y0 = randn((T, h_out), 0.5, gen, dtype, DEV)
    idx = _indices(T, n_adapters, gen)
    idx_d = idx.to(DEV)
    # entries no token refers to hold a null pointer and must never be dereferenced
    unused = [a for a in range(n_adapters) if a not in set(idx.tolist())]
    wa_ptr = ptr_table(wa_t, DEV, null_at=unused)
    wb_ptr = ptr_table(wb_t, DEV, null_at=unused)

    v = torch.zeros((T, r), dtype=dtype, device=DEV)
    sgmv.add_lora_a_bgmv(v, x, wa_ptr, idx_d, layer)
    y = y0.clone()
    sgmv.add_lora_b_bgmv(y, v, wb_ptr, idx_d, layer)
    torch.cuda.synchronize()

    v_ref = torch.zeros((T, r), dtype=dtype)
    O.bgmv_ref(v_ref, x.cpu(), [w.cpu() for w in wa_t], idx.tolist(), layer)
    y_ref = y0.cpu().clone()
    O.bgmv_ref(y_ref, v_ref, [w.cpu() for w in wb_t], idx.tolist(), layer)

    assert_close(v, v_ref, "shrink output v")
    assert_close(y, y_ref, "expand output y")
    assert_close(y.float() - y0.float(), y_ref.float() - y0.cpu().float(), "delta")
    untouched = idx < 0
    assert torch.equal(y.cpu()[untouched], y0.cpu()[untouched])
    assert torch.count_nonzero(v.cpu()[untouched]) == 0


@pytest.mark.parametrize("r", [24, 48, 96, 120])
def test_bgmv_ranks_that_are_not_powers_of_two(r):
    print(f"case r={r}", flush=True)
    gen = torch.Generator().manual_seed(r)
    dtype, T, h_in, h_out, n, L = torch.bfloat16, 19, 2752, 1152, 5, 2
    wa_t = _stacks(n, L, r, h_in, gen, dtype)
    wb_t = _stacks(n, L, h_out, r, gen, dtype)
    x = randn((T, h_in), 1.0, gen, dtype, DEV)
    idx = _indices(T, n, gen)
    v = torch.zeros((T, r), dtype=dtype, device=DEV)
    y = torch.zeros((T, h_out), dtype=dtype, device=DEV)
    sgmv.add_lora_a_bgmv(v, x, ptr_table(wa_t, DEV), idx.to(DEV), 1)
    sgmv.add_lora_b_bgmv(y, v, ptr_table(wb_t, DEV), idx.to(DEV), 1)
    v_ref = torch.zeros((T, r), dtype=dtype)
    y_ref = torch.zeros((T, h_out), dtype=dtype)
    O.bgmv_ref(v_ref, x.cpu(), [w.cpu() for w in wa_t], idx.tolist(), 1)
    O.bgmv_ref(y_ref, v_ref, [w.cpu() for w in wb_t], idx.tolist(), 1)
    assert_close(v, v_ref, "v")
    assert_close(y, y_ref, "y")


def test_bgmv_routing_is_bit_exact():
    """Weights crafted so that the result names the adapter: A_i picks x[:, 0] (= 1), B_i column j is
    (i + 1) / 256 + j / 16 in exactly representable values. Any routing slip changes bits."""
    dtype, T, h_in, h_out, r, n, L, layer = torch.float16, 300, 256, 64, 8, 37, 2, 1
    gen = torch.Generator().manual_seed(7)
    idx = _indices(T, n, gen, drop=0.2)
    wa_t, wb_t = [], []
    for i in range(n):
        a = torch.zeros(L, r, h_in)
        a[layer, 0, 0] = 1.0
        b = torch.zeros(L, h_out, r)
        b[layer, :, 0] = (i + 1) / 256.0 + torch.arange(h_out) / 16.0
        wa_t.append(a.to(dtype).to(DEV))
        wb_t.append(b.to(dtype).to(DEV))
    x = torch.zeros(T, h_in)
    x[:, 0] = 1.0
    x[:, 1:] = torch.randn(T, h_in - 1, generator=gen)
    x = x.to(dtype).to(DEV)
    v = torch.zeros((T, r), dtype=dtype, device=DEV)
    y0 = torch.full((T, h_out), 0.25, dtype=dtype)
    y = y0.to(DEV)
    sgmv.add_lora_a_bgmv(v, x, ptr_table(wa_t, DEV), idx.to(DEV), layer)
    sgmv.add_lora_b_bgmv(y, v, ptr_table(wb_t, DEV), idx.to(DEV), layer)
    expect = y0.clone().float()
    for t, i in enumerate(idx.tolist()):
        if i >= 0:
            expect[t] += (i + 1) / 256.0 + torch.arange(h_out) / 16.0
    assert torch.equal(y.cpu(), expect.to(dtype))
    exp_v = torch.zeros(T, r)
    exp_v[idx >= 0, 0] = 1.0
    assert torch.equal(v.cpu().float(), exp_v)


def test_bgmv_column_window_of_fused_output():
    dtype, T, h_in, r, n = torch.bfloat16, 40, 4096, 16, 6
    sizes = [4096, 1024, 1024]
    gen = torch.Generator().manual_seed(11)
    x = randn((T, h_in), 1.0, gen, dtype, DEV)
    idx = _indices(T, n, gen)
    y0 = randn((T, sum(sizes)), 0.5, gen, dtype, DEV)
    y = y0.clone()
    y_ref = y0.cpu().clone()
    off = 0
    for h_out in sizes:
        wa_t = _stacks(n, 1, r, h_in, gen, dtype)
        wb_t = _stacks(n, 1, h_out, r, gen, dtype)
        v = torch.zeros((T, r), dtype=dtype, device=DEV)
        sgmv.add_lora_a_bgmv(v, x, ptr_table(wa_t, DEV), idx.to(DEV), 0)
        sgmv.add_lora_b_bgmv_slice(y, v, ptr_table(wb_t, DEV), idx.to(DEV), 0, off, h_out)
        v_ref = torch.zeros((T, r), dtype=dtype)
        O.bgmv_ref(v_ref, x.cpu(), [w.cpu() for w in wa_t], idx.tolist(), 0)
        part = y_ref[:, off:off + h_out].clone()
        O.bgmv_ref(part, v_ref, [w.cpu() for w in wb_t], idx.tolist(), 0)
        y_ref[:, off:off + h_out] = part
        off += h_out
    assert_close(y, y_ref, "fused q/k/v output")


@pytest.mark.parametrize("r", [8, 16, 24, 32, 64, 128])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_bgmv_expand_vector_and_scalar_y_paths_agree_bit_for_bit(dtype, r):
    """A y whose rows are 16-byte aligned moves in 16-byte pieces, any other element by element: same sums,
    same roundings, so the same bits.  The second window starts 4 columns into rows of a pitch that is no
    multiple of 8.  Chunks of 1 to 4 tokens per adapter, a last column block that is not full."""
    print(f"case dtype={dtype} r={r}", flush=True)
    T, h_out, n = 45, 2248, 7
    gen = torch.Generator().manual_seed(500 + r)
    wb_t = _stacks(n, 2, h_out, r, gen, dtype)
    v = randn((T, r), 1.0, gen, dtype, DEV)
    idx = _indices(T, n, gen)
    idx[:9] = 0  # an adapter with more than two chunks
    y0 = randn((T, h_out), 0.5, gen, dtype, DEV)
    ya = y0.clone()
    sgmv.add_lora_b_bgmv(ya, v, ptr_table(wb_t, DEV), idx.to(DEV), 1)
    wide = torch.zeros((T, h_out + 12), dtype=dtype, device=DEV)
    wide[:, 4:4 + h_out] = y0
    sgmv.add_lora_b_bgmv_slice(wide, v, ptr_table(wb_t, DEV), idx.to(DEV), 1, 4, h_out)
    torch.cuda.synchronize()
    assert torch.equal(ya, wide[:, 4:4 + h_out])
    assert torch.count_nonzero(wide[:, :4]) == 0 and torch.count_nonzero(wide[:, 4 + h_out:]) == 0
    y_ref = y0.cpu().clone()
    O.bgmv_ref(y_ref, v.cpu(), [w.cpu() for w in wb_t], idx.tolist(), 1)
    assert_close(ya, y_ref, "expand output y")
    assert torch.equal(ya.cpu()[idx < 0], y0.cpu()[idx < 0])


@pytest.mark.parametrize("r", [8, 64])
def test_bgmv_expand_overwrite_mode(r):
    """accumulate = 0 on an expand launch stores the update instead of adding it: the routed rows equal the
    update added to zeros, the other rows keep what they held."""
    dtype, T, h_out, n = torch.bfloat16, 37, 1160, 5
    gen = torch.Generator().manual_seed(700 + r)
    wb_t = _stacks(n, 1, h_out, r, gen, dtype)
    v = randn((T, r), 1.0, gen, dtype, DEV)
    idx = _indices(T, n, gen, drop=0.25)
    ptrs, idx_d = ptr_table(wb_t, DEV), idx.to(DEV)
    added = torch.zeros((T, h_out), dtype=dtype, device=DEV)
    _native.bgmv_multi([(added, v, ptrs, idx_d, 0, None)], 0, 1.0, accumulate=True)
    junk = randn((T, h_out), 3.0, gen, dtype, DEV)
    stored = junk.clone()
    _native.bgmv_multi([(stored, v, ptrs, idx_d, 0, None)], 0, 1.0, accumulate=False)
    torch.cuda.synchronize()
    routed = (idx >= 0).to(DEV)
    assert torch.equal(stored[routed], added[routed]) and torch.count_nonzero(added[routed]) > 0
    assert torch.equal(stored[~routed], junk[~routed])


def test_bgmv_under_graph_capture_replays_identically():
    dtype, T, h_in, h_out, r, n = torch.bfloat16, 64, 4096, 4096, 32, 9
    gen = torch.Generator().manual_seed(3)
    wa_t = _stacks(n, 2, r, h_in, gen, dtype)
    wb_t = _stacks(n, 2, h_out, r, gen, dtype)
    wa_ptr, wb_ptr = ptr_table(wa_t, DEV), ptr_table(wb_t, DEV)
    x = randn((T, h_in), 1.0, gen, dtype, DEV)
    idx = _indices(T, n, gen).to(DEV)
    # graph padding rule of the reference (utils/graph.py:71-73,421-425): extra rows carry index -1
    idx[-8:] = -1

    def run(v, y):
        v.zero_()
        y.zero_()
        sgmv.add_lora_a_bgmv(v, x, wa_ptr, idx, 1)
        sgmv.add_lora_b_bgmv(y, v, wb_ptr, idx, 1)

    v_e = torch.empty((T, r), dtype=dtype, device=DEV)
    y_e = torch.empty((T, h_out), dtype=dtype, device=DEV)
    run(v_e, y_e)
    torch.cuda.synchronize()
    v_g = torch.empty_like(v_e)
    y_g = torch.empty_like(y_e)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        run(v_g, y_g)
    for _ in range(3):
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y_g, y_e) and torch.equal(v_g, v_e)
        y_g.fill_(7.0)  # eager work between replays


def test_bgmv_errors_raise_runtime_error():
    x = torch.zeros((4, 4096), dtype=torch.bfloat16, device=DEV)
    ptr = torch.zeros(1, dtype=torch.int64, device=DEV)
    idx = torch.full((4,), -1, dtype=torch.int64, device=DEV)
    with pytest.raises(RuntimeError, match="No suitable kernel"):
        sgmv.add_lora_a_bgmv(torch.zeros((4, 12), dtype=torch.bfloat16, device=DEV), x, ptr, idx, 0)
    with pytest.raises(RuntimeError, match="No suitable kernel"):
        sgmv.add_lora_a_bgmv(torch.zeros((4, 8), dtype=torch.float32, device=DEV), x.float(), ptr, idx, 0)
    with pytest.raises(RuntimeError, match="CHECK_EQ"):
        sgmv.add_lora_a_bgmv(torch.zeros((3, 8), dtype=torch.bfloat16, device=DEV), x, ptr, idx, 0)
    with pytest.raises(RuntimeError, match="contiguous"):
        sgmv.add_lora_a_bgmv(torch.zeros((4, 16), dtype=torch.bfloat16, device=DEV)[:, ::2], x, ptr, idx, 0)
    # all tokens at -1: a valid call that touches nothing
    v = torch.ones((4, 8), dtype=torch.bfloat16, device=DEV)
    sgmv.add_lora_a_bgmv(v, x, ptr, idx, 0)
    assert torch.all(v == 1)
    assert _native.available()


@pytest.mark.parametrize("r", [8, 64])
def test_bgmv_multi_matches_separate_launches(r):
    """One batched launch for q/k/v (shared input, different widths, different routing per projection)
    against the oracle; the overwrite mode of the shrink must not depend on what v held before."""
    from lorax_amd import _native

    dtype, T, h_in, n = torch.bfloat16, 100, 4096, 11
    sizes = [4096, 1024, 1024]
    gen = torch.Generator().manual_seed(21 + r)
    x = randn((T, h_in), 1.0, gen, dtype, DEV)
    y0 = randn((T, sum(sizes)), 0.5, gen, dtype, DEV)
    y = y0.clone()
    y_ref = y0.cpu().clone()
    shrink, expand, vs, keep_alive = [], [], [], []
    off = 0
    for h_out in sizes:
        wa_t = _stacks(n, 2, r, h_in, gen, dtype)
        wb_t = _stacks(n, 2, h_out, r, gen, dtype)
        keep_alive.append((wa_t, wb_t))  # the pointer tables hold raw addresses only
        idx = _indices(T, n, gen, drop=0.15)  # routing differs between the projections
        v = torch.full((T, r), float("nan"), dtype=dtype, device=DEV)
        vs.append((v, idx))
        shrink.append((v, x, ptr_table(wa_t, DEV), idx.to(DEV), 0, None))
        expand.append((y, v, ptr_table(wb_t, DEV), idx.to(DEV), off, h_out))
        v_ref = torch.zeros((T, r), dtype=dtype)
        O.bgmv_ref(v_ref, x.cpu(), [w.cpu() for w in wa_t], idx.tolist(), 1)
        part = y_ref[:, off:off + h_out].clone()
        O.bgmv_ref(part, v_ref, [w.cpu() for w in wb_t], idx.tolist(), 1)
        y_ref[:, off:off + h_out] = part
        off += h_out
    _native.bgmv_multi(shrink, 1, 1.0, accumulate=False)
    _native.bgmv_multi(expand, 1, 1.0, accumulate=True)
    torch.cuda.synchronize()
    assert_close(y, y_ref, "fused q/k/v")
    for v, idx in vs:
        routed = idx >= 0
        assert torch.isfinite(v.cpu()[routed].float()).all()
        assert torch.isnan(v.cpu()[~routed].float()).all()  # rows without adapter are not written
    with pytest.raises(RuntimeError, match="share the direction"):
        _native.bgmv_multi([shrink[0], expand[0]], 1)
    with pytest.raises(RuntimeError, match="between 1 and 16"):
        _native.bgmv_multi(shrink * 6, 1)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("use_plan", [False, True])
def test_bgmv_multi_mixed_ranks(dtype, use_plan):
    """The rank groups of a multi-rank batch in one shrink launch and one expand launch: every problem has
    its own rank, routing (a token belongs to exactly one rank group), pointer tables and column window."""
    from lorax_amd import _native
    from lorax_amd.adapters import build_bgmv_plan

    T, h_in, n = 150, 2048, 5
    ranks = [8, 16, 32, 64, 128, 24, 8]
    sizes = [1024, 512, 1160, 1024, 256, 136, 1024]  # windows of one wide y
    gen = torch.Generator().manual_seed(77)
    x = randn((T, h_in), 1.0, gen, dtype, DEV)
    y0 = randn((T, sum(sizes)), 0.5, gen, dtype, DEV)
    y, y_ref = y0.clone(), y0.cpu().clone()
    group_of_token = torch.randint(-1, len(ranks), (T,), generator=gen)  # -1: no adapter at all
    shrink, expand, plans, keep_alive, vs = [], [], [], [], []
    off = 0
    for p, (r, h_out) in enumerate(zip(ranks, sizes)):
        wa_t = _stacks(n, 2, r, h_in, gen, dtype)
        wb_t = _stacks(n, 2, h_out, r, gen, dtype)
        keep_alive.append((wa_t, wb_t))
        idx = torch.where(group_of_token == p, torch.randint(0, n, (T,), generator=gen), torch.full((T,), -1))
        v = torch.full((T, r), float("nan"), dtype=dtype, device=DEV)
        vs.append((v, idx))
        a_ptr, b_ptr = ptr_table(wa_t, DEV), ptr_table(wb_t, DEV)
        shrink.append((v, x, a_ptr, idx.to(DEV), 0, None))
        expand.append((y, v, b_ptr, idx.to(DEV), off, h_out))
        records = build_bgmv_plan(idx.tolist(), a_ptr.tolist(), b_ptr.tolist())
        plans.append(torch.tensor(records, dtype=torch.int64, device=DEV).reshape(-1, 8))
        v_ref = torch.zeros((T, r), dtype=dtype)
        O.bgmv_ref(v_ref, x.cpu(), [w.cpu() for w in wa_t], idx.tolist(), 1)
        part = y_ref[:, off:off + h_out].clone()
        O.bgmv_ref(part, v_ref, [w.cpu() for w in wb_t], idx.tolist(), 1)
        y_ref[:, off:off + h_out] = part
        off += h_out
    _native.bgmv_multi(shrink, 1, 1.0, accumulate=False, plans=plans if use_plan else None)
    _native.bgmv_multi(expand, 1, 1.0, accumulate=True, plans=plans if use_plan else None)
    torch.cuda.synchronize()
    assert_close(y, y_ref, "mixed-rank batch", rounded=[(y_ref.float() - y0.cpu().float()).to(dtype)])
    for v, idx in vs:
        routed = idx >= 0
        assert torch.isfinite(v.cpu()[routed].float()).all()
        assert torch.isnan(v.cpu()[~routed].float()).all()
    untouched = torch.ones_like(y_ref, dtype=torch.bool)
    off = 0
    for p, h_out in enumerate(sizes):
        untouched[group_of_token == p, off:off + h_out] = False
        off += h_out
    assert torch.equal(y.cpu()[untouched], y0.cpu()[untouched])


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("r", [8, 16])
@pytest.mark.parametrize("h_in,sizes", [(4096, [4096, 1024, 1024]), (2752, [1152]), (14336, [4096])])
def test_bgmv_single_launch_shrink_expand(dtype, r, h_in, sizes):
    """lorax_bgmv_lora_multi (shrink + expand in one launch, v on chip) against the two-step oracle."""
    from lorax_amd import _native
    from lorax_amd.adapters import build_bgmv_plan

    print(f"case dtype={dtype} r={r} h_in={h_in} sizes={sizes}", flush=True)
    T, n = 77, 9
    gen = torch.Generator().manual_seed(5 * r + h_in)
    x = randn((T, h_in), 1.0, gen, dtype, DEV)
    y0 = randn((T, sum(sizes)), 0.5, gen, dtype, DEV)
    y = y0.clone()
    y_ref = y0.cpu().clone()
    problems, keep_alive = [], []
    off = 0
    for h_out in sizes:
        wa_t = _stacks(n, 2, r, h_in, gen, dtype)
        wb_t = _stacks(n, 2, h_out, r, gen, dtype)
        keep_alive.append((wa_t, wb_t))
        idx = _indices(T, n, gen, drop=0.15)
        records = build_bgmv_plan(idx.tolist(), [w.data_ptr() for w in wa_t], [w.data_ptr() for w in wb_t])
        plan = torch.tensor(records, dtype=torch.int64, device=DEV).reshape(-1, 8)
        problems.append((y, x, plan, off, h_out))
        v_ref = torch.zeros((T, r), dtype=dtype)
        O.bgmv_ref(v_ref, x.cpu(), [w.cpu() for w in wa_t], idx.tolist(), 1)
        part = y_ref[:, off:off + h_out].clone()
        O.bgmv_ref(part, v_ref, [w.cpu() for w in wb_t], idx.tolist(), 1)
        y_ref[:, off:off + h_out] = part
        off += h_out
    _native.bgmv_lora_multi(problems, r, 1)
    torch.cuda.synchronize()
    assert_close(y, y_ref, "single-launch LoRA")
    with pytest.raises(RuntimeError, match="No suitable kernel"):
        _native.bgmv_lora_multi(problems, 32, 1)


@pytest.mark.parametrize("fused", [False, True])
def test_padded_plan_and_graph_replay_with_a_new_batch(fused):
    """A plan padded with all-zero records gives the same result as the plan itself, and a captured decode step
    can be replayed for a different batch by copying that batch's padded plan, inputs and y into place."""
    from lorax_amd import _native
    from lorax_amd.adapters import build_bgmv_plan, pad_bgmv_plan

    dtype, T, h_in, h_out, r, n = torch.bfloat16, 48, 1024, 1024, 8, 6
    gen = torch.Generator().manual_seed(31)
    wa_t = _stacks(n, 2, r, h_in, gen, dtype)
    wb_t = _stacks(n, 2, h_out, r, gen, dtype)
    a_ptr, b_ptr = ptr_table(wa_t, DEV), ptr_table(wb_t, DEV)
    max_records = T  # one token per chunk at worst

    def batch(seed):
        g = torch.Generator().manual_seed(seed)
        idx = _indices(T, n, g, drop=0.2)
        records = build_bgmv_plan(idx.tolist(), a_ptr.tolist(), b_ptr.tolist())
        plan = torch.tensor(records, dtype=torch.int64, device=DEV).reshape(-1, 8)
        x = randn((T, h_in), 1.0, g, dtype, DEV)
        y0 = randn((T, h_out), 0.5, g, dtype, DEV)
        v_ref = torch.zeros((T, r), dtype=dtype)
        O.bgmv_ref(v_ref, x.cpu(), [w.cpu() for w in wa_t], idx.tolist(), 1)
        y_ref = y0.cpu().clone()
        O.bgmv_ref(y_ref, v_ref, [w.cpu() for w in wb_t], idx.tolist(), 1)
        return idx.to(DEV), plan, x, y0, y_ref

    idx1, plan1, x1, y01, ref1 = batch(1)
    idx2, plan2, x2, y02, ref2 = batch(2)
    assert plan1.size(0) != plan2.size(0) or not torch.equal(plan1, plan2)

    x, y = x1.clone(), y01.clone()
    plan = pad_bgmv_plan(plan1, max_records)
    v = torch.empty((T, r), dtype=dtype, device=DEV)
    idx = idx1.clone()

    def step():
        if fused:
            _native.bgmv_lora_multi([(y, x, plan, 0, None)], r, 1)
        else:
            _native.bgmv_multi([(v, x, a_ptr, idx, 0, None)], 1, 1.0, accumulate=False, plans=[plan])
            _native.bgmv_multi([(y, v, b_ptr, idx, 0, None)], 1, 1.0, accumulate=True, plans=[plan])

    step()
    torch.cuda.synchronize()
    assert_close(y, ref1, "padded plan, eager")
    unpadded = y01.clone()
    if fused:
        _native.bgmv_lora_multi([(unpadded, x1, plan1, 0, None)], r, 1)
        assert torch.equal(unpadded, y)

    y.copy_(y01)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    for x_new, y_new, plan_new, idx_new, ref in ((x2, y02, plan2, idx2, ref2), (x1, y01, plan1, idx1, ref1)):
        x.copy_(x_new), y.copy_(y_new), idx.copy_(idx_new)
        plan.copy_(pad_bgmv_plan(plan_new, max_records))
        graph.replay()
        torch.cuda.synchronize()
        assert_close(y, ref, "graph replay with another batch's plan")
