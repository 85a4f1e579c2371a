"""Pins the oracle (oracle/lora_oracle.py) before anything is compared against it:
golden vectors of the reference's tests, an fp64 brute force, and invariants chosen so
that a dropped term, a transposed operand or a wrong index fails at least one check."""

import json
from pathlib import Path

import pytest
import torch

from oracle import lora_oracle as O

GOLDEN = Path(__file__).resolve().parent / "golden"


def _golden(name):
    return json.loads((GOLDEN / f"{name}.json").read_text())


# ---------------------------------------------------------------- integer routing
@pytest.mark.parametrize("case", _golden("segments")["find_segments"])
def test_find_segments_ref_golden(case):
    assert O.find_segments_ref(case["adapter_indices"]) == (case["segments"], case["segment_indices"])


@pytest.mark.parametrize("case", _golden("segments")["concat_segments"])
def test_concat_segments_ref_golden(case):
    assert O.concat_segments_ref(case["batches"]) == (case["segments"], case["segment_indices"])


@pytest.mark.parametrize("case", _golden("lora_batch")["decode"])
def test_rank_groups_ref_golden(case):
    ranks = {i: r for i, r in enumerate(case["lora_ranks"])}
    _, owners = O.find_segments_ref(case["adapter_indices"])
    groups = O.rank_groups_ref(owners, case["adapter_indices"], ranks)
    assert {str(k) for k in groups} == set(case["expected"])
    for rank, (positions, per_token) in groups.items():
        exp = case["expected"][str(rank)]
        assert len(positions) == exp["num_ptrs"]
        assert per_token == exp["indices"]


def test_rank_groups_ref_unknown_adapter_is_dropped():
    # adapter 7 has no weights: its run is in no group and its tokens get -1 everywhere
    groups = O.rank_groups_ref([0, 7, 0], [0, 0, 7, 0], {0: 8})
    assert groups == {8: ([0, 2], [0, 0, -1, 0])}


def test_sgmv_tmp_size_ref():
    assert [O.sgmv_tmp_size_ref(n) for n in (0, 1, 2, 32)] == [0, 60, 120, 1920]
    assert O.sgmv_tmp_size_ref(1) == _golden("sgmv_kat")["tmp_bytes_per_problem"]


# ---------------------------------------------------------------- padding / orientation
@pytest.mark.parametrize("rank,min_rank,target", [(4, 8, 8), (8, 8, 8), (9, 8, 16), (16, 8, 16), (17, 8, 32),
                                                  (8, 16, 16), (16, 16, 16), (24, 16, 32), (100, 64, 112)])
def test_pad_to_min_rank_ref_targets(rank, min_rank, target):
    t = torch.arange(3 * rank, dtype=torch.float32).view(3, rank)
    p = O.pad_to_min_rank_ref(t, 1, min_rank)
    assert p.shape == (3, target)
    assert torch.equal(p[:, :rank], t) and torch.count_nonzero(p[:, rank:]) == 0
    pt = O.pad_to_min_rank_ref(t.t().contiguous(), 0, min_rank)
    assert torch.equal(pt, p.t())


def test_pad_rank_preserves_product():
    kat = _golden("sgmv_kat")["pad_rank"]
    torch.manual_seed(0)
    for ws in kat["world_sizes"]:
        for r in kat["lora_ranks"]:
            x = torch.randn(kat["bs"], kat["h"], dtype=torch.float64)
            a = torch.randn(kat["h"], r, dtype=torch.float64)
            b = torch.randn(r, kat["h"], dtype=torch.float64)
            ap, bp = O.pad_to_min_rank_ref(a, 1, 8 * ws), O.pad_to_min_rank_ref(b, 0, 8 * ws)
            assert ap.size(1) == bp.size(0) >= r
            assert torch.allclose(x @ a @ b, x @ ap @ bp, rtol=1e-12, atol=1e-9)


def test_orient_for_rank_ref():
    t = torch.zeros(5, 7)
    assert O.orient_for_rank_ref(t, 8).shape == (5, 7)
    assert O.orient_for_rank_ref(t, 16).shape == (7, 5)
    assert O.orient_for_rank_ref(t, 128).shape == (7, 5)
    assert O.orient_for_rank_ref(t, 129).shape == (5, 7)


# ---------------------------------------------------------------- floating point
def _problem(dtype, T, h_in, h_out, ranks, L=2, seed=0, drop=(), scale_w=0.05):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(T, h_in, generator=g).to(dtype)
    a_hr, b_rh = {}, {}
    for i, r in enumerate(ranks):
        a_hr[i] = (torch.randn(L, h_in, r, generator=g) * scale_w).to(dtype)
        b_rh[i] = (torch.randn(L, r, h_out, generator=g) * scale_w).to(dtype)
    tok = torch.randint(0, len(ranks), (T,), generator=g).tolist()
    for t in drop:
        tok[t] = -1
    return x, a_hr, b_rh, tok


def _stored_a(a_hr_layerstack, r):
    # storage of LoraWeights: [L, r, h_in] for 16 <= r <= 128, else [L, h_in, r]
    return a_hr_layerstack.transpose(1, 2).contiguous() if 16 <= r <= 128 else a_hr_layerstack


def _tol(dtype):
    return (2e-2, 5e-3) if dtype == torch.bfloat16 else (4e-3, 1e-3)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("ranks", [[8, 8, 8], [16, 64], [8, 32, 128]])
def test_three_formulations_agree_with_fp64(dtype, ranks):
    """fallback loop, segment-wise sgmv_ref (on sorted tokens) and per-token bgmv_ref against fp64."""
    T, h_in, h_out, layer = 24, 256, 192, 1
    x, a_hr, b_rh, tok = _problem(dtype, T, h_in, h_out, ranks, drop=(3, 17))
    exact = O.lora_delta_f64(x, tok, {i: a[layer] for i, a in a_hr.items()}, {i: b[layer] for i, b in b_rh.items()})
    max_abs, rel = _tol(dtype)

    # (1) fallback loop
    lora_a = {i: _stored_a(a_hr[i], r) for i, r in enumerate(ranks)}
    y1 = torch.zeros(T, h_out, dtype=dtype)
    O.fallback_layer_type(y1, x, torch.tensor(tok), set(tok), lora_a, b_rh, layer, 0, h_out)

    # (2) per-token BGMV: shrink then expand, one rank group at a time
    y2 = torch.zeros(T, h_out, dtype=dtype)
    for r in sorted(set(ranks)):
        members = [i for i, ri in enumerate(ranks) if ri == r]
        slot = {a: s for s, a in enumerate(members)}
        indices = [slot.get(a, -1) for a in tok]
        wa_t = [a_hr[a].transpose(1, 2).contiguous() for a in members]  # [L, r, h_in]
        wb_t = [b_rh[a].transpose(1, 2).contiguous() for a in members]  # [L, h_out, r]
        v = torch.zeros(T, r, dtype=dtype)
        O.bgmv_ref(v, x, wa_t, indices, layer)
        O.bgmv_ref(y2, v, wb_t, indices, layer)

    # (3) segment-wise SGMV on the natural runs of the token order
    y3 = torch.zeros(T, h_out, dtype=dtype)
    bounds, owners = O.find_segments_ref(tok)
    for r in sorted(set(ranks)):
        segs = [s for s, a in enumerate(owners) if a >= 0 and ranks[a] == r]
        O.sgmv_ref(y3, x, [lora_a[owners[s]] for s in segs], [b_rh[owners[s]] for s in segs],
                   [bounds[s] for s in segs], [bounds[s + 1] for s in segs], layer, r)

    for y in (y1, y2, y3):
        err = (y.double() - exact).abs().max().item()
        l2 = ((y.double() - exact).norm() / exact.norm()).item()
        assert err <= max_abs and l2 <= rel, (err, l2)
        assert torch.count_nonzero(y[3]) == 0 and torch.count_nonzero(y[17]) == 0
    # the three formulations round at the same points: they may differ by accumulation order only
    assert (y1.float() - y2.float()).abs().max().item() <= max_abs / 4
    assert (y1.float() - y3.float()).abs().max().item() <= max_abs / 4


def test_fallback_masks_other_adapters_exactly():
    x, a_hr, b_rh, tok = _problem(torch.bfloat16, 12, 64, 48, [8, 16])
    lora_a = {0: _stored_a(a_hr[0], 8)}  # adapter 1 has no weights for this layer
    y = torch.full((12, 48), 0.5, dtype=torch.bfloat16)
    O.fallback_layer_type(y, x, torch.tensor(tok), {0, 1}, lora_a, {0: b_rh[0]}, 0, 0, 48)
    for t, a in enumerate(tok):
        assert torch.all(y[t] == 0.5) == (a != 0)


def test_fallback_respects_column_slice_and_layer():
    x, a_hr, b_rh, tok = _problem(torch.float16, 8, 64, 32, [16], L=3)
    lora_a = {0: _stored_a(a_hr[0], 16)}
    y = torch.zeros(8, 96, dtype=torch.float16)
    O.fallback_layer_type(y, x, torch.tensor(tok), {0}, lora_a, b_rh, 2, 32, 64)
    assert torch.count_nonzero(y[:, :32]) == 0 and torch.count_nonzero(y[:, 64:]) == 0
    exact = O.lora_delta_f64(x, tok, {0: a_hr[0][2]}, {0: b_rh[0][2]})
    assert (y[:, 32:64].double() - exact).abs().max().item() <= 4e-3
    wrong_layer = O.lora_delta_f64(x, tok, {0: a_hr[0][1]}, {0: b_rh[0][1]})
    assert (y[:, 32:64].double() - wrong_layer).abs().max().item() > 4e-3


def test_sgmv_ref_is_linear_in_b_and_skips_empty_segments():
    kat = _golden("sgmv_kat")
    torch.manual_seed(kat["seed"])
    B, H, L = kat["B"], 128, kat["nlayers"]
    for r in kat["lora_ranks"]:
        x = torch.randn(B, H, dtype=torch.float64)
        wa = torch.randn(L, r, H, dtype=torch.float64)
        if r < 16:
            wa = wa.transpose(1, 2).contiguous()
        wb = torch.randn(L, r, H, dtype=torch.float64)
        for starts, ends in kat["segments"]:
            wa_l = [wa if e - s > 0 else None for s, e in zip(starts, ends)]
            wb_l = [wb if e - s > 0 else None for s, e in zip(starts, ends)]
            y1 = O.sgmv_ref(torch.zeros(B, H, dtype=torch.float64), x, wa_l, wb_l, starts, ends, 0, r)
            wb2 = [2 * w if w is not None else None for w in wb_l]
            y2 = O.sgmv_ref(torch.zeros(B, H, dtype=torch.float64), x, wa_l, wb2, starts, ends, 0, r)
            assert torch.allclose(2 * y1, y2, rtol=1e-12, atol=1e-12)
            covered = torch.zeros(B, dtype=torch.bool)
            for s, e in zip(starts, ends):
                if e > s:
                    covered[s:e] = True
            a = wa[0] if r < 16 else wa[0].t()
            assert torch.allclose(y1[covered], (x @ a @ wb[0])[covered], rtol=1e-10, atol=1e-9)
            assert torch.count_nonzero(y1[~covered]) == 0


def test_bgmv_ref_rounds_delta_before_adding():
    # y = 256 in bf16 has ulp 2: a delta of 0.75 is lost, a delta of 1.5 rounds up to 258
    w = [torch.tensor([[[0.75], [1.5]]], dtype=torch.bfloat16)]  # [L=1, h_out=2, h_in=1]
    y = torch.full((1, 2), 256.0, dtype=torch.bfloat16)
    O.bgmv_ref(y, torch.ones(1, 1, dtype=torch.bfloat16), w, [0], 0)
    assert y.tolist() == [[256.0, 258.0]]
    y2 = torch.full((1, 2), 256.0, dtype=torch.bfloat16)
    O.bgmv_ref(y2, torch.ones(1, 1, dtype=torch.bfloat16), w, [-1], 0)
    assert y2.tolist() == [[256.0, 256.0]]
