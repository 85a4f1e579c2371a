"""The C-ABI shared library without a GPU: it loads, exports every function include/lorax_hip.h
declares, and rejects bad arguments on the host before anything is launched."""

import ctypes
import re
from pathlib import Path

import pytest

from lorax_amd import _native

ROOT = Path(__file__).resolve().parent.parent
HEADER = (ROOT / "include" / "lorax_hip.h").read_text()


def _declared_functions():
    body = re.sub(r"/\*.*?\*/", "", HEADER, flags=re.S)
    return sorted(set(re.findall(r"\b(lorax_[a-z0-9_]+)\s*\(", body)))


def test_library_loads():
    assert _native.available(), _native.load_error()
    assert "gfx950" in _native.version()


def test_every_declared_symbol_is_exported_and_bound():
    declared = _declared_functions()
    assert "lorax_bgmv" in declared and "lorax_sgmv_shrink" in declared and "lorax_sgmv_expand" in declared
    raw = ctypes.CDLL(str(_native.LIB_PATH))
    for name in declared:
        assert hasattr(raw, name), f"{name} is declared in lorax_hip.h but not exported"
    assert sorted(_native.EXPORTED_SYMBOLS) == declared


def test_tmp_size_is_60_bytes_per_problem():
    lib = _native.lib()
    assert [lib.lorax_sgmv_tmp_size(n) for n in (-1, 0, 1, 32, 257)] == [0, 0, 60, 1920, 15420]
    assert lib.lorax_workspace_bytes() == 8 * 1024 * 1024  # the static scratch of lorax_sgmv_shrink_static


OK, EINVAL, ENOKERNEL, ELAUNCH, ETMPSIZE = 0, 1, 2, 3, 4
P = 0x1000  # a non-null, 16-byte aligned fake address: validation failures return before any launch


def _err():
    return _native.lib().lorax_last_error().decode()


def test_bgmv_validation():
    f = _native.lib().lorax_bgmv
    assert f(None, None, None, None, 0, 4096, 8, 0, 8, 0, 1.0, 1, None) == OK  # nothing to do
    assert f(None, P, P, P, 4, 4096, 8, 0, 8, 0, 1.0, 1, None) == EINVAL and "null" in _err()
    assert f(P, P + 2, P, P, 4, 4096, 8, 0, 8, 0, 1.0, 1, None) == EINVAL and "aligned" in _err()
    assert f(P, P, P, P, 4, 4096, 8, 0, 8, 0, 1.0, 2, None) == ENOKERNEL and "No suitable kernel" in _err()
    for h_in, h_out in [(4096, 12), (4096, 136), (4100, 8), (65536, 8), (8, 1 << 20), (256, 256)]:
        assert f(P, P, P, P, 4, h_in, h_out, 0, h_out, 0, 1.0, 1, None) == ENOKERNEL, (h_in, h_out)
        assert f"h_in={h_in} h_out={h_out}" in _err()
    assert f(P, P, P, P, 4, 8, 4096, 8192, 8192, 0, 1.0, 1, None) == EINVAL  # window outside the row
    assert f(P, P, P, P, -1, 8, 4096, 0, 4096, 0, 1.0, 1, None) == EINVAL
    assert f(P, P, P, P, 4, 8, 4096, 0, 4096, -1, 1.0, 1, None) == EINVAL


def test_sgmv_shrink_validation():
    f = _native.lib().lorax_sgmv_shrink
    big = 8 * 1024 * 1024
    assert f(P, P, P, P, P, 2, 16, 4096, 16, 0, 0, 1.0, P, big - 1, 0, None) == ETMPSIZE and "8 * 1024 * 1024" in _err()
    assert f(P, P, P, P, P, 2, 16, 4096, 8, 1, 0, 1.0, P, 119, 0, None) == ETMPSIZE and "sgmv_tmp_size" in _err()
    assert f(P, P, P, P, P, 0, 16, 4096, 16, 0, 0, 1.0, P, big, 0, None) == OK  # no segments
    assert f(P, P, P, P, P, 2, 16, 4096, 16, 7, 0, 1.0, P, big, 0, None) == EINVAL  # layout
    for r, h_in in ((8, 4104), (24, 4104), (144, 4096), (12, 4096)):
        assert f(P, P, P, P, P, 2, 1000, h_in, r, 0, 0, 1.0, P, big, 0, None) == ENOKERNEL, r
    assert f(P, P, P, P, P, 2, 16, 4100, 16, 0, 0, 1.0, P, big, 0, None) == ENOKERNEL
    assert f(P, P, P, None, P, 2, 16, 4096, 16, 0, 0, 1.0, P, big, 0, None) == EINVAL
    assert f(P, P, P, P, P, 2, 16, 4096, 16, 0, 0, 1.0, P, big, 5, None) == ENOKERNEL  # dtype


def test_sgmv_shrink_multi_validation():
    f = _native.lib().lorax_sgmv_shrink_multi
    big = 8 * 1024 * 1024
    one = (_native.SgmvShrinkProblem * 1)(_native.SgmvShrinkProblem(P, P))
    two = (_native.SgmvShrinkProblem * 2)(_native.SgmvShrinkProblem(P, P), _native.SgmvShrinkProblem(P, P))
    assert f(two, 0, P, P, P, 2, 1000, 4096, 16, 0, 1.0, 1, P, big, None, 1, None) == EINVAL and "num_problems" in _err()
    assert f(two, 5, P, P, P, 2, 1000, 4096, 16, 0, 1.0, 1, P, big, None, 1, None) == EINVAL
    assert f(None, 2, P, P, P, 2, 1000, 4096, 16, 0, 1.0, 1, P, big, None, 1, None) == EINVAL
    # stacked launch (2 x 64 <= 128, h_in a multiple of 128, more than 512 rows): its own checks
    assert f(two, 2, P, P, P, 2, 1000, 4096, 64, 0, 1.0, 1, P, big - 1, None, 1, None) == ETMPSIZE
    assert f(two, 2, P, P, P, 0, 1000, 4096, 64, 0, 1.0, 1, P, big, None, 1, None) == OK  # no segments
    assert f(two, 2, P, P, None, 2, 1000, 4096, 64, 0, 1.0, 1, P, big, None, 1, None) == EINVAL and "null" in _err()
    assert f(two, 2, P, P, P, 2, 1000, 4096, 64, -1, 1.0, 1, P, big, None, 1, None) == EINVAL
    # one launch per projection (summed rank 192; or a single projection): lorax_sgmv_shrink's checks
    assert f(two, 2, P, P, P, 2, 1000, 4096, 96, 0, 1.0, 1, P, big - 1, None, 1, None) == ETMPSIZE
    assert f(one, 1, P, P, P, 2, 1000, 4100, 16, 0, 1.0, 1, P, big, None, 1, None) == ENOKERNEL
    assert f(two, 2, P, P, P, 2, 1000, 4096, 12, 0, 1.0, 1, P, big, None, 1, None) == ENOKERNEL
    assert f(two, 2, P, P, P, 2, 1000, 4096, 64, 0, 1.0, 2, P, big, None, 1, None) == EINVAL and "accumulate" in _err()
    assert f(two, 2, P, P, P, 0, 1000, 4096, 64, 0, 1.0, 0, P, 4 * big, None, 1, None) == OK  # a larger scratch is accepted
    # a row-tile plan: records must be aligned, the height bound at least 1
    bad = _native.SgmvTiles(P + 4, 3, 48)
    assert f(two, 2, P, P, P, 2, 1000, 4096, 64, 0, 1.0, 1, P, big, ctypes.byref(bad), 1, None) == EINVAL and "tile plan" in _err()
    bad = _native.SgmvTiles(P, 3, 0)
    assert f(two, 2, P, P, P, 2, 1000, 4096, 64, 0, 1.0, 1, P, big, ctypes.byref(bad), 1, None) == EINVAL
    empty = _native.SgmvTiles(P, 0, 16)  # a plan without tiles: nothing to do
    assert f(two, 2, P, P, P, 2, 1000, 4096, 64, 0, 1.0, 1, P, big, ctypes.byref(empty), 1, None) == OK


def test_sgmv_lora_multi_validation():
    f = _native.lib().lorax_sgmv_lora_multi
    one = (_native.SgmvLoraProblem * 1)(_native.SgmvLoraProblem(P, P, P, 0, 4096, 4096))
    assert f(one, 0, P, P, P, 2, 64, 4096, 16, 0, 1.0, 1, None) == EINVAL and "num_problems" in _err()
    assert f(one, 1, P, P, P, 0, 64, 4096, 16, 0, 1.0, 1, None) == OK  # no segments
    assert f(one, 1, P, P, None, 2, 64, 4096, 16, 0, 1.0, 1, None) == EINVAL and "null" in _err()
    assert f(one, 1, P, P, P, 2, 64, 4096, 32, 0, 1.0, 1, None) == ENOKERNEL  # rank
    assert f(one, 1, P, P, P, 2, 513, 4096, 16, 0, 1.0, 1, None) == ENOKERNEL  # too many rows
    assert f(one, 1, P, P, P, 2, 64, 4096, 16, -1, 1.0, 1, None) == EINVAL
    narrow = (_native.SgmvLoraProblem * 1)(_native.SgmvLoraProblem(P, P, P, 8, 4096, 4096))
    assert f(narrow, 1, P, P, P, 2, 64, 4096, 16, 0, 1.0, 1, None) == EINVAL and "y_offset" in _err()
    no_b = (_native.SgmvLoraProblem * 1)(_native.SgmvLoraProblem(P, P, None, 0, 4096, 4096))
    assert f(no_b, 1, P, P, P, 2, 64, 4096, 16, 0, 1.0, 1, None) == EINVAL


def test_sgmv_expand_validation():
    f = _native.lib().lorax_sgmv_expand
    for layout in (_native.B_RH, _native.B_HR):
        assert f(P, P, P, P, P, 2, 16, 16, 4096, layout, 0, 4096, 0, 1, P, 121, 1, None) == ETMPSIZE
        assert f(P, P, P, P, P, 0, 16, 16, 4096, layout, 0, 4096, 0, 1, None, 0, 1, None) == OK
        for r, h in [(4, 4096), (136, 4096), (16, 4100)]:
            assert f(P, P, P, P, P, 2, 16, r, h, layout, 0, h, 0, 1, P, 120, 1, None) == ENOKERNEL, (r, h)
        assert f(P, P, P, P, P, 2, 16, 16, 4096, layout, 4, 8192, 0, 1, P, 120, 1, None) == EINVAL  # unaligned window
        assert f(P, P, P, P, P, 2, 16, 16, 4096, layout, 4096, 4096, 0, 1, P, 120, 1, None) == EINVAL  # too wide
        assert f(P, P, P, P, P, 2, 16, 16, 4096, layout, 0, 1 << 24, 0, 1, P, 120, 1, None) == EINVAL  # row pitch
        assert "2^24" in _err()
    assert f(P, P, P, P, P, 2, 16, 16, 4096, 2, 0, 4096, 0, 1, P, 120, 1, None) == EINVAL  # unknown layout


def test_sgmv_expand_planned_validation():
    f = _native.lib().lorax_sgmv_expand_planned
    assert f(P, P, P, P, P, 0, 16, 16, 4096, 0, 4096, 0, 1, None, 1, None) == OK  # no segments
    assert f(P, P, P, P, P, 2, 16, 12, 4096, 0, 4096, 0, 1, None, 1, None) == ENOKERNEL
    assert f(P, P, P, P, None, 2, 16, 16, 4096, 0, 4096, 0, 1, None, 1, None) == EINVAL
    bad = _native.SgmvTiles(P, -1, 256)
    assert f(P, P, P, P, P, 2, 16, 16, 4096, 0, 4096, 0, 1, ctypes.byref(bad), 1, None) == EINVAL and "tile plan" in _err()
    empty = _native.SgmvTiles(P, 0, 256)
    assert f(P, P, P, P, P, 2, 16, 16, 4096, 0, 4096, 0, 1, ctypes.byref(empty), 1, None) == OK


def test_plan_tiles_cuts_every_row_once():
    """lorax_sgmv_plan_tiles (host only): every row of every non-empty segment in exactly one tile, tiles inside
    their segment and no higher than the bound, numbered inside the segment; empty and negative segments get none."""
    starts = [5, 100, 100, -1, 400, 2000]
    ends = [47, 100, 90, -1, 1500, 2003]
    T = 2500
    for kind, limit in ((_native.TILES_SHRINK, 64), (_native.TILES_EXPAND, 256 + 32 + 16)):
        records, tile_rows = _native.plan_tiles(starts, ends, T, kind)
        assert tile_rows <= limit
        covered = {}
        last_index = {}
        for seg, row0, row_end, index in records.tolist():
            assert starts[seg] <= row0 < row_end <= ends[seg] and row_end - row0 <= tile_rows
            assert index == last_index.get(seg, -1) + 1
            last_index[seg] = index
            for row in range(row0, row_end):
                assert row not in covered
                covered[row] = seg
        want = {row: seg for seg, (s, e) in enumerate(zip(starts, ends)) for row in range(max(s, 0), min(e, T))}
        assert covered == want
    # bounds beyond the batch are clamped; a table without rows gives an empty plan
    records, _ = _native.plan_tiles([10], [100], 50, _native.TILES_SHRINK)
    assert records[:, 2].max() == 50
    records, _ = _native.plan_tiles([3, -1], [3, -1], 50, _native.TILES_EXPAND)
    assert records.shape == (0, 4)
    # a thousand rows in ten segments: low tiles (the launch also cuts the hidden dimension); a long batch: 64 rows
    records, tile_rows = _native.plan_tiles(list(range(0, 1000, 100)), list(range(100, 1100, 100)), 1000, _native.TILES_SHRINK)
    assert tile_rows == 16 and len(records) == 70
    records, tile_rows = _native.plan_tiles([0], [40000], 40000, _native.TILES_SHRINK)
    assert tile_rows == 64 and len(records) == 625
    # tiles are not lowered below a quarter of the rank: 4096 rows at rank 128 stay at 32 rows (128 tiles), at rank
    # 64 they go down to 16 (256 tiles, one per CU)
    assert _native.plan_tiles([0], [4096], 4096, _native.TILES_SHRINK, 128)[1] == 32
    assert _native.plan_tiles([0], [4096], 4096, _native.TILES_SHRINK, 64)[1] == 16


def test_python_binding_rejects_cpu_tensors():
    import torch

    y = torch.zeros(2, 8, dtype=torch.float16)
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        _native.dispatch_bgmv(y, y, torch.zeros(1, dtype=torch.int64), torch.zeros(2, dtype=torch.int64), 0, 1.0)
