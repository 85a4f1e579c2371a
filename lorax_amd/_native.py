"""ctypes binding of liblorax_hip.so with the call signatures of the reference's pybind
module ``punica_kernels`` (server/punica_kernels/punica_kernels/punica_ops.cc:446-459):
``dispatch_bgmv``, ``sgmv_cutlass``, ``sgmv_shrink`` and ``sgmv_cutlass_tmp_size``.

The functions take torch tensors, perform the checks the reference performs with
TORCH_CHECK (punica_ops.cc:36-43, 291-411) and raise ``RuntimeError`` on any failure.
There is no other implementation behind them: if the shared library is missing every
call raises.
"""

import ctypes
import os
from pathlib import Path
from typing import Optional

import torch  # noqa: F401  (must be imported first so that its HIP runtime is the one in the process)

LIB_PATH = Path(__file__).resolve().parent / "liblorax_hip.so"

F16, BF16 = 0, 1
ESPACE = 5
A_RH, A_HR = 0, 1
B_RH, B_HR = 0, 1
SHRINK_TMP_BYTES = 8 * 1024 * 1024

_c = ctypes


class BgmvProblem(ctypes.Structure):
    """lorax_bgmv_problem_t of include/lorax_hip.h."""

    _fields_ = [
        ("y", _c.c_void_p),
        ("x", _c.c_void_p),
        ("w_ptrs", _c.c_void_p),
        ("indices", _c.c_void_p),
        ("y_offset", _c.c_int64),
        ("y_stride", _c.c_int64),
        ("h_out", _c.c_int32),
        ("plan", _c.c_void_p),
        ("num_groups", _c.c_int32),
        ("h_in", _c.c_int32),
        ("a_stack", _c.c_void_p),
        ("b_stack", _c.c_void_p),
    ]


class SgmvShrinkProblem(ctypes.Structure):
    """lorax_sgmv_shrink_problem_t of include/lorax_hip.h."""

    _fields_ = [("v", _c.c_void_p), ("w_ptrs", _c.c_void_p)]


class SgmvLoraProblem(ctypes.Structure):
    """lorax_sgmv_lora_problem_t of include/lorax_hip.h."""

    _fields_ = [("y", _c.c_void_p), ("a_ptrs", _c.c_void_p), ("b_ptrs", _c.c_void_p), ("y_offset", _c.c_int64),
                ("y_stride", _c.c_int64), ("h_out", _c.c_int32)]


class AdapterEntry(ctypes.Structure):
    """lorax_adapter_entry_t of include/lorax_hip.h."""

    _fields_ = [("adapter", _c.c_int64), ("a_addr", _c.c_int64), ("b_addr", _c.c_int64), ("rank", _c.c_int32),
                ("reserved", _c.c_int32)]


class TableGroup(ctypes.Structure):
    """lorax_table_group_t of include/lorax_hip.h."""

    _fields_ = [("layer_type", _c.c_int32), ("rank", _c.c_int32), ("use_sgmv", _c.c_int32),
                ("num_segments", _c.c_int32), ("num_chunks", _c.c_int32), ("num_long_segments", _c.c_int32),
                ("a_ptr_off", _c.c_int64), ("b_ptr_off", _c.c_int64), ("starts_off", _c.c_int64),
                ("ends_off", _c.c_int64), ("indices_off", _c.c_int64), ("plan_off", _c.c_int64),
                ("shrink_tiles_off", _c.c_int64), ("expand_tiles_off", _c.c_int64),
                ("num_shrink_tiles", _c.c_int32), ("shrink_tile_rows", _c.c_int32),
                ("num_expand_tiles", _c.c_int32), ("expand_tile_rows", _c.c_int32)]


class SgmvTiles(ctypes.Structure):
    """lorax_sgmv_tiles_t of include/lorax_hip.h."""

    _fields_ = [("tiles", _c.c_void_p), ("num_tiles", _c.c_int32), ("tile_rows", _c.c_int32)]


TILES_SHRINK, TILES_EXPAND = 0, 1


class TilePlan:
    """A row-tile plan of an SGMV launch: `records` is an int32 [num_tiles, 4] tensor on the launch's device
    (seg, row0, row_end, index per tile), `tile_rows` the bound of the tiles' heights."""

    __slots__ = ("records", "num_tiles", "tile_rows")

    def __init__(self, records: torch.Tensor, tile_rows: int):
        if records.dtype != torch.int32 or records.dim() != 2 or records.size(1) != 4 or not records.is_contiguous():
            raise RuntimeError("tile records must be a contiguous int32 [num_tiles, 4] tensor")
        self.records = records
        self.num_tiles = records.size(0)
        self.tile_rows = int(tile_rows)

    def c_struct(self, device) -> "SgmvTiles":
        if self.records.device != device:
            raise RuntimeError(f"tile plan on {self.records.device}, launch on {device}")
        # (a plan without tiles has no storage; any non-null address marks it as a plan)
        addr = self.records.data_ptr() if self.num_tiles > 0 else 16
        return SgmvTiles(addr, self.num_tiles, self.tile_rows)


MAX_BGMV_PROBLEMS = 16
MAX_BGMV_TOKENS = 65535  # rows of a BGMV launch and records of one routing plan (capi.hip: bgmv_batch)
MAX_FUSED_BGMV_PROBLEMS = 4

_SIGNATURES = {
    "lorax_bgmv": (
        _c.c_int,
        [_c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_int64, _c.c_int32, _c.c_int32,
         _c.c_int64, _c.c_int64, _c.c_int64, _c.c_float, _c.c_int32, _c.c_void_p],
    ),
    "lorax_bgmv_multi": (
        _c.c_int,
        [_c.POINTER(BgmvProblem), _c.c_int32, _c.c_int64, _c.c_int32, _c.c_int64, _c.c_float, _c.c_int32,
         _c.c_int32, _c.c_void_p],
    ),
    "lorax_bgmv_lora_multi": (
        _c.c_int,
        [_c.POINTER(BgmvProblem), _c.c_int32, _c.c_int64, _c.c_int32, _c.c_int32, _c.c_int64, _c.c_float,
         _c.c_int32, _c.c_void_p],
    ),
    "lorax_sgmv_shrink": (
        _c.c_int,
        [_c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_int32, _c.c_int64,
         _c.c_int32, _c.c_int32, _c.c_int32, _c.c_int64, _c.c_float, _c.c_void_p, _c.c_int64, _c.c_int32,
         _c.c_void_p],
    ),
    "lorax_sgmv_shrink_static": (
        _c.c_int,
        [_c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_int32, _c.c_int64,
         _c.c_int32, _c.c_int32, _c.c_int32, _c.c_int64, _c.c_float, _c.c_int32, _c.c_void_p],
    ),
    "lorax_sgmv_shrink_multi": (
        _c.c_int,
        [_c.POINTER(SgmvShrinkProblem), _c.c_int32, _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_int32, _c.c_int64,
         _c.c_int32, _c.c_int32, _c.c_int64, _c.c_float, _c.c_int32, _c.c_void_p, _c.c_int64, _c.POINTER(SgmvTiles),
         _c.c_int32, _c.c_void_p],
    ),
    "lorax_sgmv_expand_planned": (
        _c.c_int,
        [_c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_int32, _c.c_int64, _c.c_int32,
         _c.c_int32, _c.c_int64, _c.c_int64, _c.c_int64, _c.c_int32, _c.POINTER(SgmvTiles), _c.c_int32, _c.c_void_p],
    ),
    "lorax_sgmv_plan_tiles": (
        _c.c_int,
        [_c.c_void_p, _c.c_void_p, _c.c_int32, _c.c_int64, _c.c_int32, _c.c_int32, _c.c_void_p, _c.c_int32,
         _c.POINTER(_c.c_int32), _c.POINTER(_c.c_int32)],
    ),
    "lorax_set_fixed_order_shrink": (_c.c_int, [_c.c_int32]),
    "lorax_sgmv_lora_multi": (
        _c.c_int,
        [_c.POINTER(SgmvLoraProblem), _c.c_int32, _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_int32, _c.c_int64,
         _c.c_int32, _c.c_int32, _c.c_int64, _c.c_float, _c.c_int32, _c.c_void_p],
    ),
    "lorax_sgmv_expand": (
        _c.c_int,
        [_c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_void_p, _c.c_int32, _c.c_int64,
         _c.c_int32, _c.c_int32, _c.c_int32, _c.c_int64, _c.c_int64, _c.c_int64, _c.c_int32, _c.c_void_p,
         _c.c_int64, _c.c_int32, _c.c_void_p],
    ),
    "lorax_sgmv_tmp_size": (_c.c_size_t, [_c.c_int32]),
    "lorax_build_batch_tables": (
        _c.c_int,
        [_c.c_void_p, _c.c_int64, _c.c_void_p, _c.c_void_p, _c.c_int32, _c.c_int32, _c.c_void_p, _c.c_void_p,
         _c.POINTER(_c.c_int32), _c.c_void_p, _c.c_int64, _c.POINTER(_c.c_int64), _c.POINTER(TableGroup), _c.c_int32,
         _c.POINTER(_c.c_int32)],
    ),
    "lorax_init": (_c.c_int, [_c.c_int32]),
    "lorax_workspace_bytes": (_c.c_size_t, []),
    "lorax_last_error": (_c.c_char_p, []),
    "lorax_version": (_c.c_char_p, []),
}

EXPORTED_SYMBOLS = tuple(_SIGNATURES)

_lib: Optional[ctypes.CDLL] = None
_load_error: Optional[str] = None
_initialised_devices = set()


def _load() -> Optional[ctypes.CDLL]:
    global _lib, _load_error
    if _lib is not None or _load_error is not None:
        return _lib
    path = os.environ.get("LORAX_HIP_LIBRARY", str(LIB_PATH))
    try:
        lib = ctypes.CDLL(path)
        for name, (restype, argtypes) in _SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = lib
    except (OSError, AttributeError) as exc:
        _load_error = f"{path}: {exc}"
    return _lib


def available() -> bool:
    """True iff liblorax_hip.so is loaded with every expected symbol."""
    return _load() is not None


def load_error() -> Optional[str]:
    _load()
    return _load_error


def lib() -> ctypes.CDLL:
    handle = _load()
    if handle is None:
        raise RuntimeError(
            f"liblorax_hip.so is not available ({_load_error}); build it with `python -m lorax_amd.build`. "
            "There is no non-HIP implementation of the LoRA kernels in this package."
        )
    return handle


def version() -> str:
    return lib().lorax_version().decode()


def _raise_last(rc: int):
    msg = lib().lorax_last_error().decode() or f"error code {rc}"
    raise RuntimeError(msg)


def init(device) -> None:
    """lorax_init: per-device set-up of the library (idempotent; call it outside graph capture)."""
    index = torch.device(device).index
    if index is None:
        index = torch.cuda.current_device()
    if index in _initialised_devices:
        return
    rc = lib().lorax_init(index)
    if rc != 0:
        _raise_last(rc)
    _initialised_devices.add(index)


def _dtype_code(t: torch.Tensor) -> int:
    if t.dtype == torch.float16:
        return F16
    if t.dtype == torch.bfloat16:
        return BF16
    return -1


def _check_input(t: torch.Tensor, name: str, dim: int) -> None:
    if not isinstance(t, torch.Tensor):
        raise RuntimeError(f"{name} must be a torch.Tensor")
    if not t.is_cuda:
        raise RuntimeError(f"{name} must be a CUDA tensor")
    if not t.is_contiguous():
        raise RuntimeError(f"{name} must be contiguous")
    if t.dim() != dim:
        raise RuntimeError(f"{name} must be a {dim}D tensor")


def _stream(t: torch.Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


def _check_same(y: torch.Tensor, x: torch.Tensor, *rest: torch.Tensor) -> None:
    if y.dtype != x.dtype:
        raise RuntimeError(f"y and x must share one dtype, got {y.dtype} and {x.dtype}")
    for t in rest:
        if t.device != x.device:
            raise RuntimeError(f"all tensors must be on one device, got {t.device} and {x.device}")
    if y.device != x.device:
        raise RuntimeError(f"all tensors must be on one device, got {y.device} and {x.device}")


def sgmv_cutlass_tmp_size(num_problems: int) -> int:
    """sgmv_tmp_size, sgmv/sgmv_cutlass.cuh:54-58."""
    return int(lib().lorax_sgmv_tmp_size(int(num_problems)))


def bgmv(y, x, w_ptr, indicies, layer_idx, scale, y_offset=0, y_slice_size=None) -> None:
    """lorax_bgmv with an optional column window [y_offset, y_offset + y_slice_size) of y."""
    _check_input(y, "y", 2)
    _check_input(x, "x", 2)
    _check_input(w_ptr, "w_ptr", 1)
    _check_input(indicies, "indicies", 1)
    _check_same(y, x, w_ptr, indicies)
    if w_ptr.dtype != torch.int64 or indicies.dtype != torch.int64:
        raise RuntimeError("w_ptr and indicies must be int64 tensors")
    if indicies.size(0) != x.size(0):
        raise RuntimeError(f"CHECK_EQ(indicies.size(0), x.size(0)) failed. {indicies.size(0)} vs {x.size(0)}")
    if y.size(0) != x.size(0):
        raise RuntimeError(f"CHECK_EQ(y.size(0), x.size(0)) failed. {y.size(0)} vs {x.size(0)}")
    h_out = y.size(1) if y_slice_size is None else int(y_slice_size)
    with torch.cuda.device(x.device):
        rc = lib().lorax_bgmv(
            y.data_ptr(), x.data_ptr(), w_ptr.data_ptr(), indicies.data_ptr(), x.size(0), x.size(1), h_out,
            int(y_offset), y.size(1), int(layer_idx), float(scale), _dtype_code(x), _stream(x),
        )
    if rc != 0:
        _raise_last(rc)


PLAN_RECORD_WORDS = 8


def bgmv_multi(problems, layer_idx, scale=1.0, accumulate=True, plans=None, stacks=None) -> None:
    """lorax_bgmv_multi: `problems` is a list of up to 16 tuples (y, x, w_ptr, indicies, y_offset, y_slice_size)
    that share the token count and the direction; shrink problems share x.shape and may differ in rank
    (y's width), expand problems may differ in rank (x's width) and output width.  y_slice_size None means
    the whole width of y.
    `plans`, if given, holds one routing plan per problem: an int64 device tensor [num_groups, 8]; w_ptr and
    indicies of a planned problem may then be None (the kernels read the plan only).
    `stacks` (with plans): per problem the stacked weight tensor [num_adapters, rows, cols] whose entry numbers the
    plan's address words hold - lora_a stacks for a shrink launch, lora_b stacks for an expand launch."""
    if not 1 <= len(problems) <= MAX_BGMV_PROBLEMS:
        raise RuntimeError(f"between 1 and {MAX_BGMV_PROBLEMS} problems per launch, got {len(problems)}")
    arr = (BgmvProblem * len(problems))()
    x0 = problems[0][1]
    for i, (y, x, w_ptr, indicies, y_offset, y_slice_size) in enumerate(problems):
        _check_input(y, "y", 2)
        _check_input(x, "x", 2)
        planned_only = plans is not None and w_ptr is None and indicies is None  # the plan holds the routing
        if planned_only:
            _check_same(y, x)
        else:
            _check_input(w_ptr, "w_ptr", 1)
            _check_input(indicies, "indicies", 1)
            _check_same(y, x, w_ptr, indicies)
            if w_ptr.dtype != torch.int64 or indicies.dtype != torch.int64:
                raise RuntimeError("w_ptr and indicies must be int64 tensors")
        if x.size(0) != x0.size(0) or x.dtype != x0.dtype or x.device != x0.device:
            raise RuntimeError("all problems of one launch must have inputs of one row count, dtype and device")
        if (not planned_only and indicies.size(0) != x.size(0)) or y.size(0) != x.size(0):
            raise RuntimeError(
                f"CHECK_EQ(indicies.size(0), x.size(0)) / CHECK_EQ(y.size(0), x.size(0)) failed. "
                f"{'-' if planned_only else indicies.size(0)}, {y.size(0)} vs {x.size(0)}"
            )
        h_out = y.size(1) if y_slice_size is None else int(y_slice_size)
        plan_ptr, num_groups = None, 0
        if plans is not None:
            plan = plans[i]
            _check_input(plan, "plan", 2)
            if plan.dtype != torch.int64 or plan.size(1) != PLAN_RECORD_WORDS or plan.device != x.device:
                raise RuntimeError(f"plan must be an int64 [num_groups, {PLAN_RECORD_WORDS}] tensor on the device of x")
            plan_ptr, num_groups = plan.data_ptr(), plan.size(0)
            if num_groups == 0:
                plan_ptr = x.data_ptr()  # an empty plan has no storage; any non-null address will do
        stack = None
        if stacks is not None and plans is not None:
            _check_stack(stacks[i], x)
            stack = stacks[i].data_ptr()
        arr[i] = BgmvProblem(y.data_ptr(), x.data_ptr(), None if planned_only else w_ptr.data_ptr(),
                             None if planned_only else indicies.data_ptr(), int(y_offset),
                             y.size(1), h_out, plan_ptr, num_groups, x.size(1), stack, stack)
    with torch.cuda.device(x0.device):
        rc = lib().lorax_bgmv_multi(arr, len(problems), x0.size(0), x0.size(1), int(layer_idx), float(scale),
                                    1 if accumulate else 0, _dtype_code(x0), _stream(x0))
    if rc != 0:
        _raise_last(rc)


FUSED_BGMV_RANKS = (8, 16)


def bgmv_lora_fits(rank: int, h_in: int, h_out: int) -> bool:
    """True where the single-launch shrink+expand (lorax_bgmv_lora_multi) is the better choice: the adapter's
    A slab is small (<= 128 KiB) and one workgroup covers all output columns of the projection (4096 at
    rank 8, 2048 at rank 16), so no column slice has to repeat the shrink. Wider or deeper projections are
    faster as a shrink launch plus an expand launch."""
    if rank not in FUSED_BGMV_RANKS:
        return False
    return rank * h_in * 2 <= 128 * 1024 and h_out <= (256 // (rank // 8)) * 16


def _check_stack(stack, x) -> None:
    if not isinstance(stack, torch.Tensor) or stack.dim() != 3 or not stack.is_contiguous() or stack.dtype != x.dtype \
            or stack.device != x.device:
        raise RuntimeError("stacked weights must be a contiguous [num_adapters, rows, cols] tensor of the input's "
                           "dtype on its device")


def bgmv_lora_multi(problems, rank, layer_idx, scale=1.0, stacks=None) -> None:
    """lorax_bgmv_lora_multi: `problems` is a list of up to 4 tuples (y, x, plan, y_offset, y_slice_size) that
    share x.shape; y[:, window] += (x @ A^T) @ B^T per planned token chunk, rank 8 or 16.
    `stacks`: per problem a pair (lora_a [num_adapters, r, h_in], lora_b [num_adapters, h_out, r]) of stacked weight
    tensors; the plan's address words then hold entry numbers and layer_idx must be 0."""
    if not 1 <= len(problems) <= MAX_FUSED_BGMV_PROBLEMS:
        raise RuntimeError(f"between 1 and {MAX_FUSED_BGMV_PROBLEMS} problems per launch, got {len(problems)}")
    arr = (BgmvProblem * len(problems))()
    x0 = problems[0][1]
    for i, (y, x, plan, y_offset, y_slice_size) in enumerate(problems):
        _check_input(y, "y", 2)
        _check_input(x, "x", 2)
        _check_input(plan, "plan", 2)
        _check_same(y, x, plan)
        if x.shape != x0.shape or x.dtype != x0.dtype or x.device != x0.device:
            raise RuntimeError("all problems of one launch must have inputs of one shape, dtype and device")
        if y.size(0) != x.size(0):
            raise RuntimeError(f"CHECK_EQ(y.size(0), x.size(0)) failed. {y.size(0)} vs {x.size(0)}")
        if plan.dtype != torch.int64 or plan.size(1) != PLAN_RECORD_WORDS:
            raise RuntimeError(f"plan must be an int64 [num_groups, {PLAN_RECORD_WORDS}] tensor on the device of x")
        h_out = y.size(1) if y_slice_size is None else int(y_slice_size)
        plan_ptr = plan.data_ptr() if plan.size(0) > 0 else x.data_ptr()
        a_stack = b_stack = None
        if stacks is not None:
            if int(layer_idx) != 0:
                raise RuntimeError("stacked weights hold one layer: layer_idx must be 0")
            _check_stack(stacks[i][0], x)
            _check_stack(stacks[i][1], x)
            if stacks[i][0].shape[1:] != (rank, x.size(1)) or stacks[i][1].shape[1:] != (h_out, rank):
                raise RuntimeError(f"stacked weights of problem {i} do not have the shapes [n, {rank}, {x.size(1)}] "
                                   f"and [n, {h_out}, {rank}]")
            a_stack, b_stack = stacks[i][0].data_ptr(), stacks[i][1].data_ptr()
        arr[i] = BgmvProblem(y.data_ptr(), x.data_ptr(), None, None, int(y_offset), y.size(1), h_out, plan_ptr,
                             plan.size(0), 0, a_stack, b_stack)
    with torch.cuda.device(x0.device):
        rc = lib().lorax_bgmv_lora_multi(arr, len(problems), x0.size(0), x0.size(1), int(rank), int(layer_idx),
                                         float(scale), _dtype_code(x0), _stream(x0))
    if rc != 0:
        _raise_last(rc)


def dispatch_bgmv(y, x, w_ptr, indicies, layer_idx, scale) -> None:
    """dispatch_bgmv, punica_ops.cc:291-334."""
    bgmv(y, x, w_ptr, indicies, layer_idx, scale)


def _check_sgmv(y, x, w_ptr, s_start, s_end, tmp) -> None:
    _check_input(y, "y", 2)
    _check_input(x, "x", 2)
    _check_input(w_ptr, "w_ptr", 1)
    _check_input(s_start, "s_start", 1)
    _check_input(s_end, "s_end", 1)
    _check_input(tmp, "tmp", 1)
    _check_same(y, x, w_ptr, s_start, s_end, tmp)
    if w_ptr.dtype != torch.int64:
        raise RuntimeError("w_ptr must be an int64 tensor")
    if s_start.dtype != torch.int32 or s_end.dtype != torch.int32:
        raise RuntimeError("s_start and s_end must be int32 tensors")
    if not (w_ptr.size(0) == s_start.size(0) == s_end.size(0)):
        raise RuntimeError(
            f"w_ptr, s_start and s_end must have one entry per segment, got {w_ptr.size(0)}, "
            f"{s_start.size(0)}, {s_end.size(0)}"
        )
    if y.size(0) != x.size(0):
        raise RuntimeError(f"CHECK_EQ(y.size(0), x.size(0)) failed. {y.size(0)} vs {x.size(0)}")


def sgmv_expand(y, x, w_ptr, s_start, s_end, tmp, layer_idx, y_offset=0, y_slice_size=None,
                transposed: bool = False, accumulate: bool = True, tiles: Optional[TilePlan] = None) -> None:
    """lorax_sgmv_expand with an optional column window of y.  `transposed`: w_ptr addresses [L, h_out, r]
    stacks (B^T) instead of the reference's [L, r, h_out].  accumulate=False overwrites the segments' rows.
    `tiles`: a row-tile plan of the segment tables (transposed stacks only: lorax_sgmv_expand_planned)."""
    _check_sgmv(y, x, w_ptr, s_start, s_end, tmp)
    h_out = y.size(1) if y_slice_size is None else int(y_slice_size)
    if tiles is not None and transposed:
        plan = tiles.c_struct(x.device)
        with torch.cuda.device(x.device):
            rc = lib().lorax_sgmv_expand_planned(
                y.data_ptr(), x.data_ptr(), w_ptr.data_ptr(), s_start.data_ptr(), s_end.data_ptr(), s_start.size(0),
                x.size(0), x.size(1), h_out, int(y_offset), y.size(1), int(layer_idx), 1 if accumulate else 0,
                ctypes.byref(plan), _dtype_code(x), _stream(x),
            )
        if rc != 0:
            _raise_last(rc)
        return
    with torch.cuda.device(x.device):
        rc = lib().lorax_sgmv_expand(
            y.data_ptr(), x.data_ptr(), w_ptr.data_ptr(), s_start.data_ptr(), s_end.data_ptr(), s_start.size(0),
            x.size(0), x.size(1), h_out, B_HR if transposed else B_RH, int(y_offset), y.size(1), int(layer_idx),
            1 if accumulate else 0, tmp.data_ptr(),
            tmp.numel() * tmp.element_size(), _dtype_code(x), _stream(x),
        )
    if rc != 0:
        _raise_last(rc)


def _sgmv_shrink(y, x, w_ptr, s_start, s_end, tmp, layer_idx, a_layout, scale: float = 1.0) -> None:
    _check_sgmv(y, x, w_ptr, s_start, s_end, tmp)
    if not torch.cuda.is_current_stream_capturing():
        init(x.device)
    with torch.cuda.device(x.device):
        rc = lib().lorax_sgmv_shrink(
            y.data_ptr(), x.data_ptr(), w_ptr.data_ptr(), s_start.data_ptr(), s_end.data_ptr(), s_start.size(0),
            x.size(0), x.size(1), y.size(1), a_layout, int(layer_idx), float(scale), tmp.data_ptr(),
            tmp.numel() * tmp.element_size(), _dtype_code(x), _stream(x),
        )
    if rc != 0:
        _raise_last(rc)


def sgmv_cutlass(y, x, w_ptr, s_start, s_end, tmp, layer_idx) -> None:
    """dispatch_sgmv_cutlass, punica_ops.cc:338-367: weights are [L, d_in, d_out]; d_in < d_out is the
    expand configuration, anything else the shrink one (sgmv_cutlass.cuh:86,132)."""
    if isinstance(x, torch.Tensor) and isinstance(y, torch.Tensor) and x.dim() == 2 and y.dim() == 2:
        if x.size(1) < y.size(1):
            return sgmv_expand(y, x, w_ptr, s_start, s_end, tmp, layer_idx)
    return _sgmv_shrink(y, x, w_ptr, s_start, s_end, tmp, layer_idx, A_HR)


def sgmv_shrink(y, x, w_ptr, s_start, s_end, tmp, layer_idx, scale: float = 1.0) -> None:
    """dispatch_sgmv_shrink, punica_ops.cc:369-411: weights are [L, d_out, d_in], tmp is 8 MiB of uint8.
    `scale` (not in the reference's binding) multiplies the sums before they are rounded."""
    if isinstance(tmp, torch.Tensor) and tmp.dtype != torch.uint8:
        raise RuntimeError(f"CHECK_EQ(tmp.scalar_type(), at::ScalarType::Byte) failed. {tmp.dtype}")
    return _sgmv_shrink(y, x, w_ptr, s_start, s_end, tmp, layer_idx, A_RH, scale)


def sgmv_shrink_static(y, x, w_ptr, s_start, s_end, layer_idx, a_layout=A_RH, scale: float = 1.0) -> None:
    """lorax_sgmv_shrink_static: sgmv_shrink / the shrink direction of sgmv_cutlass without a tmp tensor; the
    library's own static device array serves as split-K scratch, so the call allocates nothing."""
    _check_sgmv(y, x, w_ptr, s_start, s_end, s_start)
    with torch.cuda.device(x.device):
        rc = lib().lorax_sgmv_shrink_static(
            y.data_ptr(), x.data_ptr(), w_ptr.data_ptr(), s_start.data_ptr(), s_end.data_ptr(), s_start.size(0),
            x.size(0), x.size(1), y.size(1), a_layout, int(layer_idx), float(scale), _dtype_code(x), _stream(x),
        )
    if rc != 0:
        _raise_last(rc)


MAX_SGMV_SHRINK_PROBLEMS = 4


def sgmv_shrink_multi(ys, x, w_ptrs, s_start, s_end, tmp, layer_idx, scale: float = 1.0,
                      accumulate: bool = True, tiles: Optional[TilePlan] = None) -> None:
    """lorax_sgmv_shrink_multi: sgmv_shrink for up to 4 projections (outputs `ys`, pointer tables `w_ptrs`) that
    share x, the segment tables and the rank; one launch that reads x once where the kernels allow it.
    accumulate=False overwrites the rows of the segments (no zero-fill of the outputs needed).
    `tiles`: a row-tile plan of the segment tables (plan_tiles, or the batch tables' own)."""
    if not 1 <= len(ys) <= MAX_SGMV_SHRINK_PROBLEMS or len(ys) != len(w_ptrs):
        raise RuntimeError(f"between 1 and {MAX_SGMV_SHRINK_PROBLEMS} outputs with one pointer table each")
    if isinstance(tmp, torch.Tensor) and tmp.dtype != torch.uint8:
        raise RuntimeError(f"CHECK_EQ(tmp.scalar_type(), at::ScalarType::Byte) failed. {tmp.dtype}")
    arr = (SgmvShrinkProblem * len(ys))()
    for i, (y, w_ptr) in enumerate(zip(ys, w_ptrs)):
        _check_sgmv(y, x, w_ptr, s_start, s_end, tmp)
        if y.size(1) != ys[0].size(1):
            raise RuntimeError("the projections of one call share the rank")
        arr[i] = SgmvShrinkProblem(y.data_ptr(), w_ptr.data_ptr())
    if not torch.cuda.is_current_stream_capturing():
        init(x.device)
    plan = tiles.c_struct(x.device) if tiles is not None else None
    with torch.cuda.device(x.device):
        rc = lib().lorax_sgmv_shrink_multi(
            arr, len(ys), x.data_ptr(), s_start.data_ptr(), s_end.data_ptr(), s_start.size(0), x.size(0), x.size(1),
            ys[0].size(1), int(layer_idx), float(scale), 1 if accumulate else 0, tmp.data_ptr(),
            tmp.numel() * tmp.element_size(), ctypes.byref(plan) if plan is not None else None, _dtype_code(x),
            _stream(x),
        )
    if rc != 0:
        _raise_last(rc)


def plan_tiles(s_start, s_end, num_tokens: int, kind: int, rank: int = 0):
    """lorax_sgmv_plan_tiles on host copies of the segment tables (sequences of int): returns (records as a numpy
    int32 [num_tiles, 4] array, tile_rows).  `rank`: the LoRA rank of the launch, 0 = unknown."""
    import numpy as np

    starts = np.ascontiguousarray(s_start, dtype=np.int32)
    ends = np.ascontiguousarray(s_end, dtype=np.int32)
    if starts.shape != ends.shape or starts.ndim != 1:
        raise RuntimeError("s_start and s_end must be one-dimensional and of one length")
    n, rows = _c.c_int32(0), _c.c_int32(0)
    capacity = max(16, int(num_tokens) // 16 + 2 * starts.shape[0])
    while True:
        records = np.empty((capacity, 4), dtype=np.int32)
        rc = lib().lorax_sgmv_plan_tiles(starts.ctypes.data, ends.ctypes.data, starts.shape[0], int(num_tokens),
                                         int(kind), int(rank), records.ctypes.data, capacity, ctypes.byref(n),
                                         ctypes.byref(rows))
        if rc == ESPACE:
            capacity = int(n.value)
            continue
        if rc != 0:
            raise RuntimeError(f"lorax_sgmv_plan_tiles failed with code {rc}")
        return records[: n.value], int(rows.value)


def set_fixed_order_shrink(on: bool) -> bool:
    """lorax_set_fixed_order_shrink: the SGMV shrinks add their sums over the hidden dimension in one fixed order
    whatever the batch (slower on some shapes).  Returns the previous setting."""
    return bool(lib().lorax_set_fixed_order_shrink(1 if on else 0))


SGMV_LORA_MAX_TOKENS = 512


def sgmv_lora_fits(rank: int, h_in: int, num_tokens: int, h_out: int = 0) -> bool:
    """True where the single-launch prefill update (lorax_sgmv_lora_multi) applies and pays: rank 8 or 16 with a
    small A slab, a batch short enough to be bound by launches, and an output that is not so wide (an LM head)
    that recomputing the shrink in every column slice would dominate."""
    return (rank in FUSED_BGMV_RANKS and rank * h_in * 2 <= 128 * 1024 and num_tokens <= SGMV_LORA_MAX_TOKENS
            and h_out <= 16384)


def sgmv_lora_multi(problems, x, s_start, s_end, rank, layer_idx, scale: float = 1.0) -> None:
    """lorax_sgmv_lora_multi: `problems` is a list of up to 4 tuples (y, a_t_ptr, b_t_ptr, y_offset, y_slice_size)
    whose projections share x and the segment tables; y[s:e, window] += (x[s:e] @ A_i^T) @ B_i^T per segment,
    rank 8 or 16, at most 512 rows, in one launch."""
    if not 1 <= len(problems) <= MAX_FUSED_BGMV_PROBLEMS:
        raise RuntimeError(f"between 1 and {MAX_FUSED_BGMV_PROBLEMS} problems per launch, got {len(problems)}")
    _check_input(x, "x", 2)
    _check_input(s_start, "s_start", 1)
    _check_input(s_end, "s_end", 1)
    if s_start.dtype != torch.int32 or s_end.dtype != torch.int32 or s_start.size(0) != s_end.size(0):
        raise RuntimeError("s_start and s_end must be int32 tensors of one length")
    arr = (SgmvLoraProblem * len(problems))()
    for i, (y, a_ptr, b_ptr, y_offset, y_slice_size) in enumerate(problems):
        _check_input(y, "y", 2)
        _check_input(a_ptr, "a_ptr", 1)
        _check_input(b_ptr, "b_ptr", 1)
        _check_same(y, x, a_ptr, b_ptr, s_start, s_end)
        if a_ptr.dtype != torch.int64 or b_ptr.dtype != torch.int64:
            raise RuntimeError("a_ptr and b_ptr must be int64 tensors")
        if a_ptr.size(0) != s_start.size(0) or b_ptr.size(0) != s_start.size(0):
            raise RuntimeError("a_ptr and b_ptr must have one entry per segment")
        if y.size(0) != x.size(0):
            raise RuntimeError(f"CHECK_EQ(y.size(0), x.size(0)) failed. {y.size(0)} vs {x.size(0)}")
        h_out = y.size(1) if y_slice_size is None else int(y_slice_size)
        arr[i] = SgmvLoraProblem(y.data_ptr(), a_ptr.data_ptr(), b_ptr.data_ptr(), int(y_offset), y.size(1), h_out)
    with torch.cuda.device(x.device):
        rc = lib().lorax_sgmv_lora_multi(arr, len(problems), x.data_ptr(), s_start.data_ptr(), s_end.data_ptr(),
                                         s_start.size(0), x.size(0), x.size(1), int(rank), int(layer_idx),
                                         float(scale), _dtype_code(x), _stream(x))
    if rc != 0:
        _raise_last(rc)


ENTRY_DTYPE = [("adapter", "<i8"), ("a_addr", "<i8"), ("b_addr", "<i8"), ("rank", "<i4"), ("reserved", "<i4")]


_table_capacity = [64 * 1024, 64]  # bytes of packed tables, number of group records


def build_batch_tables(adapter_indices, entries, entry_counts, prefill: bool):
    """lorax_build_batch_tables on numpy arrays: adapter_indices int64 [T]; entries a structured array of
    ENTRY_DTYPE, the layer types' adapters one after the other, each type sorted by adapter; entry_counts int32
    per type.  Returns (segment bounds int32 [S+1], segment owners int64 [S], packed uint8 buffer, groups)."""
    import numpy as np

    adapter_indices = np.ascontiguousarray(adapter_indices, dtype=np.int64)
    entries = np.ascontiguousarray(entries, dtype=ENTRY_DTYPE)
    entry_counts = np.ascontiguousarray(entry_counts, dtype=np.int32)
    T = adapter_indices.shape[0]
    bounds = np.zeros(T + 1, dtype=np.int32)
    owners = np.zeros(max(T, 1), dtype=np.int64)
    nseg, ngroups, nbytes = _c.c_int32(0), _c.c_int32(0), _c.c_int64(0)
    capacity, group_capacity = _table_capacity
    while True:
        packed = np.empty(capacity, dtype=np.uint8)  # the builder writes every byte it reports as used
        groups = (TableGroup * group_capacity)()
        rc = lib().lorax_build_batch_tables(
            adapter_indices.ctypes.data, T, entries.ctypes.data, entry_counts.ctypes.data, entry_counts.shape[0],
            1 if prefill else 0, bounds.ctypes.data, owners.ctypes.data, ctypes.byref(nseg), packed.ctypes.data,
            capacity, ctypes.byref(nbytes), groups, group_capacity, ctypes.byref(ngroups),
        )
        if rc == ESPACE:  # remembered: the next batch of this size takes one call
            capacity = max(capacity, int(nbytes.value) * 5 // 4)
            group_capacity = max(group_capacity, int(ngroups.value) * 2)
            _table_capacity[:] = [capacity, group_capacity]
            continue
        if rc != 0:
            _raise_last(rc)
        return bounds[: nseg.value + 1], owners[: nseg.value], packed[: nbytes.value], list(groups[: ngroups.value])
