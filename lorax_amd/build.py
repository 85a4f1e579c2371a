"""Builds liblorax_hip.so (the HIP kernels and their C ABI) for gfx950 with hipcc.

Run as ``python -m lorax_amd.build``.  The library is built in-tree, next to this file,
so that it travels with the source tree to a machine that has the GPU.
"""

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC = PKG_DIR / "csrc"
LIB_PATH = PKG_DIR / "liblorax_hip.so"
SOURCES = ["capi.hip", "bgmv.hip", "sgmv_shrink.hip", "sgmv_shrink_lds.hip", "sgmv_expand.hip", "sgmv_expand_t.hip",
           "batch_tables.hip"]
ARCH = "gfx950"

# -packed-fp32-ops is switched off on purpose: the packed fp32 forms hipcc would
# otherwise pick for plain float code are not wanted in these kernels.
HIPCC_FLAGS = [
    f"--offload-arch={ARCH}",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Xclang",
    "-target-feature",
    "-Xclang",
    "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; liblorax_hip.so cannot be built")
    return exe


def _compile(src: str, obj_dir: Path) -> Path:
    obj = obj_dir / (Path(src).stem + ".o")
    extra = os.environ.get("LORAX_EXTRA_HIPCC_FLAGS", "").split()  # e.g. -DLORAX_EXPAND_STAGES=4 for tuning builds
    cmd = [hipcc(), *HIPCC_FLAGS, *extra, "-c", str(CSRC / src), "-o", str(obj)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{proc.stderr}")
    return obj


def build(verbose: bool = True, out: Path = LIB_PATH) -> Path:
    """Compiles every source and links the shared library. Always recompiles."""
    obj_dir = PKG_DIR / "build"
    obj_dir.mkdir(exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(4, len(SOURCES))) as pool:
        objs = list(pool.map(lambda s: _compile(s, obj_dir), SOURCES))
    tmp = Path(str(out) + ".tmp")
    cmd = [hipcc(), f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", str(tmp), *map(str, objs)]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"link failed:\n{proc.stderr}")
    os.replace(tmp, out)
    if verbose:
        print(f"built {out} ({out.stat().st_size} bytes)")
    return out


if __name__ == "__main__":
    build(out=Path(sys.argv[1]).resolve() if len(sys.argv) > 1 else LIB_PATH)
    sys.exit(0)
