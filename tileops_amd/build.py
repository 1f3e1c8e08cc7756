"""Build libmi355_tileops.so (HIP kernels + C ABI) for gfx950 with hipcc, in-tree.

``python -m tileops_amd.build`` compiles every translation unit under ``tileops_amd/csrc`` and links
``tileops_amd/lib/libmi355_tileops.so``.  hipcc cross-compiles, so no GPU is needed to build.
"""

from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG = Path(__file__).resolve().parent
CSRC = PKG / "csrc"
LIB_DIR = PKG / "lib"
LIB_PATH = LIB_DIR / "libmi355_tileops.so"
OBJ_DIR = PKG / "build"

SOURCES = ["abi.hip", "paged_decode_generic.hip", "paged_decode_mfma.hip", "paged_cache_utils.hip"]

# -packed-fp32-ops: keep the compiler from forming v_pk_*_f32 out of scalar float code.
HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Wall",
    "-Wno-unused-function",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; the MI355X library cannot be built")
    return exe


def _compile(src: str, extra: tuple = (), tag: str = "") -> Path:
    obj = OBJ_DIR / (src + tag + ".o")
    cmd = [_hipcc(), *HIPCC_FLAGS, *extra, "-c", str(CSRC / src), "-o", str(obj)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{res.stderr}")
    # the host pass does not know the packed-fp32 feature name and says so; anything else is shown
    noise = "is not a recognized feature for this target"
    rest = [ln for ln in res.stderr.splitlines() if ln.strip() and noise not in ln]
    if rest:
        print("\n".join(rest), file=sys.stderr)
    return obj


def build(verbose: bool = True, extra_flags: tuple = (), lib_path: Path = LIB_PATH) -> Path:
    """Compile and link.  ``extra_flags`` / ``lib_path`` let a developer build an instrumented copy beside the product."""
    OBJ_DIR.mkdir(exist_ok=True)
    lib_path.parent.mkdir(exist_ok=True)
    tag = "" if not extra_flags else "." + lib_path.stem
    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as pool:
        objs = list(pool.map(lambda src: _compile(src, tuple(extra_flags), tag), SOURCES))
    tmp = lib_path.with_suffix(".so.tmp")
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", *map(str, objs), "-o", str(tmp)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stderr}")
    os.replace(tmp, lib_path)
    if verbose:
        print(f"built {lib_path} ({lib_path.stat().st_size} bytes)")
    return lib_path


if __name__ == "__main__":
    build()
