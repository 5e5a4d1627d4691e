"""Build the HIP shared library in-tree: ``python -m adasplash_amd.build``.

Every ``csrc/*.hip`` translation unit is compiled for gfx950 with hipcc and linked into
``adasplash_amd/lib/libadasplash_hip.so`` (the C ABI declared in ``include/adasplash_hip.h``).
"""

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG = Path(__file__).resolve().parent
CSRC = PKG / "csrc"
LIB_DIR = PKG / "lib"
LIB_PATH = LIB_DIR / "libadasplash_hip.so"
OBJ_DIR = PKG / "build"

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Wno-unused-command-line-argument",
    # packed fp32 VALU forms are kept out of the generated code on purpose
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


# The attention kernels never produce or consume NaNs on purpose (masked scores are -inf and are clamped
# before any product), so fmax/fmin need no sNaN-quieting pre-pass there.
_ATTN_FLAGS = ["-fno-honor-nans"] + os.environ.get("ADSP_ATTN_FLAGS", "").split()
EXTRA_FLAGS = {f"attn_{kind}{ty}": _ATTN_FLAGS for kind in ("", "multi_") for ty in ("bf16", "f16", "f32")}


def _compile(src: Path) -> Path:
    obj = OBJ_DIR / (src.stem + ".o")
    cmd = [HIPCC, *FLAGS, *EXTRA_FLAGS.get(src.stem, []), "-c", str(src), "-o", str(obj)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src.name}:\n{res.stderr}")
    return obj


def build(jobs: int = 8, verbose: bool = True) -> Path:
    """Compile all kernels (always recompiles) and return the path of the shared library."""
    OBJ_DIR.mkdir(exist_ok=True)
    LIB_DIR.mkdir(exist_ok=True)
    srcs = sorted(CSRC.glob("*.hip"))
    if verbose:
        print(f"[adasplash_amd.build] compiling {len(srcs)} HIP sources for gfx950", flush=True)
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(_compile, srcs))
    tmp = LIB_PATH.with_suffix(".so.tmp")
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", *map(str, objs), "-o", str(tmp)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stderr}")
    os.replace(tmp, LIB_PATH)
    if verbose:
        print(f"[adasplash_amd.build] wrote {LIB_PATH}", flush=True)
    return LIB_PATH


if __name__ == "__main__":
    build()
    sys.exit(0)
