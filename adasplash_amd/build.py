"""Build the HIP shared library in-tree: ``python -m adasplash_amd.build [--force] [-j N]``.

The kernels are compiled for gfx950 with hipcc, one object per (element type, head dim, instance), and
linked into ``adasplash_amd/lib/libadasplash_hip.so`` (the C ABI declared in ``include/adasplash_hip.h``).

* An object is recompiled when the hash of its command line, its source and every header it includes
  (transitively, quoted includes) differs from the one recorded beside it; ``--force`` recompiles everything.
* The library carries ``adsp_build_id()``: a hash over all kernel sources, headers and flags, and
  ``adsp_build_flags()``: the extra flags it was built with (``ADSP_ATTN_FLAGS`` in the environment of the build:
  profiling builds).  ``source_id(extra)`` recomputes the id from the tree for the library's own extra flags, and the
  loader and the tests compare the two, so a library that is older than the sources next to it is an error instead
  of a silent stale binary, whatever the environment of the process that loads it.
* The link step always runs, and the library is replaced atomically after a successful link only.
"""

import hashlib
import os
import re
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG = Path(__file__).resolve().parent
CSRC = PKG / "csrc"
INCLUDE = PKG.parent / "include"
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
ATTN_FLAGS = ["-fno-honor-nans"]
EXTRA_ATTN_FLAGS = os.environ.get("ADSP_ATTN_FLAGS", "").split()  # of this process: what a build started here adds

TYPES = {"f32": "float", "bf16": "bf16_t", "f16": "f16_t"}
HEAD_DIMS = (16, 32, 64, 128, 256)


def units(extra=None):
    """(object stem, source file, extra flags) of every translation unit; ``extra``: flags added to the attention units
    (default: ``ADSP_ATTN_FLAGS`` of this process)."""
    attn_flags = ATTN_FLAGS + (EXTRA_ATTN_FLAGS if extra is None else list(extra))
    out = [("attn_api", "attn_api.hip", []), ("entmax_rows", "entmax_rows.hip", [])]
    for tag, ty in TYPES.items():
        for d in HEAD_DIMS:
            base = [f"-DADSP_T={ty}", f"-DADSP_TAG={tag}", f"-DADSP_D={d}"]
            for multi in (0, 1):
                out.append((f"attn_fwd_{tag}_d{d}_m{multi}", "attn_fwd_unit.hip", base + [f"-DADSP_MULTI={multi}"] + attn_flags))
            out.append((f"attn_bwd_{tag}_d{d}", "attn_bwd_unit.hip", base))
            if tag != "f32" and d in (64, 128):
                out.append((f"attn_sparse_{tag}_d{d}", "attn_sparse_unit.hip", base + attn_flags))
                out.append((f"attn_bwd_sparse_{tag}_d{d}", "attn_bwd_sparse_unit.hip", base + attn_flags))
    return out


_INCLUDE_RE = re.compile(r'^\s*#\s*include\s*"([^"]+)"', re.M)


def _deps(path: Path, seen=None):
    """The file and every header it includes with quotes, transitively, resolved next to the including file."""
    seen = {} if seen is None else seen
    path = path.resolve()
    if path in seen or not path.exists():
        return seen
    text = path.read_bytes()
    seen[path] = text
    for inc in _INCLUDE_RE.findall(text.decode()):
        _deps(path.parent / inc, seen)
    return seen


def _digest(parts) -> str:
    h = hashlib.sha256()
    for p in parts:
        h.update(p if isinstance(p, bytes) else p.encode())
        h.update(b"\0")
    return h.hexdigest()


def source_id(extra=None) -> str:
    """Hash of everything the library is built from; what ``adsp_build_id()`` of an up-to-date library returns.
    ``extra``: the extra attention flags to assume (a string or a list; default: those of this process)."""
    if isinstance(extra, str):
        extra = extra.split()
    files = sorted(list(CSRC.glob("*.hip")) + list(CSRC.glob("*.h")) + list(INCLUDE.glob("*.h")))
    parts = []
    for f in files:
        parts += [f.name, f.read_bytes()]
    parts += FLAGS + ["--"] + [u[0] + " " + " ".join(u[2]) for u in units(extra)]
    return _digest(parts)[:16]


def _compile(unit, build_id: str, force: bool):
    stem, src, extra = unit
    obj = OBJ_DIR / (stem + ".o")
    sig_file = OBJ_DIR / (stem + ".sig")
    src_path = CSRC / src
    extra = list(extra)
    if stem == "attn_api":
        extra.append(f'-DADSP_BUILD_ID="{build_id}"')
        extra.append('-DADSP_BUILD_FLAGS="' + " ".join(EXTRA_ATTN_FLAGS).replace('"', "") + '"')
    cmd = [HIPCC, *FLAGS, *extra, "-c", str(src_path), "-o", str(obj)]
    deps = _deps(src_path)
    sig = _digest([" ".join(cmd)] + [x for p in sorted(deps) for x in (str(p), deps[p])])
    if not force and obj.exists() and sig_file.exists() and sig_file.read_text() == sig:
        return obj, False
    sig_file.unlink(missing_ok=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed for {stem} ({src}):\n{res.stderr}")
    sig_file.write_text(sig)
    return obj, True


def build(jobs: int = 8, verbose: bool = True, force: bool = False) -> Path:
    """Compile what changed (everything with ``force``), link, and return the path of the shared library."""
    OBJ_DIR.mkdir(exist_ok=True)
    LIB_DIR.mkdir(exist_ok=True)
    build_id = source_id()
    todo = units()
    if verbose:
        print(f"[adasplash_amd.build] {len(todo)} translation units for gfx950, build id {build_id}", flush=True)
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        results = list(pool.map(lambda u: _compile(u, build_id, force), todo))
    objs = [o for o, _ in results]
    stale = {o.name for o in objs}
    for old in OBJ_DIR.glob("*.o"):  # objects of units that no longer exist
        if old.name not in stale:
            old.unlink()
            old.with_suffix(".sig").unlink(missing_ok=True)
    tmp = LIB_PATH.with_suffix(".so.tmp")
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", *map(str, objs), "-o", str(tmp)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stderr}")
    os.replace(tmp, LIB_PATH)
    if verbose:
        n = sum(1 for _, done in results if done)
        print(f"[adasplash_amd.build] compiled {n} of {len(objs)} objects, wrote {LIB_PATH}", flush=True)
    return LIB_PATH


if __name__ == "__main__":
    args = sys.argv[1:]
    jobs = 8
    if "-j" in args:
        jobs = int(args[args.index("-j") + 1])
    build(jobs=jobs, force="--force" in args)
    sys.exit(0)
