"""ctypes binding of ``libadasplash_hip.so`` (the C ABI in ``include/adasplash_hip.h``).

There is no CPU or eager fallback: if the library has not been built, or a tensor is not on a
ROCm device, the call fails.
"""

import contextlib
import ctypes
from pathlib import Path

import torch

_LIB_PATH = Path(__file__).resolve().parent / "lib" / "libadasplash_hip.so"
_lib = None

ADSP_F32, ADSP_BF16, ADSP_F16 = 0, 1, 2
_DTYPES = {torch.float32: ADSP_F32, torch.bfloat16: ADSP_BF16, torch.float16: ADSP_F16}

_vp, _i, _i64, _sz, _dbl = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_size_t, ctypes.c_double

_SIGNATURES = {
    "adsp_version": (_i, []),
    "adsp_build_id": (ctypes.c_char_p, []),
    "adsp_build_flags": (ctypes.c_char_p, []),
    "adsp_status_string": (ctypes.c_char_p, [_i]),
    "adsp_entmax_rows_fwd": (_i, [_vp, _vp, _i64, _i64, _i, _dbl, _i, _i, _i, _vp]),
    "adsp_entmax_rows_bwd": (_i, [_vp, _vp, _vp, _i64, _i64, _i, _dbl, _vp]),
    "adsp_attn_workspace_bytes": (_sz, [_i, _i, _i, _i, _i, _i]),
    "adsp_attn_bmask_words": (_sz, [_i]),
    "adsp_attn_v2_fwd": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _vp, _sz, _vp]),
    "adsp_attn_v2_fwd_noalloc_max_bytes": (_sz, []),
    "adsp_attn_v2_fwd_noalloc": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _vp]),
    "adsp_attn_v1_fwd": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _dbl, _i, _i, _vp, _sz,
                              _vp, _vp]),
    "adsp_attn_supports_bytes": (_sz, [_i, _i, _i, _i, _i, _i]),
    "adsp_attn_v2_fwd_keep": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _vp, _sz, _vp, _sz,
                                   _vp]),
    "adsp_attn_v1_fwd_keep": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _dbl, _i, _i, _vp, _sz,
                                   _vp, _sz, _vp]),
    "adsp_attn_bwd_kept": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i,
                                _dbl, _i, _vp, _sz, _vp, _sz, _vp]),
    "adsp_attn_bwd_workspace_bytes": (_sz, [_i, _i, _i, _i, _i, _i]),
    "adsp_attn_bwd_workspace_bytes_causal": (_sz, [_i, _i, _i, _i, _i, _i, _i]),
    "adsp_attn_bwd": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _dbl,
                           _i, _vp, _sz, _vp]),
}


def lib_path() -> Path:
    return _LIB_PATH


def load():
    """Load the shared library once; raise if it is missing (no fallback path exists)."""
    global _lib
    if _lib is None:
        if not _LIB_PATH.exists():
            raise RuntimeError(
                f"{_LIB_PATH} not found: build the HIP kernels first with `python -m adasplash_amd.build` "
                "(hipcc, gfx950)."
            )
        lib = ctypes.CDLL(str(_LIB_PATH))
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _check_build_id(lib)
        _lib = lib
    return _lib


def build_id() -> str:
    """The source hash baked into the loaded library."""
    return load().adsp_build_id().decode()


def _check_build_id(lib):
    """Refuse a library that was built from other sources than the ones next to it.  The kernel sources travel
    with the package; when they are absent (a stripped install) there is nothing to compare with."""
    from . import build as _build

    if not _build.CSRC.is_dir() or not _build.INCLUDE.is_dir():
        return
    # (the id covers the extra flags of the build, which the library names itself: the environment of this process,
    # which may differ from the build's, does not enter)
    have, want = lib.adsp_build_id().decode(), _build.source_id(lib.adsp_build_flags().decode())
    if have != want:
        raise RuntimeError(
            f"{_LIB_PATH} is stale: it was built from sources with id {have}, the tree has id {want}. "
            "Rebuild with `python -m adasplash_amd.build`."
        )


def dtype_code(t: torch.Tensor) -> int:
    try:
        return _DTYPES[t.dtype]
    except KeyError:
        raise TypeError(f"unsupported dtype {t.dtype}; expected float32, bfloat16 or float16") from None


def require_device(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError("adasplash_amd kernels run on a ROCm device only; got a CPU tensor")


def device_guard(device):
    """Context that makes `device` current for the launch; a no-op when it already is (the common case: entering
    torch's guard costs the host more than a short kernel lasts)."""
    if device.index is None or device.index == torch.cuda.current_device():
        return contextlib.nullcontext()
    return torch.cuda.device(device)


def current_stream(device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


def check(status: int, what: str):
    if status != 0:
        msg = load().adsp_status_string(status).decode()
        raise RuntimeError(f"{what} failed: {msg} (status {status})")


def ptr(t):
    return None if t is None else t.data_ptr()
