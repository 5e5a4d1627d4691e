"""Shared host side of the two attention entry points: buffer allocation and the C-ABI call."""

import torch

from . import _lib


def _varlen_bits(varlen):
    if varlen is None:
        return 0
    if varlen.dtype == torch.int32:
        return 32
    if varlen.dtype == torch.int64:
        return 64
    raise AssertionError(f"varlen must be int32/int64; got {varlen.dtype}.")


def launch_forward(q, k, v, *, version, alpha, is_causal, niter, varlen, tile_counts=None):
    """Allocate out / taus / bmask / workspace with torch and enqueue the fused forward on the
    current stream.  Returns ``(out, taus, bmask)``."""
    _lib.require_device(q, k, v, varlen)
    lib = _lib.load()
    B, Hq, N, D = q.shape
    Hkv = k.shape[1]
    dt = _lib.dtype_code(q)
    assert k.dtype == q.dtype and v.dtype == q.dtype, "q, k and v must share a dtype"
    out = torch.empty_like(q)
    taus = torch.empty((B, Hq, N), device=q.device, dtype=torch.float32)
    bmask = torch.empty((B, Hq, lib.adsp_attn_bmask_words(N)), device=q.device, dtype=torch.int32)
    ws_bytes = lib.adsp_attn_workspace_bytes(B, Hkv, N, D, dt)
    ws = torch.empty((ws_bytes,), device=q.device, dtype=torch.uint8) if ws_bytes else None
    bits = _varlen_bits(varlen)
    with torch.cuda.device(q.device):
        stream = _lib.current_stream(q.device)
        if version == 2:
            st = lib.adsp_attn_v2_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), taus.data_ptr(),
                                      bmask.data_ptr(), _lib.ptr(varlen), bits, B, Hq, Hkv, N, D, dt, int(niter),
                                      _lib.ptr(ws), ws_bytes, stream)
            _lib.check(st, "adsp_attn_v2_fwd")
        else:
            st = lib.adsp_attn_v1_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), taus.data_ptr(),
                                      bmask.data_ptr(), _lib.ptr(varlen), bits, B, Hq, N, D, dt, float(alpha),
                                      int(bool(is_causal)), int(niter), _lib.ptr(ws), ws_bytes,
                                      _lib.ptr(tile_counts), stream)
            _lib.check(st, "adsp_attn_v1_fwd")
    return out, taus, bmask


def assert_contiguous(*inputs, msg="Inputs are not contiguous."):
    assert all(t.is_contiguous() for t in inputs), msg


_BACKWARD_MSG = (
    "the MI355X build implements the forward pass of sparse entmax attention only; "
    "the backward kernels are not built yet"
)


def backward_not_built():
    raise NotImplementedError(_BACKWARD_MSG)
