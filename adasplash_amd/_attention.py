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
    ws_bytes = lib.adsp_attn_workspace_bytes(B, Hq, Hkv, N, D, dt)
    ws = torch.empty((ws_bytes,), device=q.device, dtype=torch.uint8) if ws_bytes else None
    bits = _varlen_bits(varlen)
    with _lib.device_guard(q.device):
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


def launch_backward(q, k, v, dout, taus, bmask, *, alpha, is_causal, varlen):
    """Enqueue the dQ and dK/dV kernels on the current stream; returns ``(dq, dk, dv)``.

    ``taus`` / ``bmask`` are the thresholds and the tile mask the forward produced.  Rows of ``dout`` past a
    sequence's valid length are never used, whatever they hold (the kernels mask them as the reference's
    loads do, adasplash/adasplash_v2.py:1030-1033).
    """
    _lib.require_device(q, k, v, dout, varlen)
    lib = _lib.load()
    B, Hq, N, D = q.shape
    Hkv = k.shape[1]
    dt = _lib.dtype_code(q)
    dout = dout.to(q.dtype).contiguous()
    dq = torch.empty_like(q)
    dk = torch.empty_like(k)
    dv = torch.empty_like(v)
    delta = torch.empty((B, Hq, N), device=q.device, dtype=torch.float32)
    zinv = torch.empty((B, Hq, N), device=q.device, dtype=torch.float32)
    ws_bytes = lib.adsp_attn_bwd_workspace_bytes(B, Hq, Hkv, N, D, dt)
    ws = torch.empty((ws_bytes,), device=q.device, dtype=torch.uint8) if ws_bytes else None
    with _lib.device_guard(q.device):
        st = lib.adsp_attn_bwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), dout.data_ptr(), taus.data_ptr(),
                               _lib.ptr(bmask), _lib.ptr(varlen), _varlen_bits(varlen), dq.data_ptr(), dk.data_ptr(),
                               dv.data_ptr(), delta.data_ptr(), zinv.data_ptr(), B, Hq, Hkv, N, D, dt, float(alpha),
                               int(bool(is_causal)), _lib.ptr(ws), ws_bytes, _lib.current_stream(q.device))
        _lib.check(st, "adsp_attn_bwd")
    return dq, dk, dv
