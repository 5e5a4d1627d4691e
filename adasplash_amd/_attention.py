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


# What the forward of the autograd functions keeps for the backward besides q, k, v, taus and bmask: the supports it
# found (51.7 KB per 128 query rows and head, whatever the head dim), with which the backward needs no score walk of
# its own.  "auto" keeps them when they take at most twice the bytes of q -- the reference keeps a second output of
# q's size for its backward (adasplash/adasplash_v2.py:1421-1426) -- or 256 MiB; "always" and "never" say what they
# mean.  ``ADSP_KEEP_SUPPORTS`` in the environment sets the initial mode (0 / never, 1 / always, auto).
_KEEP_MODES = ("auto", "always", "never")
_keep_mode = None


def set_keep_supports(mode):
    """Choose what the attention forward keeps for its backward: ``"auto"`` (default), ``"always"`` or ``"never"``.
    Returns the previous mode."""
    global _keep_mode
    if mode not in _KEEP_MODES:
        raise ValueError(f"mode must be one of {_KEEP_MODES}; got {mode!r}")
    old = get_keep_supports()
    _keep_mode = mode
    return old


def get_keep_supports():
    global _keep_mode
    if _keep_mode is None:
        import os

        env = os.environ.get("ADSP_KEEP_SUPPORTS", "auto").lower()
        _keep_mode = {"0": "never", "1": "always"}.get(env, env if env in _KEEP_MODES else "auto")
    return _keep_mode


def _keeps(sup_bytes, q):
    mode = get_keep_supports()
    if mode == "never" or sup_bytes == 0:
        return False
    return mode == "always" or sup_bytes <= max(2 * q.numel() * q.element_size(), 256 << 20)


def launch_forward(q, k, v, *, version, alpha, is_causal, niter, varlen, tile_counts=None, keep_supports=False):
    """Allocate out / taus / bmask / workspace with torch and enqueue the fused forward on the
    current stream.  Returns ``(out, taus, bmask)``, and with ``keep_supports`` a fourth value: the buffer in which the
    forward keeps the supports it found for ``launch_backward`` (``None`` where the library keeps none: fp32, head dims
    other than 64 / 128, a caller that asks for the tile statistics, or a buffer beyond what ``set_keep_supports``
    allows; ``keep_supports="always"`` asks for the buffer whatever the mode)."""
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
    sup = None
    if keep_supports and tile_counts is None:
        sup_bytes = lib.adsp_attn_supports_bytes(B, Hq, Hkv, N, D, dt)
        if keep_supports == "always" or _keeps(sup_bytes, q):  # ("always": a caller that asks for them by name)
            sup = torch.empty((sup_bytes,), device=q.device, dtype=torch.uint8) if sup_bytes else None
    with _lib.device_guard(q.device):
        stream = _lib.current_stream(q.device)
        if sup is not None and version == 2:
            st = lib.adsp_attn_v2_fwd_keep(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), taus.data_ptr(),
                                           bmask.data_ptr(), _lib.ptr(varlen), bits, B, Hq, Hkv, N, D, dt, int(niter),
                                           _lib.ptr(ws), ws_bytes, sup.data_ptr(), sup.numel(), stream)
            _lib.check(st, "adsp_attn_v2_fwd_keep")
        elif sup is not None:
            st = lib.adsp_attn_v1_fwd_keep(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), taus.data_ptr(),
                                           bmask.data_ptr(), _lib.ptr(varlen), bits, B, Hq, N, D, dt, float(alpha),
                                           int(bool(is_causal)), int(niter), _lib.ptr(ws), ws_bytes, sup.data_ptr(),
                                           sup.numel(), stream)
            _lib.check(st, "adsp_attn_v1_fwd_keep")
        elif version == 2:
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
    if keep_supports:
        return out, taus, bmask, sup
    return out, taus, bmask


def assert_contiguous(*inputs, msg="Inputs are not contiguous."):
    assert all(t.is_contiguous() for t in inputs), msg


def launch_backward(q, k, v, dout, taus, bmask, *, alpha, is_causal, varlen, supports=None):
    """Enqueue the dQ and dK/dV kernels on the current stream; returns ``(dq, dk, dv)``.

    ``taus`` / ``bmask`` are the thresholds and the tile mask the forward produced, ``supports`` what it kept for this
    call (``launch_forward(..., keep_supports=True)``) or ``None``: then the dQ kernel finds the supports again.  Rows of ``dout`` past a
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
    ws_bytes = lib.adsp_attn_bwd_workspace_bytes_causal(B, Hq, Hkv, N, D, dt, 1 if is_causal else 0)
    ws = torch.empty((ws_bytes,), device=q.device, dtype=torch.uint8) if ws_bytes else None
    with _lib.device_guard(q.device):
        if supports is not None:
            st = lib.adsp_attn_bwd_kept(q.data_ptr(), k.data_ptr(), v.data_ptr(), dout.data_ptr(), taus.data_ptr(),
                                        _lib.ptr(bmask), _lib.ptr(varlen), _varlen_bits(varlen), dq.data_ptr(),
                                        dk.data_ptr(), dv.data_ptr(), delta.data_ptr(), zinv.data_ptr(), B, Hq, Hkv, N, D,
                                        dt, float(alpha), int(bool(is_causal)), _lib.ptr(ws), ws_bytes,
                                        supports.data_ptr(), supports.numel(), _lib.current_stream(q.device))
            _lib.check(st, "adsp_attn_bwd_kept")
        else:
            st = lib.adsp_attn_bwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), dout.data_ptr(), taus.data_ptr(),
                                   _lib.ptr(bmask), _lib.ptr(varlen), _varlen_bits(varlen), dq.data_ptr(), dk.data_ptr(),
                                   dv.data_ptr(), delta.data_ptr(), zinv.data_ptr(), B, Hq, Hkv, N, D, dt, float(alpha),
                                   int(bool(is_causal)), _lib.ptr(ws), ws_bytes, _lib.current_stream(q.device))
            _lib.check(st, "adsp_attn_bwd")
    return dq, dk, dv
