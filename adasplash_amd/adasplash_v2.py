"""AdaSplash-2: causal entmax-1.5 attention with GQA and variable lengths on gfx950.

Same call surface as the reference module of this name: ``sparse_attn(q, k, v, niter=1, varlen=None)``
(``adasplash/adasplash_v2.py:1567-1591``), same argument checks as its autograd wrapper
(``adasplash/adasplash_v2.py:1243-1276``).
"""

import torch

from . import _attention

BMASK_TILE = 64


class _SparseAttentionV2(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, v, niter=10, varlen=None):
        B, N_H, N_CTX, H_DIM = q.shape
        assert H_DIM in {16, 32, 64, 128, 256}
        assert k.shape == v.shape, f"K and V must share shape; got k.shape={tuple(k.shape)} v.shape={tuple(v.shape)}"
        N_KV_H = k.shape[1]
        assert N_KV_H >= 1 and N_H % N_KV_H == 0, f"N_H ({N_H}) must be a positive multiple of N_KV_H ({N_KV_H})."
        assert k.shape[0] == B and k.shape[2] == N_CTX and k.shape[3] == H_DIM, (
            f"K/V must have shape (B={B}, N_KV_H, N_CTX={N_CTX}, H_DIM={H_DIM}); got {tuple(k.shape)}."
        )
        assert N_CTX >= BMASK_TILE, f"N_CTX={N_CTX} must be at least BMASK_TILE={BMASK_TILE}."
        if varlen is None:
            assert (N_CTX & (N_CTX - 1)) == 0, "If varlen is None, N_CTX must be a power of two."
        else:
            assert varlen.dim() == 1 and varlen.shape[0] == B, (
                f"varlen must be a 1-D tensor of shape (B={B},); got {tuple(varlen.shape)}."
            )
            assert varlen.dtype in (torch.int32, torch.int64), f"varlen must be int32/int64; got {varlen.dtype}."
            assert varlen.device == q.device, "varlen must be on the same device as q."
            assert varlen.is_contiguous(), "varlen must be contiguous."
        _attention.assert_contiguous(q, k, v, msg="Q, K and/or V are not contiguous.")

        # (when a gradient will be asked for, the forward keeps the supports it found: the backward then finds none again)
        keep = any(ctx.needs_input_grad[:3])
        res = _attention.launch_forward(
            q, k, v, version=2, alpha=1.5, is_causal=True, niter=niter, varlen=varlen,
            keep_supports=keep,
        )
        out, taus, bmask = res[:3]
        supports = res[3] if keep else None
        ctx.save_for_backward(q, k, v, taus, bmask, supports)
        ctx.varlen = varlen
        return out

    @staticmethod
    def backward(ctx, do):
        q, k, v, taus, bmask, supports = ctx.saved_tensors
        dq, dk, dv = _attention.launch_backward(
            q, k, v, do, taus, bmask, alpha=1.5, is_causal=True, varlen=ctx.varlen, supports=supports
        )
        return dq, dk, dv, None, None


def sparse_attn(q, k, v, niter=1, varlen=None):
    """Causal entmax-1.5 sparse attention.

    q: ``(batch, n_heads, seq_len, head_dim)``; k, v: ``(batch, n_kv_heads, seq_len, head_dim)`` with
    ``n_heads`` a multiple of ``n_kv_heads``; ``niter``: refinement passes of the threshold solver after
    its histogram bracket; ``varlen``: optional ``(batch,)`` int32/int64 valid lengths (right padding),
    padded output rows are zero.  Returns a tensor like ``q``.
    """
    return _SparseAttentionV2.apply(q, k, v, niter, varlen)


def _install_callable_module():
    import inspect
    import sys
    import types

    class _CallableModule(types.ModuleType):
        def __call__(self, *args, **kwargs):
            return sparse_attn(*args, **kwargs)

    module = sys.modules[__name__]
    module.__class__ = _CallableModule
    module.__signature__ = inspect.signature(sparse_attn)


_install_callable_module()
