"""AdaSplash-1 (block-mask): alpha-entmax attention for any alpha in (1, 2], causal or not, on gfx950.

Same call surface as the reference module of this name:
``sparse_attn(q, k, v, alpha=1.5, is_causal=False, varlen=None, niter=10)``
(``adasplash/adasplash_block_mask.py:1213-1232``), same argument checks as its autograd wrapper
(``adasplash/adasplash_block_mask.py:922-960``).
"""

import torch

from . import _attention


class _SparseAttentionV1(torch.autograd.Function):
    @staticmethod
    def forward(ctx, q, k, v, alpha=1.5, is_causal=False, varlen=None, niter=10):
        B, N_H, N_CTX, H_DIM = q.shape
        assert H_DIM in {16, 32, 64, 128, 256}
        if varlen is None:
            assert N_CTX.bit_count() == 1, "If varlen is not used, the context length must be a power of two."
        else:
            assert varlen.dim() == 1, "varlen must be a one-dimensional tensor."
            assert varlen.shape[0] == B, f"varlen must have one entry per batch item (B={B})."
        assert k.shape == q.shape and v.shape == q.shape, "q, k and v must share one shape (no GQA in v1)."
        _attention.assert_contiguous(q, k, v, msg="Q, K and/or V are not contiguous.")
        if varlen is not None and not varlen.is_contiguous():
            varlen = varlen.contiguous()

        # (when a gradient will be asked for, the forward keeps the supports it found: the backward then finds none again)
        keep = any(ctx.needs_input_grad[:3])
        res = _attention.launch_forward(
            q, k, v, version=1, alpha=alpha, is_causal=is_causal, niter=niter, varlen=varlen,
            keep_supports=keep,
        )
        out, taus, bmask = res[:3]
        supports = res[3] if keep else None
        ctx.save_for_backward(q, k, v, taus, bmask, supports)
        ctx.alpha = alpha
        ctx.is_causal = is_causal
        ctx.varlen = varlen
        return out

    @staticmethod
    def backward(ctx, do):
        q, k, v, taus, bmask, supports = ctx.saved_tensors
        dq, dk, dv = _attention.launch_backward(
            q, k, v, do, taus, bmask, alpha=ctx.alpha, is_causal=ctx.is_causal, varlen=ctx.varlen, supports=supports
        )
        return dq, dk, dv, None, None, None, None


def sparse_attn(q, k, v, alpha=1.5, is_causal=False, varlen=None, niter=10):
    """alpha-entmax sparse attention (block-mask variant).

    q, k, v: ``(batch, n_heads, seq_len, head_dim)``; ``alpha`` in (1, 2]; ``varlen``: optional
    ``(batch,)`` valid lengths (right padding), padded output rows are zero; ``niter``: Halley /
    bisection passes of the threshold solver.
    """
    return _SparseAttentionV1.apply(q, k, v, alpha, is_causal, varlen, niter)


def tile_sparsity(q, k, v, alpha=1.5, is_causal=False, varlen=None, niter=10):
    """Run the forward and also return ``(tiles_in_domain, tiles_active)`` counted on 16x16 score tiles,
    the granularity the reference's block mask uses (``adasplash/adasplash_block_mask.py:964-976``)."""
    counts = torch.zeros(2, device=q.device, dtype=torch.int64)
    out, _, _ = _attention.launch_forward(
        q, k, v, version=1, alpha=alpha, is_causal=is_causal, niter=niter, varlen=varlen, tile_counts=counts
    )
    total, active = (int(c) for c in counts.tolist())
    return out, total, active


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
