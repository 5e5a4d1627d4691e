"""adasplash_amd: MI355X (gfx950) implementation of AdaSplash sparse entmax attention.

The public names, signatures, defaults and routing are those of the reference package
(``adasplash/__init__.py:1-85``); every call ends in a hand-written HIP kernel reached through the
C ABI of ``libadasplash_hip.so``.  Importing this package touches neither the GPU nor the library;
both are loaded on first use.
"""

__version__ = "0.2.0"


def adasplash_v1(q, k, v, alpha=1.5, is_causal=False, varlen=None, niter=10):
    from .adasplash_block_mask import sparse_attn

    return sparse_attn(q, k, v, alpha=alpha, is_causal=is_causal, varlen=varlen, niter=niter)


def adasplash_v2(q, k, v, niter=1, varlen=None):
    return _adasplash_v2(q, k, v, niter=niter, varlen=varlen)


def _adasplash_v2(q, k, v, niter=1, varlen=None):
    from .adasplash_v2 import sparse_attn

    return sparse_attn(q, k, v, niter=niter, varlen=varlen)


def adasplash(q, k, v, alpha=1.5, is_causal=True, varlen=None, niter=None):
    """Dispatcher: causal alpha = 1.5 goes to AdaSplash-2 (niter defaults to 1), anything else to the
    block-mask kernel (niter defaults to 10), as in ``adasplash/__init__.py:20-30``."""
    if alpha != 1.5 or not is_causal:
        return adasplash_v1(
            q, k, v, alpha=alpha, is_causal=is_causal, varlen=varlen, niter=10 if niter is None else niter
        )
    return _adasplash_v2(q, k, v, niter=1 if niter is None else niter, varlen=varlen)


def adasplash_no_block_mask(q, k, v, alpha=1.5, is_causal=False, varlen=None, niter=10):
    """Served by the block-mask kernel: the two reference variants compute the same function and differ
    only in whether tiles are skipped."""
    return adasplash_v1(q, k, v, alpha=alpha, is_causal=is_causal, varlen=varlen, niter=niter)


def triton_entmax_v1(x, alpha=1.5, n_iter=10, fast_math=True):
    """Served by the rows kernel without histogram initialisation (the original solver starts from
    ``[max - 1, max]``, ``adasplash/triton_entmax.py:94``)."""
    from .triton_entmax_v2 import triton_entmax

    return triton_entmax(x, alpha=alpha, n_iter=n_iter, use_histogram=False, fast_math=fast_math)


def triton_entmax_v2(x, alpha=1.5, n_iter=2, use_histogram=True, fast_math=False):
    return _triton_entmax_v2(x, alpha=alpha, n_iter=n_iter, use_histogram=use_histogram, fast_math=fast_math)


def _triton_entmax_v2(x, alpha=1.5, n_iter=2, use_histogram=True, fast_math=False):
    from .triton_entmax_v2 import triton_entmax

    return triton_entmax(x, alpha=alpha, n_iter=n_iter, use_histogram=use_histogram, fast_math=fast_math)


def triton_entmax(x, alpha=1.5, n_iter=2, use_histogram=True, fast_math=False):
    return _triton_entmax_v2(x, alpha=alpha, n_iter=n_iter, use_histogram=use_histogram, fast_math=fast_math)


def triton_sparsemax(x, **kwargs):
    from .triton_entmax_v2 import triton_sparsemax

    return triton_sparsemax(x, **kwargs)


def triton_entmax15(x, **kwargs):
    from .triton_entmax_v2 import triton_entmax15

    return triton_entmax15(x, **kwargs)


def set_keep_supports(mode):
    """What the attention forward keeps for its backward besides the reference's saved tensors: ``"auto"`` (the supports
    it found, when they take at most twice the bytes of q or 256 MiB), ``"always"`` or ``"never"`` (the backward then
    finds the supports again with a score walk).  Returns the previous mode.  Not part of the reference's surface."""
    from ._attention import set_keep_supports as _set

    return _set(mode)


adasplash2 = _adasplash_v2

__all__ = [
    "__version__",
    "adasplash",
    "adasplash2",
    "adasplash_v1",
    "adasplash_v2",
    "adasplash_no_block_mask",
    "triton_entmax",
    "triton_entmax_v1",
    "triton_entmax_v2",
    "triton_sparsemax",
    "triton_entmax15",
]
