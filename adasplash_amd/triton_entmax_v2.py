"""Row-wise alpha-entmax backed by the gfx950 rows kernel.

Same call surface as the reference module of this name (``adasplash/triton_entmax_v2.py:690-731``):
``triton_entmax(x, alpha=1.5, n_iter=2, use_histogram=True, fast_math=False)``,
``triton_sparsemax(x, **kw)``, ``triton_entmax15(x, **kw)``.  The name is kept for drop-in use; no
Triton is involved.
"""

import torch

from . import _lib


class _EntmaxRows(torch.autograd.Function):
    """Counterpart of ``_entmax_triton`` (``adasplash/triton_entmax_v2.py:620-687``)."""

    @staticmethod
    def forward(ctx, x, alpha=1.5, n_iter=10, use_histogram=True, fast_math=False):
        size_n = x.shape[-1]
        assert x.is_contiguous(), "x must be contiguous"
        _lib.require_device(x)
        lib = _lib.load()
        y = torch.empty_like(x)  # the kernel writes every element, zeros included
        rows = x.numel() // size_n if size_n > 0 else 0
        with _lib.device_guard(x.device):
            st = lib.adsp_entmax_rows_fwd(x.data_ptr(), y.data_ptr(), rows, size_n, _lib.dtype_code(x), float(alpha),
                                          int(n_iter), int(bool(use_histogram)), int(bool(fast_math)),
                                          _lib.current_stream(x.device))
        _lib.check(st, "adsp_entmax_rows_fwd")
        ctx.save_for_backward(y)
        ctx.alpha = alpha
        return y

    @staticmethod
    def backward(ctx, dy):
        (y,) = ctx.saved_tensors
        size_n = y.shape[-1]
        if not dy.is_contiguous():
            dy = dy.contiguous()
        if dy.dtype != y.dtype:
            dy = dy.to(y.dtype)
        dx = torch.empty_like(dy)
        rows = y.numel() // size_n if size_n > 0 else 0
        lib = _lib.load()
        with _lib.device_guard(y.device):
            st = lib.adsp_entmax_rows_bwd(y.data_ptr(), dy.data_ptr(), dx.data_ptr(), rows, size_n, _lib.dtype_code(y),
                                          float(ctx.alpha), _lib.current_stream(y.device))
        _lib.check(st, "adsp_entmax_rows_bwd")
        return dx, None, None, None, None


def triton_entmax(x, alpha=1.5, n_iter=2, use_histogram=True, fast_math=False):
    """alpha-entmax over the last dimension of a contiguous tensor (any leading shape).

    For alpha outside {1.5, 2.0} the histogram initialisation is switched off and at least ten
    refinement steps are taken, as the reference does (``adasplash/triton_entmax_v2.py:713-716``).
    """
    if alpha not in (1.5, 2.0):
        use_histogram = False
        n_iter = max(n_iter, 10)
    return _EntmaxRows.apply(x, alpha, n_iter, use_histogram, fast_math)


def triton_sparsemax(x, **kwargs):
    """Sparsemax (entmax with alpha = 2.0)."""
    return triton_entmax(x, alpha=2.0, **kwargs)


def triton_entmax15(x, **kwargs):
    """Entmax-1.5 with histogram initialisation."""
    return triton_entmax(x, alpha=1.5, **kwargs)


def _install_callable_module():
    # keeps `adasplash_amd.triton_entmax_v2(x)` callable after the submodule import rebinds the name
    import inspect
    import sys
    import types

    class _CallableModule(types.ModuleType):
        def __call__(self, *args, **kwargs):
            return triton_entmax(*args, **kwargs)

    module = sys.modules[__name__]
    module.__class__ = _CallableModule
    module.__signature__ = inspect.signature(triton_entmax)


_install_callable_module()
