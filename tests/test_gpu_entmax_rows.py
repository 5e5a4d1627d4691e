"""GPU parity of the entmax rows kernel (through the C ABI) against the exact CPU oracle."""

import numpy as np
import pytest
import torch

import adasplash_amd as A
from oracle import exact
from tests.gpu_util import DEV, max_err, tol_for

pytestmark = pytest.mark.gpu

ALPHAS = [1.333, 1.5, 2.0]


def test_golden_rows(golden_dir):
    g = np.load(golden_dir / "entmax_rows_128x256.npz")
    x = torch.tensor(g["x"]).to(DEV)
    for key, alpha in (("y15", 1.5), ("y20", 2.0), ("y1333", 1.333)):
        y = A.triton_entmax(x, alpha=alpha)
        assert max_err(y, torch.tensor(g[key])) < tol_for(torch.float32, alpha)


@pytest.mark.parametrize("impl", ["triton_entmax_v1", "triton_entmax_v2", "triton_entmax"])
@pytest.mark.parametrize("shape", [(2,), (2, 4), (2, 4, 8), (2, 4, 8, 16)])
@pytest.mark.parametrize("alpha", ALPHAS)
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_forward_matches_oracle_reference_matrix(impl, shape, alpha, dtype):
    # case list of tests/test_triton_entmax.py:47-64 (seed 42, n_iter 10, both fast_math settings)
    torch.manual_seed(42)
    x = torch.randn(*shape).to(dtype)
    want = exact.entmax_rows(x, alpha)
    fn = getattr(A, impl)
    for fast_math in (False, True):
        if impl == "triton_entmax_v1":
            y = fn(x.to(DEV), alpha=alpha, n_iter=10, fast_math=fast_math)
        else:
            y = fn(x.to(DEV), alpha=alpha, n_iter=10, use_histogram=True, fast_math=fast_math)
        assert y.dtype == dtype and y.shape == x.shape
        assert max_err(y, want) < tol_for(dtype, alpha)
        assert (y.float().sum(-1) - 1).abs().max().item() < 1e-2


def test_histogram_toggle_and_aliases():
    # tests/test_triton_entmax.py:101-114
    torch.manual_seed(42)
    x = torch.randn(4, 16)
    xd = x.to(DEV)
    r15, r20 = exact.entmax_rows(x, 1.5), exact.entmax_rows(x, 2.0)
    assert max_err(A.triton_entmax_v2(xd, alpha=1.5, use_histogram=True), r15) < 1e-4
    assert max_err(A.triton_entmax_v2(xd, alpha=1.5, use_histogram=False, n_iter=10), r15) < 1e-4
    assert max_err(A.triton_entmax15(xd), r15) < 1e-4
    assert max_err(A.triton_sparsemax(xd), r20) < 1e-4


@pytest.mark.parametrize("alpha", ALPHAS)
def test_large_magnitude_inputs_stay_finite(alpha):
    # tests/test_triton_entmax.py:117-126
    torch.manual_seed(0)
    x = (torch.randn(2, 32) * 100).to(DEV)
    y = A.triton_entmax(x, alpha=alpha, n_iter=10)
    assert torch.isfinite(y).all() and (y >= 0).all()
    assert max_err(y, exact.entmax_rows(x.cpu(), alpha)) < 1e-4


@pytest.mark.parametrize("cols", [1, 3, 17, 255, 1000, 1023, 4096, 8192, 12288, 40000, 70001])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_ragged_and_long_rows(cols, dtype):
    torch.manual_seed(cols)
    x = (torch.randn(5, cols) * 2).to(dtype)
    for alpha in (1.5, 2.0):
        y = A.triton_entmax(x.to(DEV), alpha=alpha)
        assert max_err(y, exact.entmax_rows(x, alpha)) < tol_for(dtype, alpha)


def test_empty_and_constant_rows():
    y = A.triton_entmax(torch.zeros(0, 16, device=DEV))
    assert y.shape == (0, 16)
    y = A.triton_entmax(torch.full((3, 64), 2.5, device=DEV))
    assert torch.allclose(y.cpu(), torch.full((3, 64), 1 / 64), atol=1e-6)
    x = torch.zeros(2, 40, device=DEV)
    x[:, 7] = 10.0
    for alpha in ALPHAS:
        y = A.triton_entmax(x, alpha=alpha)
        assert torch.allclose(y[:, 7].cpu(), torch.ones(2), atol=1e-6) and (y > 0).sum().item() == 2


def test_unaligned_view_takes_the_streaming_path():
    torch.manual_seed(3)
    base = torch.randn(4 * 100 + 1, device=DEV)
    x = base[1:].view(4, 100)  # contiguous but 4-byte aligned only
    assert x.is_contiguous() and x.data_ptr() % 16 != 0
    assert max_err(A.triton_entmax(x), exact.entmax_rows(x.cpu(), 1.5)) < 1e-4


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("alpha", [1.5, 2.0])
def test_benchmark_rows_sample(dtype, alpha):
    # rows of the bandwidth workload: x = 4 * N(0,1), 8192 columns, histogram init, n_iter = 2
    torch.manual_seed(42)
    x = (4 * torch.randn(256, 8192)).to(dtype)
    y = A.triton_entmax(x.to(DEV), alpha=alpha, n_iter=2, use_histogram=True)
    want, tau = exact.entmax_rows(x, alpha, return_tau=True)
    assert max_err(y, want) < tol_for(dtype, alpha)
    # identical support away from ties
    margin = exact.support_margin(x, tau, alpha)
    clear = margin > 1e-3
    assert ((y.cpu() > 0) == (want > 0))[clear].all()


def test_benchmark_rows_full_size_properties():
    g = torch.Generator().manual_seed(7)
    x = (4 * torch.randn(16384, 8192, generator=g)).to(torch.bfloat16)
    xd = x.to(DEV)
    for alpha in (1.5, 2.0):
        y = A.triton_entmax(xd, alpha=alpha)
        yf = y.float()
        assert (yf >= 0).all()
        assert (yf.sum(-1) - 1).abs().max().item() < 2e-2
        # shift invariance by an exactly representable shift, and a sample of rows against the oracle
        rows = torch.arange(0, 16384, 257)
        assert max_err(y[rows.to(DEV)], exact.entmax_rows(x[rows], alpha)) < 2e-2
    del xd


@pytest.mark.parametrize("alpha", ALPHAS)
def test_backward_matches_finite_differences_of_the_oracle(alpha):
    torch.manual_seed(42)
    x = torch.randn(6, 24, dtype=torch.float64)
    dy = torch.randn(6, 24, dtype=torch.float64)
    xg = x.float().to(DEV).requires_grad_(True)
    y = A.triton_entmax(xg, alpha=alpha, n_iter=10)
    (dx,) = torch.autograd.grad(y, xg, dy.float().to(DEV))
    eps = 1e-6
    for _ in range(8):
        w = torch.randn_like(x)
        fd = ((exact.entmax_rows(x + eps * w, alpha) - exact.entmax_rows(x - eps * w, alpha)) / (2 * eps) * dy).sum()
        assert abs((dx.double().cpu() * w).sum().item() - fd.item()) < 2e-3 * (1 + abs(fd.item()))


def _rows_backward_reference(y, dy, alpha):
    """dx = u * (dy - sum(u dy) / sum(u)), u = y^(2 - alpha) on the support (adasplash/triton_entmax_v2.py:541-617),
    in fp64 torch ops on the kernel's own y."""
    y64, g64 = y.double().cpu(), dy.double().cpu()
    # generic alpha: the power is taken of max(y, 1e-6), the reference's clamp (triton_entmax_v2.py:35-39)
    floor = 1e-300 if alpha in (1.5, 2.0) else 1e-6
    u = torch.where(y64 > 0, y64.clamp_min(floor) ** (2.0 - alpha), torch.zeros_like(y64))
    q = (u * g64).sum(-1, keepdim=True) / u.sum(-1, keepdim=True)
    return u * (g64 - q)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("alpha", ALPHAS)
@pytest.mark.parametrize("shape", [(64, 8192), (37, 4096), (5, 1000), (9, 24), (3, 16384), (2, 40000)])
def test_backward_kernels_match_the_closed_form(shape, alpha, dtype):
    """Every dispatch of the backward (a wave per row, a block per row, streaming for ragged or very long rows)
    against the closed form; tolerance = the output type's rounding (fp32 1e-5, or 1e-4 where the power goes
    through the hardware exp2 / log2; 16-bit 1e-2 of the largest |dx|)."""
    g = torch.Generator().manual_seed(42)
    x = (4 * torch.randn(*shape, generator=g)).to(dtype).to(DEV)
    dy = torch.randn(*shape, generator=g).to(dtype).to(DEV)
    xg = x.clone().requires_grad_(True)
    y = A.triton_entmax(xg, alpha=alpha)
    (dx,) = torch.autograd.grad(y, xg, dy)
    want = _rows_backward_reference(y.detach(), dy, alpha)
    tol = (1e-5 if alpha in (1.5, 2.0) else 1e-4) if dtype == torch.float32 else 1e-2  # generic alpha: exp2/log2 units
    scale = max(1.0, want.abs().max().item())
    assert (dx.double().cpu() - want).abs().max().item() < tol * scale
    # entries outside the support get exactly zero
    assert (dx[y == 0] == 0).all()


def test_backward_of_an_all_zero_row_is_zero():
    y = torch.zeros(4, 512, device=DEV)
    dy = torch.randn(4, 512, device=DEV)
    dx = torch.full_like(y, float("nan"))
    from adasplash_amd import _lib
    st = _lib.load().adsp_entmax_rows_bwd(y.data_ptr(), dy.data_ptr(), dx.data_ptr(), 4, 512, _lib.dtype_code(y), 1.5,
                                          _lib.current_stream(y.device))
    assert st == 0
    assert (dx == 0).all()


def test_backward_with_unaligned_buffers_takes_the_streaming_path():
    """y, dy and dx that are only 4-byte aligned cannot use 16-byte loads: same result through the fallback."""
    from adasplash_amd import _lib
    torch.manual_seed(5)
    rows, cols = 6, 256
    y_al = A.triton_entmax(4 * torch.randn(rows, cols, device=DEV), alpha=1.5)
    dy_al = torch.randn(rows, cols, device=DEV)
    bufs = [torch.empty(rows * cols + 1, device=DEV) for _ in range(3)]
    y, dy, dx = (b[1:].view(rows, cols) for b in bufs)
    y.copy_(y_al)
    dy.copy_(dy_al)
    assert all(t.data_ptr() % 16 != 0 for t in (y, dy, dx))
    lib = _lib.load()
    st = lib.adsp_entmax_rows_bwd(y.data_ptr(), dy.data_ptr(), dx.data_ptr(), rows, cols, _lib.dtype_code(y), 1.5,
                                  _lib.current_stream(y.device))
    assert st == 0
    want = _rows_backward_reference(y_al, dy_al, 1.5)
    assert (dx.double().cpu() - want).abs().max().item() < 1e-5


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("alpha", ALPHAS)
@pytest.mark.parametrize("cols", [8, 16, 24, 64, 128, 136, 256, 512, 520, 1024, 1032, 2048, 4096, 4104])
def test_forward_across_the_dispatch_boundaries(cols, alpha, dtype):
    """Row lengths on both sides of every switch between the kernel variants (16 threads per row with 1-8 chunks
    per lane, a wave per row, four waves per row) and row counts that leave the last wave / block partly empty."""
    g = torch.Generator().manual_seed(cols)
    x = (3 * torch.randn(37, cols, generator=g)).to(dtype)
    y = A.triton_entmax(x.to(DEV), alpha=alpha)
    assert max_err(y, exact.entmax_rows(x, alpha)) < tol_for(dtype, alpha)
    # a flat row has full support: every candidate list overflows its fast path
    flat = torch.zeros(5, cols).to(dtype)
    y = A.triton_entmax(flat.to(DEV), alpha=alpha)
    assert (y.float().cpu() - 1.0 / cols).abs().max().item() < (1e-6 if dtype == torch.float32 else 2e-3 / cols + 1e-4)
