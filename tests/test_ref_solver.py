"""The numpy restatement of the reference's iterative solvers stays within the reference's own test
tolerances of the exact answer, and the histogram bracket it relies on is a valid bracket."""

import numpy as np
import pytest
import torch

from oracle import exact, ref_solver


@pytest.mark.parametrize("alpha", [1.333, 1.5, 2.0])
@pytest.mark.parametrize("shape", [(2, 16), (8, 64), (32, 256)])
def test_rows_iterate_matches_exact_at_the_reference_test_settings(alpha, shape):
    # tests/test_triton_entmax.py:47-64 runs n_iter = 10 against entmax_bisect with 1e-4 (5e-4 for 1.333)
    torch.manual_seed(42)
    x = torch.randn(*shape)
    y, _ = ref_solver.entmax_rows_iterate(x.numpy(), alpha, n_iter=10, use_histogram=True)
    want = exact.entmax_rows(x, alpha).numpy()
    tol = 5e-4 if alpha == 1.333 else 1e-4
    assert np.abs(y - want).max() < tol
    assert np.abs(y.sum(-1) - 1.0).max() < 1e-2


@pytest.mark.parametrize("alpha", [1.5, 2.0])
def test_rows_default_two_steps_on_small_rows(alpha):
    # tests/test_triton_entmax.py:101-114: default n_iter with histogram, x = randn(4, 16), 1e-4
    torch.manual_seed(42)
    x = torch.randn(4, 16)
    y, _ = ref_solver.entmax_rows_iterate(x.numpy(), alpha, n_iter=2, use_histogram=True)
    assert np.abs(y - exact.entmax_rows(x, alpha).numpy()).max() < 1e-4


@pytest.mark.parametrize("sigma,n", [(0.5, 512), (0.0625, 4096), (3.0, 1024), (1.0, 64)])
def test_v2_histogram_gives_a_bracket_and_halley_converges(sigma, n):
    torch.manual_seed(0)
    z = (torch.randn(64, n) * sigma).numpy().astype(np.float32)
    bins = ref_solver.select_bins(n)
    tau_exact = exact.entmax15_threshold(torch.tensor(z, dtype=torch.float64)).numpy()
    _, t_hist, _ = ref_solver.v2_tau_iterate(z, 0, bins)
    assert (tau_exact - t_hist).min() > -1e-5            # lower bound
    assert (tau_exact - t_hist).max() < 1.0 / bins + 1e-5  # bracket width the next stage assumes
    t10, _, _ = ref_solver.v2_tau_iterate(z, 10, bins)
    assert np.abs(t10 - tau_exact).max() < 2e-6


def test_select_bins_thresholds():
    assert ref_solver.select_bins(4096) == 8 and ref_solver.select_bins(8192) == 8
    assert ref_solver.select_bins(16320) == 8 and ref_solver.select_bins(16384) == 4
    assert ref_solver.select_bins(64 * 65535) == 4 and ref_solver.select_bins(64 * 65536) == 2


@pytest.mark.parametrize("alpha", [1.333, 1.5, 2.0])
def test_v1_bracket_and_iteration(alpha):
    torch.manual_seed(1)
    z = ((alpha - 1.0) * torch.randn(32, 256) * 2.0).numpy().astype(np.float32)
    tau_exact = exact.entmax_threshold(torch.tensor(z, dtype=torch.float64), alpha).numpy()
    zmax = z.max(1)
    assert (tau_exact >= zmax - 1 - 1e-6).all() and (tau_exact <= zmax - 256.0 ** (1 - alpha) + 1e-6).all()
    t = ref_solver.v1_tau_iterate(z, alpha, 10, np.full(32, 256.0))
    assert np.abs(t - tau_exact).max() < 5e-5
