"""Helpers shared by the GPU parity tests."""

import math

import torch

from oracle import exact

DEV = "cuda"


def tol_for(dtype, alpha=1.5):
    """Tolerances on max |got - oracle|: fp32 1e-4 (5e-4 for alpha = 1.333, as the reference's own tests
    allow, tests/test_triton_entmax.py:17-20), 16-bit types 2e-2."""
    if dtype == torch.float32:
        return 5e-4 if alpha == 1.333 else 1e-4
    return 2e-2


# Every 16-bit comparison made through max_err leaves its raw figures here; tests/conftest.py prints the worst of
# them at the end of a GPU run, beside the magnitude-scaled figure the assertions use.
RAW_16BIT = []


def max_err(got, want, report=True):
    """max |got - want|.  For 16-bit outputs the error of entries with |want| > 2 is divided by |want| / 2:
    a bf16 value in [2, 4) cannot be stored more accurately than 2^-7 (in [4, 8): 2^-6), so the 2e-2
    max-abs bound is meant for outputs of ordinary size and scales with the magnitude beyond it.  Entries with
    |want| <= 2 are therefore held to the caller's bound unscaled; the raw maximum over all entries and over those
    entries is recorded for the end-of-run report (``report=False``: a comparison that is held to another bound on
    purpose, such as niter = 0, stays out of it)."""
    g = got.detach().double().cpu()
    w = want.double()
    err = (g - w).abs()
    if got.dtype in (torch.bfloat16, torch.float16):
        small = w.abs() <= 2.0
        raw_small = err[small].max().item() if small.any() else 0.0
        scaled = (err / torch.clamp(w.abs() / 2.0, min=1.0)).max().item()
        if report:
            RAW_16BIT.append((err.max().item(), raw_small, scaled, w.abs().max().item()))
        return max(scaled, raw_small)
    return err.max().item()


def oracle_rows_of_attention(q, k, v, b, h, rows, alpha, is_causal, L):
    """Exact output for a few query rows of one (batch, head) against all keys (cheap at any N)."""
    Hq, Hkv = q.shape[1], k.shape[1]
    kvh = h // (Hq // Hkv)
    D = q.shape[-1]
    qq = q[b, h, rows].double().cpu()
    kk = k[b, kvh, :L].double().cpu()
    vv = v[b, kvh, :L].double().cpu()
    s = qq @ kk.t() / math.sqrt(D)
    if is_causal:
        pos = torch.arange(L)[None, :]
        s = s.masked_fill(pos > torch.as_tensor(rows)[:, None], float("-inf"))
    p = exact.entmax_rows(s, alpha)
    return p @ vv
