"""Numpy restatement of the reference's iterative threshold solvers, acting on dense score rows.

TEST INFRASTRUCTURE ONLY -- never imported by the shipped package.

The reference's kernels cannot be executed in this build's environments (they depend on CUDA-only
Triton externs), and the reference stores no vectors for their iterates, so the *iterates* below are
"parity unpinned".  They are used to check claims the native design relies on: that the histogram
initialisation yields a valid bracket ``tau_lo <= tau* <= tau_lo + 1/BINS`` and that the documented
number of refinement steps lands within the reference's own test tolerances of the exact entmax.

All arithmetic is float32 like the kernels'.  ``z`` always denotes already-scaled scores
``(alpha - 1) * x``; masked entries are ``-inf``.
"""

import numpy as np

F = np.float32


# --------------------------------------------------------------------------------------------------
# Standalone entmax rows: adasplash/triton_entmax_v2.py
# --------------------------------------------------------------------------------------------------
def hybrid_update(t, t_lo, t_hi, t_prev, f_prev, a0, a1, a2, alpha, allow_secant):
    """Halley -> Newton -> secant -> bisection (``adasplash/triton_entmax_v2.py:43-110``)."""
    EPS, EPS_DENOM = F(1e-6), F(1e-12)
    c0 = F(1.0 / (alpha - 1.0))
    c1 = F(c0 - 1.0)
    with np.errstate(all="ignore"):
        ff = a0 - F(1.0)
        df = -c0 * a1
        ddf = c0 * c1 * a2
        t_lo = np.where(ff > 0, t, t_lo).astype(F)
        t_hi = np.where(ff < 0, t, t_hi).astype(F)

        h_den = F(2) * df * df - ff * ddf
        t_h = t - (F(2) * ff * df) / h_den
        ok_h = (t_h > t_lo - EPS) & (t_h < t_hi + EPS) & ~np.isinf(t_h) & (np.abs(h_den) > EPS_DENOM)
        ok_h &= alpha <= 1.5
        cand = np.where(ok_h, t_h, F(0))
        has = ok_h

        t_n = t - ff / df
        ok_n = (t_n > t_lo - EPS) & (t_n < t_hi + EPS) & ~np.isinf(t_n) & (np.abs(df) > EPS_DENOM)
        ok_n &= alpha <= 2.0
        take = ok_n & ~has
        cand = np.where(take, t_n, cand)
        has = has | take

        if allow_secant:
            s_den = ff - f_prev
            t_s = t - ff * (t - t_prev) / s_den
            ok_s = (t_s > t_lo - EPS) & (t_s < t_hi + EPS) & ~np.isinf(t_s) & (np.abs(s_den) > EPS_DENOM)
            take = ok_s & ~has
            cand = np.where(take, t_s, cand)
            has = has | take
    return np.where(has, cand, F(0.5) * (t_lo + t_hi)).astype(F), t_lo, t_hi


def histogram_counts(z, t_init, bins):
    """Counts of ``proj = z - t_init`` in ``bins`` equal bins of [0, 1]; entries with proj < 0 dropped,
    proj >= 1 clamped into the top bin (``adasplash/triton_entmax_v2.py:426-431``,
    ``adasplash/adasplash_v2.py:402-410``)."""
    with np.errstate(all="ignore"):
        proj = (z - t_init[:, None]).astype(F)
        b = np.floor(proj * F(bins))
    b = np.where(np.isfinite(b), b, -1.0)
    b = np.minimum(b, bins - 1).astype(np.int64)
    counts = np.zeros((z.shape[0], bins), dtype=np.float32)
    for j in range(bins):
        counts[:, j] = ((b == j) & (proj >= 0)).sum(axis=1)
    return counts


def hist_init_alpha2(counts, t_init):
    """``adasplash/triton_entmax_v2.py:114-131``: greedy top-down scan with every element of a bin placed
    on the bin's lower edge; the max element itself enters as (z=1, k=1)."""
    bins = counts.shape[1]
    sum_z = np.ones(counts.shape[0], F)
    sum_k = np.ones(counts.shape[0], F)
    for sj in range(bins - 1, -1, -1):
        c = counts[:, sj].copy()
        if sj == bins - 1:
            c -= 1
        c_tau = F(sj / bins)
        new_z = sum_z + c * c_tau
        new_k = sum_k + c
        good = (new_z - new_k * c_tau) < 1.0
        sum_z = np.where(good, new_z, sum_z)
        sum_k = np.where(good, new_k, sum_k)
    return (t_init + (sum_z - F(1)) / sum_k).astype(F)


def hist_init_alpha15(counts, t_init):
    """``adasplash/triton_entmax_v2.py:135-155`` and ``adasplash/adasplash_v2.py:434-461``."""
    bins = counts.shape[1]
    n = counts.shape[0]
    sum_z, sum_k, sum_zz = np.ones(n, F), np.ones(n, F), np.ones(n, F)
    for sj in range(bins - 1, -1, -1):
        c = counts[:, sj].copy()
        if sj == bins - 1:
            c -= 1
        c_tau = F(sj / bins)
        new_z = sum_z + c * c_tau
        new_k = sum_k + c
        new_zz = sum_zz + c * (c_tau * c_tau)
        good = new_k * c_tau * c_tau - F(2) * new_z * c_tau + new_zz < 1.0
        sum_zz = np.where(good, new_zz, sum_zz)
        sum_z = np.where(good, new_z, sum_z)
        sum_k = np.where(good, new_k, sum_k)
    disc = np.maximum(sum_z * sum_z - sum_k * (sum_zz - F(1)), 0)
    return (t_init + (sum_z - np.sqrt(disc)) / sum_k).astype(F)


def evaluate_f_hist(tau, t_shift, counts):
    """Bin-centre surrogate ``sum_b c_b [centre_b - tau]_+^2 - 1`` (``triton_entmax_v2.py:165-204``)."""
    bins = counts.shape[1]
    acc = np.zeros_like(tau)
    for b in range(bins):
        d = np.maximum(t_shift + F((b + 0.5) / bins) - tau, 0)
        acc = acc + counts[:, b] * d * d
    return (acc - F(1)).astype(F)


def hist_init_tau_muller(t_lo, t_hi, t_shift, counts):
    """Quadratic fit of the surrogate at lo/mid/hi, root nearest ``hi`` (``triton_entmax_v2.py:208-322``)."""
    EPS = F(1e-10)
    a, c = t_lo, t_hi
    b = F(0.5) * (a + c)
    fa, fb, fc = (evaluate_f_hist(p, t_shift, counts) for p in (a, b, c))
    with np.errstate(all="ignore"):
        den = (a - b) * (a - c) * (b - c)
        A = (fa * (b - c) + fb * (c - a) + fc * (a - b)) / den
        B = (fa * (c * c - b * b) + fb * (a * a - c * c) + fc * (b * b - a * a)) / den
        C = (fa * b * c * (b - c) + fb * a * c * (c - a) + fc * a * b * (a - b)) / den
        mid = F(0.5) * (a + c)
        x_lin = np.where(np.abs(B) > EPS, -C / B, mid)
        disc = B * B - F(4) * A * C
        sq = np.sqrt(np.maximum(disc, 0))
        r1, r2 = (-B + sq) / (F(2) * A), (-B - sq) / (F(2) * A)
        v1, v2 = (r1 >= a) & (r1 <= c), (r2 >= a) & (r2 <= c)
        x_quad = np.where(v1 & v2, np.where(np.abs(c - r1) <= np.abs(c - r2), r1, r2),
                          np.where(v1, r1, np.where(v2, r2, mid)))
        s_den = fc - fa
        x_sec = np.where(np.abs(s_den) > EPS, c - fc * (c - a) / s_den, mid)
        x_quad = np.where(disc >= 0, x_quad, x_sec)
        x = np.where(np.abs(A) < EPS, x_lin, x_quad)
        x = np.where(np.abs(den) < EPS, mid, x)
    return np.minimum(np.maximum(x, a), c).astype(F)


def _stats(z, t, alpha):
    """acc_0, acc_1, acc_2 of ``triton_entmax_v2.py:461-489`` for threshold ``t``."""
    with np.errstate(all="ignore"):
        d = (z - t[:, None]).astype(F)
        m = d > 0
        u = np.where(m, d, F(0))
        if alpha == 2.0:
            return u.sum(1, dtype=F), m.sum(1).astype(F), np.zeros(z.shape[0], F)
        if alpha == 1.5:
            return (u * u).sum(1, dtype=F), u.sum(1, dtype=F), m.sum(1).astype(F)
        c0 = 1.0 / (alpha - 1.0)
        lg = np.log2(np.maximum(u, F(1e-6)))

        def mp(c):
            return np.where(m, np.exp2(lg * F(c)), F(0)).sum(1, dtype=F)

        return mp(c0), mp(c0 - 1), mp(c0 - 2)


def entmax_rows_iterate(x, alpha=1.5, n_iter=2, use_histogram=True):
    """The reference's standalone entmax forward (``triton_entmax_v2.py:363-536`` behind the argument
    fix-ups of ``:713-716``) on rows ``x`` (2-D, float).  Returns ``(y, tau)`` in float32."""
    if alpha not in (1.5, 2.0):
        use_histogram = False
        n_iter = max(n_iter, 10)
    BINS = 4
    z = (np.asarray(x, dtype=F) * F(alpha - 1.0)).astype(F)
    zmax = z.max(axis=1)
    if use_histogram and alpha <= 2.0:
        t_shift = (zmax - F(1)).astype(F)
        counts = histogram_counts(z, t_shift, BINS)
        t_lo = hist_init_alpha15(counts, t_shift) if alpha == 1.5 else hist_init_alpha2(counts, t_shift)
        t_hi = (t_lo + F(1.0 / BINS)).astype(F)
        t = hist_init_tau_muller(t_lo, t_hi, t_shift, counts)
    else:
        t_hi = zmax.copy()
        t_lo = (zmax - F(1)).astype(F)
        t = (F(0.5) * (t_lo + t_hi)).astype(F)
    t_prev, f_prev = t.copy(), np.zeros_like(t)
    for it in range(n_iter):
        a0, a1, a2 = _stats(z, t, alpha)
        t_new, t_lo, t_hi = hybrid_update(t, t_lo, t_hi, t_prev, f_prev, a0, a1, a2, alpha, it > 0)
        t_prev, f_prev, t = t, (a0 - F(1)).astype(F), t_new
    with np.errstate(all="ignore"):
        u = np.maximum(z - t[:, None], 0).astype(F)
    y = u if alpha == 2.0 else (u * u if alpha == 1.5 else np.where(u > 0, np.exp2(
        np.log2(np.maximum(u, F(1e-6))) * F(1.0 / (alpha - 1.0))), F(0)))
    return y.astype(F), t


# --------------------------------------------------------------------------------------------------
# AdaSplash-2 threshold pipeline on dense scaled score rows: adasplash/adasplash_v2.py
# --------------------------------------------------------------------------------------------------
def select_bins(n_ctx, block_n=64):
    """``adasplash/adasplash_v2.py:273-289``."""
    max_count = (n_ctx + block_n - 1) // block_n
    for bins in (8, 4, 2):
        if max_count <= (1 << (64 // bins)) - 1:
            return bins
    raise ValueError(f"N_CTX={n_ctx} too large for uint64 packed histogram")


def halley_bisect_update_v2(t, t_lo, t_hi, a0, a1, a2):
    """``adasplash/adasplash_v2.py:69-90`` (alpha = 1.5)."""
    EPS = F(1e-5)
    with np.errstate(all="ignore"):
        ff = a0 - F(1)
        df = F(-2) * a1
        ddf = F(2) * a2
        t_lo = np.where(ff > 0, t, t_lo).astype(F)
        t_hi = np.where(ff < 0, t, t_hi).astype(F)
        new_t = t - (ff * df) / (df * df - F(0.5) * ff * ddf)
        good = (new_t > t_lo - EPS) & (new_t < t_hi + EPS)
    return np.where(good, new_t, F(0.5) * (t_lo + t_hi)).astype(F), t_lo, t_hi


def v2_tau_iterate(z, niter=1, bins=8):
    """max -> histogram bracket -> ``niter`` Halley passes -> one more stats pass + final update
    (``adasplash/adasplash_v2.py:239-270,402-461,563-681``).  ``z`` = 0.5 * scores / sqrt(D), masked = -inf.
    Returns ``(tau, tau_lo_hist, tau_before_final_update)``."""
    z = np.asarray(z, dtype=F)
    t0 = (z.max(axis=1) - F(1)).astype(F)
    counts = histogram_counts(z, t0, bins)
    t_lo = hist_init_alpha15(counts, t0)
    t_hist = t_lo.copy()
    t_hi = (t_lo + F(1.0 / bins)).astype(F)
    t = (F(0.5) * (t_lo + t_hi)).astype(F)
    t_pre = t
    for _ in range(niter + 1):
        t_pre = t
        a0, a1, a2 = _stats(z, t, 1.5)
        t, t_lo, t_hi = halley_bisect_update_v2(t, t_lo, t_hi, a0, a1, a2)
    return t, t_hist, t_pre


# --------------------------------------------------------------------------------------------------
# AdaSplash-1 threshold pipeline on dense scaled score rows: adasplash/adasplash_block_mask.py
# --------------------------------------------------------------------------------------------------
def v1_tau_iterate(z, alpha, niter, n_valid):
    """Bracket ``[max - 1, max - n^(1-alpha)]``, midpoint start, ``niter`` generic-alpha Halley/bisect
    steps (``adasplash/adasplash_block_mask.py:15-36,167-227``).  ``n_valid`` is the per-row element
    count the reference plugs in (``1 + q_idx`` causal, ``1 + seqlen`` otherwise -- sic)."""
    EPS = F(1e-6)
    z = np.asarray(z, dtype=F)
    c0 = F(1.0 / (alpha - 1.0))
    c1 = F(c0 - 1)
    zmax = z.max(axis=1)
    t_hi = (zmax - np.exp2(F(1 - alpha) * np.log2(np.asarray(n_valid, dtype=F)))).astype(F)
    t_lo = (zmax - F(1)).astype(F)
    t = (F(0.5) * (t_lo + t_hi)).astype(F)
    for _ in range(niter):
        with np.errstate(all="ignore"):
            d = z - t[:, None]
            m = d > 0
            lg = np.log2(np.where(m, d, F(1)))
            a0 = np.where(m, np.exp2(lg * c0), F(0)).sum(1, dtype=F)
            a1 = np.where(m, np.exp2(lg * c1), F(0)).sum(1, dtype=F)
            a2 = np.where(m, np.exp2(lg * F(c1 - 1)), F(0)).sum(1, dtype=F)
            ff = a0 - F(1)
            df = -c0 * a1
            ddf = c0 * c1 * a2
            t_lo = np.where(ff > 0, t, t_lo).astype(F)
            t_hi = np.where(ff < 0, t, t_hi).astype(F)
            new_t = t - (F(2) * ff * df) / (F(2) * df * df - ff * ddf)
            good = (new_t > t_lo - EPS) & (new_t < t_hi + EPS)
        t = np.where(good, new_t, F(0.5) * (t_lo + t_hi)).astype(F)
    return t
