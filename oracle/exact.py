"""Exact alpha-entmax rows and dense entmax attention on the CPU (torch, fp64 by default).

TEST INFRASTRUCTURE ONLY -- never imported by the shipped package.

Conventions follow the reference:

* ``entmax_alpha(x)_j = [(alpha-1) x_j - tau]_+^{1/(alpha-1)}`` with ``tau`` the root of
  ``sum_j [(alpha-1) x_j - tau]_+^{1/(alpha-1)} = 1``
  (``adasplash/triton_entmax_v2.py:390-393,520-536``: scores are scaled by ``alpha-1`` before the
  threshold is applied, the output is not renormalised).
* attention: ``scores = q k^T / sqrt(D)``, causal / varlen masks fill with ``-inf``, padded query
  rows get score 0 so the row stays finite and are zeroed in the output
  (``examples/attention.py:61-90``); GQA repeats each K/V head over its query group
  (``tests/test_adasplash_v2.py:340-342``, ``adasplash/adasplash_v2.py:194-195``).

Three independent threshold algorithms are provided so they can be checked against each other:
sort based sparsemax (Martins & Astudillo 2016), sort based entmax-1.5 (Peters, Niculae & Martins
2019, Alg. 2) and plain bisection for any alpha > 1.
"""

import math

import torch

NEG_INF = float("-inf")


def _as2d(z):
    return z.reshape(-1, z.shape[-1])


def sparsemax_threshold(z):
    """tau of sparsemax for rows ``z`` (already scaled by alpha-1 = 1).  ``-inf`` entries are ignored.

    k* = max{k : 1 + k z_(k) > sum_{i<=k} z_(i)},  tau = (sum_{i<=k*} z_(i) - 1) / k*.
    """
    z2 = _as2d(z)
    zmax = z2.max(dim=-1, keepdim=True).values
    zs = torch.sort(z2 - zmax, dim=-1, descending=True).values  # shift: exact arithmetic near 0
    finite = torch.isfinite(zs)
    zs0 = torch.where(finite, zs, torch.zeros_like(zs))
    csum = torch.cumsum(zs0, dim=-1)
    ks = torch.arange(1, z2.shape[-1] + 1, dtype=z2.dtype).expand_as(zs)
    cond = (1.0 + ks * zs0 > csum) & finite
    kstar = cond.to(torch.int64).sum(dim=-1, keepdim=True).clamp(min=1)
    tau = (torch.gather(csum, -1, kstar - 1) - 1.0) / kstar.to(z2.dtype)
    return (tau + zmax).reshape(z.shape[:-1])


def entmax15_threshold(z):
    """tau of entmax-1.5 for rows ``z`` (already scaled by alpha-1 = 0.5): sum [z - tau]_+^2 = 1.

    For the top-k prefix with mean M_k and mean square Q_k the candidate threshold is
    tau_k = M_k - sqrt((1 - k (Q_k - M_k^2)) / k); the support size is #{k : tau_k <= z_(k)}.
    """
    z2 = _as2d(z)
    zmax = z2.max(dim=-1, keepdim=True).values
    zs = torch.sort(z2 - zmax, dim=-1, descending=True).values
    finite = torch.isfinite(zs)
    zs0 = torch.where(finite, zs, torch.zeros_like(zs))
    ks = torch.arange(1, z2.shape[-1] + 1, dtype=z2.dtype).expand_as(zs)
    mean = torch.cumsum(zs0, dim=-1) / ks
    mean_sq = torch.cumsum(zs0 * zs0, dim=-1) / ks
    ss = ks * (mean_sq - mean * mean)
    delta = ((1.0 - ss) / ks).clamp(min=0.0)
    tau_k = mean - torch.sqrt(delta)
    cond = (tau_k <= zs0) & finite
    kstar = cond.to(torch.int64).sum(dim=-1, keepdim=True).clamp(min=1)
    tau = torch.gather(tau_k, -1, kstar - 1)
    return (tau + zmax).reshape(z.shape[:-1])


def bisect_threshold(z, alpha, n_iter=120):
    """tau by bisection of f(tau) = sum [z - tau]_+^{1/(alpha-1)} - 1 on [max-1, max]; any alpha > 1."""
    z2 = _as2d(z)
    c0 = 1.0 / (alpha - 1.0)
    zmax = z2.max(dim=-1, keepdim=True).values
    lo = zmax - 1.0
    hi = zmax.clone()
    for _ in range(n_iter):
        mid = 0.5 * (lo + hi)
        f = torch.clamp(z2 - mid, min=0.0).pow(c0).sum(dim=-1, keepdim=True) - 1.0
        pos = f > 0
        lo = torch.where(pos, mid, lo)
        hi = torch.where(pos, hi, mid)
    return (0.5 * (lo + hi)).reshape(z.shape[:-1])


def entmax_threshold(z, alpha):
    """Exact tau for already-scaled rows ``z = (alpha-1) x``."""
    if alpha == 2.0:
        return sparsemax_threshold(z)
    if alpha == 1.5:
        return entmax15_threshold(z)
    return bisect_threshold(z, alpha)


def entmax_rows(x, alpha=1.5, dtype=torch.float64, return_tau=False):
    """Exact entmax over the last dim of ``x``.  Returns ``y`` (and ``tau`` in scaled units)."""
    if not alpha > 1.0:
        raise ValueError("alpha must be > 1")
    z = x.to(dtype) * (alpha - 1.0)
    tau = entmax_threshold(z, alpha)
    u = torch.clamp(z - tau.unsqueeze(-1), min=0.0)
    if alpha == 2.0:
        y = u
    elif alpha == 1.5:
        y = u * u
    else:
        y = u.pow(1.0 / (alpha - 1.0))
    return (y, tau) if return_tau else y


def support_margin(x, tau, alpha):
    """|(alpha-1) x_j - tau| per element: entries with a small margin are ties whose support may differ."""
    return (x.to(tau.dtype) * (alpha - 1.0) - tau.unsqueeze(-1)).abs()


def attention_scores(q, k, is_causal, varlen=None, dtype=torch.float64):
    """Dense masked scores ``q k^T / sqrt(D)`` (``examples/attention.py:61-83``), right padding.

    Returns ``(scores, row_valid)`` where ``row_valid`` is ``None`` or a bool ``(B, 1, N, 1)`` mask of
    non-padded query rows.  K/V heads are repeated over the query group when ``Hkv < Hq``.
    """
    B, Hq, Nq, D = q.shape
    Hkv, Nk = k.shape[1], k.shape[2]
    if Hq % Hkv:
        raise ValueError("Hq must be a multiple of Hkv")
    qd = q.to(dtype)
    kd = k.to(dtype)
    if Hkv != Hq:
        kd = kd.repeat_interleave(Hq // Hkv, dim=1)
    scores = torch.matmul(qd, kd.transpose(-1, -2)) / math.sqrt(D)
    if is_causal:
        q_pos = torch.arange(Nq) + (Nk - Nq)
        k_pos = torch.arange(Nk)
        causal = q_pos[:, None] >= k_pos[None, :]
        scores = scores.masked_fill(~causal.view(1, 1, Nq, Nk), NEG_INF)
    row_valid = None
    if varlen is not None:
        vl = varlen.to(torch.int64).cpu()
        key_mask = torch.arange(Nk)[None, :] < vl[:, None]
        scores = scores.masked_fill(~key_mask[:, None, None, :], NEG_INF)
        if Nq == Nk:
            row_valid = (torch.arange(Nq)[None, :] < vl[:, None])[:, None, :, None]
            scores = scores.masked_fill(~row_valid, 0.0)
    return scores, row_valid


def dense_entmax_attention(q, k, v, alpha=1.5, is_causal=False, varlen=None, dtype=torch.float64,
                           return_aux=False):
    """Dense exact entmax attention; the parity oracle for the fused kernels.

    q: (B, Hq, N, D); k, v: (B, Hkv, N, D); varlen: optional (B,) valid lengths (right padding).
    Output has q's shape in ``dtype``; padded query rows are exactly zero.
    """
    scores, row_valid = attention_scores(q, k, is_causal, varlen, dtype)
    probs, tau = entmax_rows(scores, alpha, dtype=dtype, return_tau=True)
    vd = v.to(dtype)
    if v.shape[1] != q.shape[1]:
        vd = vd.repeat_interleave(q.shape[1] // v.shape[1], dim=1)
    out = torch.matmul(probs, vd)
    if row_valid is not None:
        out = out.masked_fill(~row_valid, 0.0)
    if return_aux:
        return out, probs, tau, scores
    return out


def dense_entmax_attention_general(q, k, v, alpha=1.5, is_causal=False, varlen=None, padding="right",
                                   alibi_slopes=None, dtype=torch.float64):
    """The dense example path with all its options (``examples/attention.py:8-31,34-91``), exact entmax, fp64.

    ALiBi adds ``slope_h * (j - i)`` to the score of query ``i`` and key ``j`` (``j - (k_len - 1)`` for a single
    query row); ``padding="left"`` keeps the *last* ``varlen[b]`` positions; a causal mask with
    ``q_len != k_len`` is aligned to the bottom right; padded query rows (only defined when
    ``q_len == k_len``) are zero.  Written as explicit loops over batch and head so that it shares no tensor
    expression with the implementation under test.
    """
    B, H, Nq, D = q.shape
    Nk = k.shape[2]
    out = torch.zeros(B, H, Nq, v.shape[3], dtype=dtype)
    for b in range(B):
        if varlen is None:
            keys = list(range(Nk))
        else:
            L = int(varlen[b])
            keys = list(range(L)) if padding == "right" else list(range(Nk - L, Nk))
        keyset = set(keys)
        for h in range(H):
            for i in range(Nq):
                if varlen is not None and Nq == Nk and i not in keyset:
                    continue  # padded query row: zero
                pos_i = i + (Nk - Nq)  # position of the query among the keys (bottom-right alignment)
                cols = [j for j in keys if (not is_causal) or j <= pos_i]
                if not cols:
                    continue
                s = (k[b, h, cols].to(dtype) @ q[b, h, i].to(dtype)) / math.sqrt(D)
                if alibi_slopes is not None:
                    ref_i = (Nk - 1) if (Nq == 1 and Nk > 1) else i
                    s = s + float(alibi_slopes[h]) * (torch.tensor(cols, dtype=dtype) - ref_i)
                p = entmax_rows(s[None, :], alpha, dtype=dtype)[0]
                out[b, h, i] = p @ v[b, h, cols].to(dtype)
    return out


def dense_entmax_attention_general_grads(q, k, v, dout, alpha=1.5, is_causal=False, varlen=None, padding="right",
                                         alibi_slopes=None, dtype=torch.float64):
    """Gradients (dq, dk, dv) of ``dense_entmax_attention_general`` for the upstream gradient ``dout``: what autograd
    returns for the example path (``examples/attention.py:34-91``; its test takes them at
    ``tests/test_attention.py:50-77``).  Per query row, on the keys it sees: p = entmax(s), u = p^(2 - alpha),
    dP = v_j . dout_i, dX = u * (dP - sum(u dP) / sum(u)); dq_i = sum_j dX_j k_j / sqrt(D), dk_j += dX_j q_i / sqrt(D),
    dv_j += p_j dout_i.  The ALiBi term is a constant added to the scores and has no gradient; padded query rows and
    the rows of ``dout`` that belong to them contribute nothing.  The same loops as the forward, so that it shares no
    tensor expression with the implementation under test; pinned by finite differences in tests/test_oracle.py."""
    B, H, Nq, D = q.shape
    Nk = k.shape[2]
    dq = torch.zeros(B, H, Nq, D, dtype=dtype)
    dk = torch.zeros(B, H, Nk, D, dtype=dtype)
    dv = torch.zeros(B, H, Nk, v.shape[3], dtype=dtype)
    for b in range(B):
        if varlen is None:
            keys = list(range(Nk))
        else:
            L = int(varlen[b])
            keys = list(range(L)) if padding == "right" else list(range(Nk - L, Nk))
        keyset = set(keys)
        for h in range(H):
            for i in range(Nq):
                if varlen is not None and Nq == Nk and i not in keyset:
                    continue
                pos_i = i + (Nk - Nq)
                cols = [j for j in keys if (not is_causal) or j <= pos_i]
                if not cols:
                    continue
                kc, vc = k[b, h, cols].to(dtype), v[b, h, cols].to(dtype)
                qi, doi = q[b, h, i].to(dtype), dout[b, h, i].to(dtype)
                s = (kc @ qi) / math.sqrt(D)
                if alibi_slopes is not None:
                    ref_i = (Nk - 1) if (Nq == 1 and Nk > 1) else i
                    s = s + float(alibi_slopes[h]) * (torch.tensor(cols, dtype=dtype) - ref_i)
                p = entmax_rows(s[None, :], alpha, dtype=dtype)[0]
                u = torch.where(p > 0, p.clamp_min(1e-300) ** (2.0 - alpha), torch.zeros_like(p))
                dp = vc @ doi
                dx = u * (dp - (u * dp).sum() / u.sum())
                dq[b, h, i] = (dx @ kc) / math.sqrt(D)
                dk[b, h, cols] += dx[:, None] * qi[None, :] / math.sqrt(D)
                dv[b, h, cols] += p[:, None] * doi[None, :]
    return dq, dk, dv


def dense_entmax_attention_grads(q, k, v, dout, alpha=1.5, is_causal=False, varlen=None, dtype=torch.float64):
    """Gradients (dq, dk, dv) of ``dense_entmax_attention`` for the upstream gradient ``dout``.

    Closed form of the entmax Jacobian: with u = p^(2 - alpha), dX = u * (dP - sum(u dP) / sum(u)) on the
    scaled scores x = q.k / sqrt(D), where dP = dout . v^T (what adasplash/adasplash_v2.py:1062-1068 and
    :1196-1215 compute with u = [z - tau]_+ for alpha = 1.5).  Checked in tests/test_oracle.py against central
    finite differences of the forward oracle.  Padded query rows contribute nothing; padded keys get zero.
    """
    out, probs, tau, scores = dense_entmax_attention(q, k, v, alpha, is_causal, varlen, dtype, return_aux=True)
    B, Hq, N, D = q.shape
    Hkv = k.shape[1]
    g = Hq // Hkv
    qd, kd, vd, dod = (t.to(dtype) for t in (q, k, v, dout))
    ke = kd.repeat_interleave(g, dim=1) if g > 1 else kd
    ve = vd.repeat_interleave(g, dim=1) if g > 1 else vd
    if varlen is not None:
        row_valid = (torch.arange(N)[None, :] < varlen.to(torch.long)[:, None])[:, None, :, None]
        dod = dod.masked_fill(~row_valid, 0.0)
        probs = probs.masked_fill(~row_valid, 0.0)
    u = torch.where(probs > 0, probs.clamp_min(1e-300) ** (2.0 - alpha), torch.zeros_like(probs))
    dp = torch.matmul(dod, ve.transpose(-1, -2))
    delta = (u * dp).sum(-1, keepdim=True) / u.sum(-1, keepdim=True).clamp_min(1e-300)
    dx = u * (dp - delta)
    sm = 1.0 / math.sqrt(D)
    dq = torch.matmul(dx, ke) * sm
    dk = torch.matmul(dx.transpose(-1, -2), qd) * sm
    dv = torch.matmul(probs.transpose(-1, -2), dod)
    if g > 1:
        dk = dk.view(B, Hkv, g, N, D).sum(2)
        dv = dv.view(B, Hkv, g, N, D).sum(2)
    return dq, dk, dv


def dense_entmax_attention_loop(q, k, v, alpha=1.5, is_causal=False, varlen=None):
    """Brute-force per-row restatement (python loops, tiny sizes only) used to pin the dense version."""
    B, Hq, N, D = q.shape
    Hkv = k.shape[1]
    g = Hq // Hkv
    out = torch.zeros(B, Hq, N, D, dtype=torch.float64)
    for b in range(B):
        L = N if varlen is None else int(varlen[b])
        for h in range(Hq):
            kk = k[b, h // g, :L].double()
            vv = v[b, h // g, :L].double()
            for i in range(L):
                n_keys = i + 1 if is_causal else L
                s = (kk[:n_keys] @ q[b, h, i].double()) / math.sqrt(D)
                p = entmax_rows(s[None, :], alpha)[0]
                out[b, h, i] = p @ vv[:n_keys]
    return out
