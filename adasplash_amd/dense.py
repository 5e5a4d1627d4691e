"""Dense entmax attention built from the rows kernel: the counterpart of ``examples/attention.py``.

``slow_entmax_attention`` materialises the score matrix (library GEMMs through ``torch.matmul``), applies
ALiBi, causal and padding masks, and takes the entmax of every row with the HIP rows kernel behind
``triton_entmax``.  It serves the options the fused kernels do not have -- ALiBi slopes, left padding,
``q_len != k_len`` with a bottom-right aligned causal mask -- and small correctness checks; it needs memory
quadratic in the sequence length.  Names, arguments, defaults and errors follow
``examples/attention.py:8-31`` (helpers) and ``:34-91`` (``slow_entmax_attention``), ``:94-104``
(``flash_entmax_attention``).
"""

import math

import torch


def _varlen_mask(varlen, size, padding):
    """(B, size) boolean map of the positions inside each sequence: the first ``varlen[b]`` of them with right
    padding, the last ``varlen[b]`` with left padding."""
    if padding not in ("right", "left"):
        raise ValueError("padding must be either 'right' or 'left'.")
    first = torch.zeros_like(varlen) if padding == "right" else size - varlen
    idx = torch.arange(size, device=varlen.device).unsqueeze(0)
    return (idx >= first.unsqueeze(1)) & (idx < (first + varlen).unsqueeze(1))


def _alibi_bias(q, k, alibi_slopes):
    n_heads, q_len = q.shape[1], q.shape[2]
    k_len = k.shape[-2]
    if alibi_slopes.shape != (n_heads,):
        raise ValueError(f"alibi_slopes must have shape ({n_heads},); got {tuple(alibi_slopes.shape)}.")
    k_pos = torch.arange(k_len, device=q.device)
    if q_len == 1 and k_len > 1:
        rel_pos = (k_pos - (k_len - 1)).view(1, 1, 1, k_len)  # a single decoding step sits on the last key
    else:
        rel_pos = (k_pos[None, :] - torch.arange(q_len, device=q.device)[:, None]).view(1, 1, q_len, k_len)
    return alibi_slopes.to(q.device).view(1, n_heads, 1, 1) * rel_pos


def slow_entmax_attention(q, k, v, alpha=1.5, varlen=None, is_causal=False, padding="right", niter=2,
                          alibi_slopes=None):
    """Dense entmax attention ``entmax_alpha(q k^T / sqrt(D) + bias) v`` (``examples/attention.py:34-91``).

    q: (B, H, q_len, D); k, v: (B, H, k_len, D).  ``varlen`` (B,) masks keys outside each sequence (right or left
    padded); with ``q_len == k_len`` the padded query rows are returned as zeros.  ``is_causal`` with
    ``q_len != k_len`` aligns the mask to the bottom right (the queries are the last ``q_len`` positions).
    """
    from . import triton_entmax

    if q.dim() != 4 or k.dim() != 4 or v.dim() != 4:
        raise ValueError("q, k and v must have shape (batch, heads, seq_len, head_dim).")
    if k.shape != v.shape:
        raise ValueError(f"k and v must have the same shape; got {tuple(k.shape)} and {tuple(v.shape)}.")
    if q.shape[0] != k.shape[0] or q.shape[1] != k.shape[1] or q.shape[3] != k.shape[3]:
        raise ValueError("q, k and v must agree on batch, heads and head_dim.")

    if varlen is not None and (varlen.dim() != 1 or varlen.shape[0] != q.shape[0]):
        raise ValueError(f"varlen must be a 1-D tensor of shape ({q.shape[0]},).")

    dev = q.device
    q_len, k_len, head_dim = q.shape[2], k.shape[2], q.shape[3]
    # the score matrix is formed and kept in fp32 whatever the input type (a 16-bit GEMM result would round scores of
    # a few units by up to 2^-8 of their size before the entmax, which the fused kernels never do)
    scores = torch.matmul(q.float(), k.float().transpose(-1, -2)) * (1.0 / math.sqrt(head_dim))
    if alibi_slopes is not None:
        scores = scores + _alibi_bias(q, k, alibi_slopes)

    # one boolean (B or 1, 1, q_len, k_len) map of the (query, key) pairs that may interact
    k_pos = torch.arange(k_len, device=dev)
    keep = None
    if is_causal:
        q_pos = torch.arange(q_len, device=dev) + (k_len - q_len)  # the queries are the last q_len positions
        keep = (k_pos[None, :] <= q_pos[:, None])[None, None]
    rows_live = None
    if varlen is not None:
        keys_live = _varlen_mask(varlen.to(dev), k_len, padding)[:, None, None, :]
        keep = keys_live if keep is None else (keep & keys_live)
        if q_len == k_len:
            rows_live = _varlen_mask(varlen.to(dev), q_len, padding)[:, None, :, None]
    if keep is not None:
        scores = scores.masked_fill(~keep, float("-inf"))
    if rows_live is not None:
        scores = scores.masked_fill(~rows_live, 0.0)  # padded rows stay finite here and are zeroed below

    probs = triton_entmax(scores.contiguous(), alpha=alpha, n_iter=niter, fast_math=False)
    # the probabilities go back to v's type for the second product
    out = torch.matmul(probs.to(v.dtype), v)
    return out if rows_live is None else out.masked_fill(~rows_live, 0)


def flash_entmax_attention(q, k, v, alpha=1.5, varlen=None, is_causal=True, niter=None):
    """The fused dispatcher under the example's name (``examples/attention.py:94-104``)."""
    from . import adasplash

    return adasplash(q, k, v, alpha=alpha, is_causal=is_causal, varlen=varlen, niter=niter)
