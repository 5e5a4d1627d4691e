"""Pins the CPU oracle against evidence that does not share its code path:
the variational definition of alpha-entmax, closed forms, limits, invariances, brute force."""

import itertools
import math

import numpy as np
import pytest
import torch
from scipy.optimize import minimize

from oracle import exact

ALPHAS = [1.333, 1.5, 2.0]


def tsallis_objective(p, x, alpha):
    """p.x + H_alpha(p), H_alpha(p) = sum_j (p_j - p_j^alpha) / (alpha (alpha - 1)); entmax is its argmax."""
    p = np.clip(p, 0.0, None)
    return float(p @ x + (p - p**alpha).sum() / (alpha * (alpha - 1.0)))


@pytest.mark.parametrize("alpha", ALPHAS)
def test_entmax_is_the_maximiser_of_the_tsallis_objective(alpha):
    rng = np.random.default_rng(0)
    for n in (2, 3, 5, 7):
        for scale in (0.3, 1.0, 4.0):
            x = rng.normal(size=n) * scale
            p = exact.entmax_rows(torch.tensor(x)[None], alpha)[0].numpy()
            best = tsallis_objective(p, x, alpha)
            # no random feasible point does better
            for _ in range(200):
                r = rng.dirichlet(np.ones(n) * rng.choice([0.2, 1.0, 5.0]))
                assert tsallis_objective(r, x, alpha) <= best + 1e-12
            # an independent constrained optimiser lands on the same point
            res = minimize(lambda r: -tsallis_objective(r, x, alpha), np.full(n, 1.0 / n), method="SLSQP",
                           bounds=[(0.0, 1.0)] * n, constraints={"type": "eq", "fun": lambda r: r.sum() - 1.0},
                           options={"ftol": 1e-14, "maxiter": 500})
            assert -res.fun <= best + 1e-9
            assert np.abs(res.x - p).max() < 2e-4


def test_two_element_closed_forms():
    for t in np.linspace(0.0, 3.0, 31):
        x = torch.tensor([[t, 0.0]], dtype=torch.float64)
        # sparsemax: p1 = clip((t + 1) / 2, 0, 1)
        p = exact.entmax_rows(x, 2.0)[0]
        assert abs(p[0].item() - min(1.0, (t + 1.0) / 2.0)) < 1e-12
        # entmax-1.5: with d = t/2, both in the support iff d <= 1 and then sqrt(p1) = (d + sqrt(2 - d^2)) / 2
        d = t / 2.0
        p = exact.entmax_rows(x, 1.5)[0]
        want = ((d + math.sqrt(2.0 - d * d)) / 2.0) ** 2 if d <= 1.0 else 1.0
        assert abs(p[0].item() - want) < 1e-12
        assert abs(p.sum().item() - 1.0) < 1e-12


@pytest.mark.parametrize("alpha", ALPHAS)
def test_constant_row_is_uniform_and_dominant_logit_is_one_hot(alpha):
    for n in (1, 2, 17, 256):
        p = exact.entmax_rows(torch.full((1, n), 0.7, dtype=torch.float64), alpha)[0]
        assert torch.allclose(p, torch.full((n,), 1.0 / n, dtype=torch.float64), atol=1e-12)
    x = torch.zeros(1, 9, dtype=torch.float64)
    x[0, 4] = 1.0 / (alpha - 1.0) + 1e-9  # gap of 1/(alpha-1) pushes every other entry out of the support
    p = exact.entmax_rows(x, alpha)[0]
    assert p[4].item() == pytest.approx(1.0, abs=1e-7) and (p > 0).sum().item() == 1


def test_softmax_limit():
    torch.manual_seed(0)
    x = torch.randn(16, 12, dtype=torch.float64)
    p = exact.entmax_rows(x, 1.0005)
    assert (p - torch.softmax(x, -1)).abs().max().item() < 2e-3


@pytest.mark.parametrize("alpha", ALPHAS)
def test_invariances_and_cross_agreement(alpha):
    torch.manual_seed(1)
    x = torch.randn(32, 100, dtype=torch.float64) * 2.0
    p, tau = exact.entmax_rows(x, alpha, return_tau=True)
    assert (p >= 0).all() and torch.allclose(p.sum(-1), torch.ones(32, dtype=torch.float64), atol=1e-12)
    # shift invariance, permutation equivariance
    assert torch.allclose(exact.entmax_rows(x + 3.25, alpha), p, atol=1e-12)
    perm = torch.randperm(100)
    assert torch.allclose(exact.entmax_rows(x[:, perm], alpha), p[:, perm], atol=1e-12)
    # the three threshold algorithms are independent pieces of code
    tb = exact.bisect_threshold(x * (alpha - 1.0), alpha)
    assert (tau - tb).abs().max().item() < 1e-12
    # support is exactly {z > tau}
    assert ((x * (alpha - 1.0) > tau[:, None]) == (p > 0)).all()


@pytest.mark.parametrize("alpha", [1.5, 2.0])
def test_sort_forms_against_brute_force_support_enumeration(alpha):
    rng = np.random.default_rng(3)
    for _ in range(40):
        n = int(rng.integers(2, 7))
        z = np.sort(rng.normal(size=n) * rng.choice([0.2, 1.0, 3.0]))[::-1].copy()
        found = []
        for k in range(1, n + 1):  # the support of entmax is a prefix of the sorted scores
            top = z[:k]
            if alpha == 2.0:
                tau = (top.sum() - 1.0) / k
            else:
                mean = top.mean()
                disc = (1.0 - ((top - mean) ** 2).sum()) / k
                if disc < 0:
                    continue
                tau = mean - math.sqrt(disc)
            if top[-1] > tau and (k == n or z[k] <= tau):
                found.append(tau)
        assert len(found) == 1
        zz = torch.tensor(z)[None]
        tau = (exact.sparsemax_threshold(zz) if alpha == 2.0 else exact.entmax15_threshold(zz)).item()
        assert abs(tau - found[0]) < 1e-12


@pytest.mark.parametrize("alpha", ALPHAS)
def test_minus_inf_entries_are_ignored(alpha):
    torch.manual_seed(2)
    x = torch.randn(4, 20, dtype=torch.float64)
    xm = x.clone()
    xm[:, 13:] = float("-inf")
    p = exact.entmax_rows(xm, alpha)
    assert (p[:, 13:] == 0).all()
    assert torch.allclose(p[:, :13], exact.entmax_rows(x[:, :13], alpha), atol=1e-12)


# ---- dense attention ---------------------------------------------------------------------------------
@pytest.mark.parametrize("alpha,causal", list(itertools.product(ALPHAS, [False, True])))
def test_dense_attention_matches_row_by_row_loop(alpha, causal):
    torch.manual_seed(4)
    q = torch.randn(2, 4, 24, 8)
    k = torch.randn(2, 2, 24, 8)
    v = torch.randn(2, 2, 24, 8)
    varlen = torch.tensor([24, 13])
    got = exact.dense_entmax_attention(q, k, v, alpha, causal, varlen)
    want = exact.dense_entmax_attention_loop(q, k, v, alpha, causal, varlen)
    assert (got - want).abs().max().item() < 1e-12
    assert (got[1, :, 13:] == 0).all()  # padded rows exactly zero (tests/test_adasplash.py:187-201)


def test_zero_scores_return_the_mean_of_v():
    # tests/test_adasplash.py:173-184
    for n in (64, 128):
        q = torch.zeros(1, 1, n, 64)
        v = torch.randn(1, 1, n, 64, generator=torch.Generator().manual_seed(5))
        out = exact.dense_entmax_attention(q, q.clone(), v, 1.5, False)
        assert torch.allclose(out, v.double().mean(-2, keepdim=True).expand_as(out), atol=1e-12)


def test_gqa_equals_repeat_interleave_and_varlen_equals_slicing():
    # tests/test_adasplash_v2.py:340-342 and :67-78
    torch.manual_seed(6)
    q = torch.randn(2, 8, 32, 16)
    k = torch.randn(2, 2, 32, 16)
    v = torch.randn(2, 2, 32, 16)
    a = exact.dense_entmax_attention(q, k, v, 1.5, True)
    b = exact.dense_entmax_attention(q, k.repeat_interleave(4, 1), v.repeat_interleave(4, 1), 1.5, True)
    assert torch.equal(a, b)
    varlen = torch.tensor([20, 32])
    c = exact.dense_entmax_attention(q, k, v, 1.5, True, varlen)
    for bi in range(2):
        L = int(varlen[bi])
        d = exact.dense_entmax_attention(q[bi:bi + 1, :, :L], k[bi:bi + 1, :, :L], v[bi:bi + 1, :, :L], 1.5, True)
        assert (c[bi:bi + 1, :, :L] - d).abs().max().item() < 1e-12
        assert (c[bi, :, L:] == 0).all()


def test_oracle_reproduces_the_committed_golden_vectors(golden_dir):
    g = np.load(golden_dir / "entmax_rows_128x256.npz")
    x = torch.tensor(g["x"])
    for key, alpha in (("y15", 1.5), ("y20", 2.0), ("y1333", 1.333)):
        assert np.abs(exact.entmax_rows(x, alpha).float().numpy() - g[key]).max() < 1e-7
    g = np.load(golden_dir / "attn_v2_b1h8n128d64.npz")
    out = exact.dense_entmax_attention(*(torch.tensor(g[n]) for n in "qkv"), 1.5, True)
    assert np.abs(out.float().numpy() - g["out"]).max() < 1e-6


@pytest.mark.parametrize(
    "alpha,causal,shape,varlen",
    [
        (1.5, True, (1, 2, 1, 12, 4), None),
        (2.0, False, (1, 1, 1, 10, 4), None),
        (1.333, True, (2, 2, 2, 9, 4), [9, 6]),
    ],
)
def test_closed_form_gradients_match_finite_differences(alpha, causal, shape, varlen):
    # pins dense_entmax_attention_grads (a dropped -delta term, a missing 1/sqrt(D), a transposed dk or a
    # wrong GQA reduction all fail here): central differences of the forward oracle in fp64
    B, Hq, Hkv, N, D = shape
    g = torch.Generator().manual_seed(3)
    q = torch.randn(B, Hq, N, D, generator=g, dtype=torch.float64)
    k = torch.randn(B, Hkv, N, D, generator=g, dtype=torch.float64)
    v = torch.randn(B, Hkv, N, D, generator=g, dtype=torch.float64)
    do = torch.randn(B, Hq, N, D, generator=g, dtype=torch.float64)
    vl = torch.tensor(varlen) if varlen is not None else None
    grads = exact.dense_entmax_attention_grads(q, k, v, do, alpha, causal, vl)

    def loss():
        return (exact.dense_entmax_attention(q, k, v, alpha, causal, vl) * do).sum().item()

    eps = 1e-6
    for t, gr in zip((q, k, v), grads):
        flat, num = t.view(-1), torch.zeros(t.numel(), dtype=torch.float64)
        for i in range(flat.numel()):
            old = flat[i].item()
            flat[i] = old + eps
            fp = loss()
            flat[i] = old - eps
            fm = loss()
            flat[i] = old
            num[i] = (fp - fm) / (2 * eps)
        assert (num.view_as(gr) - gr).abs().max() < 1e-7


# ---- the dense example path with ALiBi, left padding and q_len != k_len (examples/attention.py:8-91) ----------
@pytest.mark.parametrize("alpha", [1.5, 2.0, 1.333])
@pytest.mark.parametrize("causal,padding,nq,varlen", [
    (True, "right", 7, [7, 4]), (False, "left", 7, [5, 7]), (True, "left", 7, [3, 6]), (True, "right", 3, None),
    (False, "right", 1, [7, 2]),
])
def test_general_path_gradients_match_finite_differences(alpha, causal, padding, nq, varlen):
    # pins dense_entmax_attention_general_grads (ALiBi, both padding sides, fewer queries than keys): central
    # differences of the general forward oracle in fp64 along random directions of (q, k, v) -- a wrong term in any of
    # the three gradients shows in every direction -- and, for one case, along every coordinate
    B, H, Nk, D = 2, 2, 7, 3
    g = torch.Generator().manual_seed(17)
    q = torch.randn(B, H, nq, D, generator=g, dtype=torch.float64)
    k = torch.randn(B, H, Nk, D, generator=g, dtype=torch.float64)
    v = torch.randn(B, H, Nk, D, generator=g, dtype=torch.float64)
    do = torch.randn(B, H, nq, D, generator=g, dtype=torch.float64)
    vl = torch.tensor(varlen) if varlen is not None else None
    slopes = torch.tensor([0.3, 0.05], dtype=torch.float64)
    kw = dict(alpha=alpha, is_causal=causal, varlen=vl, padding=padding, alibi_slopes=slopes)
    grads = exact.dense_entmax_attention_general_grads(q, k, v, do, **kw)

    def loss(qq, kk, vv):
        return (exact.dense_entmax_attention_general(qq, kk, vv, **kw) * do).sum().item()

    eps = 1e-6
    every_coordinate = alpha == 1.5 and causal and padding == "left"
    dirs = []
    if every_coordinate:
        for which, t in enumerate((q, k, v)):
            for i in range(t.numel()):
                d = [torch.zeros_like(x) for x in (q, k, v)]
                d[which].view(-1)[i] = 1.0
                dirs.append(d)
    else:
        for which in range(6):  # two directions in each of q, k, v alone, so that no two gradients can trade errors
            d = [torch.zeros_like(x) for x in (q, k, v)]
            d[which % 3] = torch.randn(d[which % 3].shape, generator=g, dtype=torch.float64)
            dirs.append(d)
    for dq_, dk_, dv_ in dirs:
        num = (loss(q + eps * dq_, k + eps * dk_, v + eps * dv_) - loss(q - eps * dq_, k - eps * dk_, v - eps * dv_)) / (2 * eps)
        ana = (grads[0] * dq_).sum().item() + (grads[1] * dk_).sum().item() + (grads[2] * dv_).sum().item()
        assert abs(num - ana) < 1e-7 * max(1.0, abs(ana))


def test_general_path_gradients_reduce_to_the_plain_ones():
    # without ALiBi, right padded, q_len == k_len: the closed form over whole tensors must agree with the loops
    g = torch.Generator().manual_seed(19)
    q, k, v, do = (torch.randn(2, 2, 9, 4, generator=g, dtype=torch.float64) for _ in range(4))
    vl = torch.tensor([9, 5])
    a = exact.dense_entmax_attention_general_grads(q, k, v, do, 1.5, True, vl)
    b = exact.dense_entmax_attention_grads(q, k, v, do, 1.5, True, vl)
    for x, y in zip(a, b):
        assert (x - y).abs().max() < 1e-12



def _rand_qkv(B, H, Nq, Nk, D, seed=0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(B, H, Nq, D, generator=g, dtype=torch.float64), torch.randn(B, H, Nk, D, generator=g, dtype=torch.float64),
            torch.randn(B, H, Nk, D, generator=g, dtype=torch.float64))


def test_general_dense_path_reduces_to_the_plain_oracle():
    q, k, v = _rand_qkv(2, 2, 12, 12, 8)
    vl = torch.tensor([7, 12])
    for alpha in (1.5, 2.0, 1.333):
        for causal in (False, True):
            a = exact.dense_entmax_attention(q, k, v, alpha, causal, varlen=vl)
            b = exact.dense_entmax_attention_general(q, k, v, alpha, causal, varlen=vl)
            assert (a - b).abs().max().item() < 1e-9


def test_alibi_sign_and_row_shift_invariance():
    """A large positive slope must pull a causal row onto its most recent key (out_i -> v_i): a bias of the wrong
    sign, or taken over queries instead of keys, sends it to the first key or changes nothing.  And the bias of a
    row, slope * (j - i), differs from slope * j by a per-row constant, which entmax ignores."""
    q, k, v = _rand_qkv(1, 2, 10, 10, 4, seed=1)
    out = exact.dense_entmax_attention_general(q, k, v, 1.5, True, alibi_slopes=torch.tensor([60.0, 80.0]))
    assert (out - v).abs().max().item() < 1e-9
    slopes = torch.tensor([0.3, 0.05])
    got = exact.dense_entmax_attention_general(q, k, v, 1.5, True, alibi_slopes=slopes)
    # same thing by hand: fold slope * j into the scores through an extra (q, k) feature pair
    D = q.shape[-1]
    j = torch.arange(10, dtype=torch.float64)
    q2 = torch.cat([q, torch.ones(1, 2, 10, 1, dtype=torch.float64)], -1) * math.sqrt((D + 1) / D)
    k2 = torch.cat([k, (slopes[:, None] * j[None, :])[None, :, :, None] * math.sqrt(D)], -1)
    want = exact.dense_entmax_attention(q2, k2, v, 1.5, True)
    assert (got - want).abs().max().item() < 1e-9
    # without a causal mask the bias is not a row shift of anything simpler, but slope 0 must be a no-op
    a = exact.dense_entmax_attention_general(q, k, v, 2.0, False, alibi_slopes=torch.zeros(2))
    assert (a - exact.dense_entmax_attention(q, k, v, 2.0, False)).abs().max().item() < 1e-12


def test_left_padding_is_the_unpadded_problem_at_the_end():
    q, k, v = _rand_qkv(2, 2, 9, 9, 4, seed=2)
    vl = torch.tensor([5, 9])
    for causal in (False, True):
        out = exact.dense_entmax_attention_general(q, k, v, 1.5, causal, varlen=vl, padding="left")
        assert (out[0, :, :4] == 0).all()
        tail = exact.dense_entmax_attention(q[:1, :, 4:], k[:1, :, 4:], v[:1, :, 4:], 1.5, causal)
        assert (out[:1, :, 4:] - tail).abs().max().item() < 1e-9
        full = exact.dense_entmax_attention(q[1:], k[1:], v[1:], 1.5, causal)
        assert (out[1:] - full).abs().max().item() < 1e-9


def test_bottom_right_causal_mask_and_single_query_alibi():
    """q_len < k_len: the queries are the last q_len positions, so the result is the tail of the square problem;
    a single query row takes the ALiBi bias of the last position."""
    q, k, v = _rand_qkv(1, 2, 11, 11, 4, seed=3)
    slopes = torch.tensor([0.2, 0.7])
    square = exact.dense_entmax_attention_general(q, k, v, 1.5, True)
    tail = exact.dense_entmax_attention_general(q[:, :, -3:], k, v, 1.5, True)
    assert (square[:, :, -3:] - tail).abs().max().item() < 1e-9
    sq_alibi = exact.dense_entmax_attention_general(q, k, v, 1.5, True, alibi_slopes=slopes)
    one = exact.dense_entmax_attention_general(q[:, :, -1:], k, v, 1.5, True, alibi_slopes=slopes)
    assert (sq_alibi[:, :, -1:] - one).abs().max().item() < 1e-9
