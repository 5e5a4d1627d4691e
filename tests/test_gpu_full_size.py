"""GPU parity at the benchmark's full sizes and at the reference's longest test shapes.

* The headline workload (c4) and the block-mask workload (c5) through both routes -- the sparse-support kernels and the
  dense kernels alone -- compared over the whole output tensor on the device, with the thresholds and the supports of
  sampled rows held to the oracle.
* The reference's fp32 cases that the smaller files stop short of: forward and backward at N = 4096
  (tests/test_adasplash_v2.py:124-179), the long contexts N = 16384 and 32768 (:182-241), and the backward over the
  GQA ratios Hkv in {1, 2, 4, 8} of Hq = 8 (:353-382).

Tolerances: fp32 1e-4 (the reference's own), 16-bit 2e-2 on the magnitude-aware scale of tests/gpu_util.max_err.
"""

import math
import os

import pytest
import torch

import adasplash_amd as A
from adasplash_amd import _attention
from oracle import exact
from tests.gpu_util import DEV, max_err, oracle_rows_of_attention

pytestmark = pytest.mark.gpu


def _scaled_diff_on_device(a, b):
    a, b = a.float(), b.float()
    return ((a - b).abs() / torch.clamp(b.abs() / 2, min=1.0)).max().item()


def _forward_both_routes(q, k, v, **kw):
    """(out, taus) from the sparse-support kernel (the default) and from the dense kernel alone, on the device."""
    old = os.environ.get("ADSP_SPARSE")
    res = {}
    try:
        for mode in ("1", "0"):
            os.environ["ADSP_SPARSE"] = mode
            out, taus, _ = _attention.launch_forward(q, k, v, **kw)
            torch.cuda.synchronize()
            res[mode] = (out, taus)
    finally:
        if old is None:
            os.environ.pop("ADSP_SPARSE", None)
        else:
            os.environ["ADSP_SPARSE"] = old
    return res["1"], res["0"]


def _oracle_rows(q, k, b, h, rows, alpha, causal, L):
    """Scaled scores z = (alpha - 1) q.k / sqrt(D), exact thresholds and probabilities of a few query rows."""
    g = q.shape[1] // k.shape[1]
    s = q[b, h, rows].double().cpu() @ k[b, h // g, :L].double().cpu().t() / math.sqrt(q.shape[-1])
    if causal:
        s = s.masked_fill(torch.arange(L)[None, :] > torch.as_tensor(rows)[:, None], float("-inf"))
    probs, tau = exact.entmax_rows(s, alpha, return_tau=True)
    return (alpha - 1.0) * s, tau, probs


def test_headline_workload_both_routes_over_the_whole_tensor():
    g = torch.Generator().manual_seed(42)
    B, Hq, Hkv, N, D = 8, 32, 8, 8192, 128
    q = torch.randn(B, Hq, N, D, generator=g).to(torch.bfloat16).to(DEV)
    k = torch.randn(B, Hkv, N, D, generator=g).to(torch.bfloat16).to(DEV)
    v = torch.randn(B, Hkv, N, D, generator=g).to(torch.bfloat16).to(DEV)
    lens = torch.randint(N // 4, N + 1, (B,), generator=g, dtype=torch.int32)
    (out_s, tau_s), (out_d, tau_d) = _forward_both_routes(q, k, v, version=2, alpha=1.5, is_causal=True, niter=10,
                                                          varlen=lens.to(DEV))
    assert torch.isfinite(out_s.float()).all() and torch.isfinite(out_d.float()).all()
    d = _scaled_diff_on_device(out_s, out_d)
    print("c4 forward, sparse against dense route over the whole tensor, magnitude-scaled:", d)
    assert d < 2e-2
    valid = (torch.arange(N)[None, :] < lens[:, None].long())[:, None, :].expand(B, Hq, N).to(DEV)
    dt = (tau_s - tau_d).abs()[valid].max().item()
    print("c4 thresholds, sparse against dense route, all valid rows:", dt)
    assert dt < 1e-3  # (the dense kernel's sums over 16-bit inputs are taken in packed f16: a few 1e-4)
    for b, h in ((0, 0), (3, 17), (5, 9), (7, 31)):
        L = int(lens[b])
        rows = [0, 1, 63, 64, 127, 128, 1000, L // 3, L // 2, L - 130, L - 2, L - 1]
        z, tau, probs = _oracle_rows(q, k, b, h, rows, 1.5, True, L)
        got_tau = tau_s[b, h, rows].double().cpu()
        assert (got_tau - tau).abs().max().item() < 2e-4
        # identical support away from ties: a key is in the support when its scaled score exceeds the threshold
        clear = (z - tau[:, None]).abs() > 1e-3
        assert ((z > got_tau[:, None]) == (probs > 0))[clear].all()
        want = oracle_rows_of_attention(q, k, v, b, h, rows, 1.5, True, L)
        assert max_err(out_s[b, h, rows], want) < 2e-2 and max_err(out_d[b, h, rows], want) < 2e-2


def test_block_mask_workload_both_routes_over_the_whole_tensor():
    g = torch.Generator().manual_seed(42)
    B, H, N, D = 2, 16, 16384, 64
    q = (3 * torch.randn(B, H, N, D, generator=g)).to(torch.bfloat16).to(DEV)
    k = (3 * torch.randn(B, H, N, D, generator=g)).to(torch.bfloat16).to(DEV)
    v = torch.randn(B, H, N, D, generator=g).to(torch.bfloat16).to(DEV)
    (out_s, tau_s), (out_d, tau_d) = _forward_both_routes(q, k, v, version=1, alpha=1.333, is_causal=False, niter=10,
                                                          varlen=None)
    assert torch.isfinite(out_s.float()).all() and torch.isfinite(out_d.float()).all()
    d = _scaled_diff_on_device(out_s, out_d)
    print("c5 forward, sparse against dense route over the whole tensor, magnitude-scaled:", d)
    assert d < 2e-2
    for b, h in ((0, 0), (1, 15)):
        rows = [0, 127, 128, 5000, 8191, 16383]
        z, tau, probs = _oracle_rows(q, k, b, h, rows, 1.333, False, N)
        got_tau = tau_s[b, h, rows].double().cpu()
        assert (got_tau - tau).abs().max().item() < 5e-4
        clear = (z - tau[:, None]).abs() > 2e-3
        assert ((z > got_tau[:, None]) == (probs > 0))[clear].all()
        want = oracle_rows_of_attention(q, k, v, b, h, rows, 1.333, False, N)
        assert max_err(out_s[b, h, rows], want) < 2e-2 and max_err(out_d[b, h, rows], want) < 2e-2


def test_fp32_forward_and_backward_at_4096():
    """tests/test_adasplash_v2.py:124-179 at its longest length: B=2, H=2, D=64, fp32, seed 42, niter=10, 1e-4."""
    g = torch.Generator().manual_seed(42)
    q, k, v, do = (torch.randn(2, 2, 4096, 64, generator=g) for _ in range(4))
    qg, kg, vg = (t.to(DEV).requires_grad_(True) for t in (q, k, v))
    out = A.adasplash_v2(qg, kg, vg, niter=10)
    out.backward(do.to(DEV))
    want = exact.dense_entmax_attention(q, k, v, 1.5, True)
    assert (out.detach().double().cpu() - want).abs().max().item() < 1e-4
    for name, got, w in zip(("dq", "dk", "dv"), (qg.grad, kg.grad, vg.grad),
                            exact.dense_entmax_attention_grads(q, k, v, do, 1.5, True)):
        assert (got.double().cpu() - w).abs().max().item() < 1e-4, name


@pytest.mark.parametrize("n_kv,seq_len", [(1, 1024), (2, 1024), (4, 1024), (8, 1024), (2, 2048), (4, 2048)])
def test_fp32_gqa_backward_matrix(n_kv, seq_len):
    """tests/test_adasplash_v2.py:353-382: Hq = 8 over every K/V head count, dk and dv summed over each group."""
    g = torch.Generator().manual_seed(42)
    B, Hq, D = 2, 8, 64
    q = torch.randn(B, Hq, seq_len, D, generator=g)
    k = torch.randn(B, n_kv, seq_len, D, generator=g)
    v = torch.randn(B, n_kv, seq_len, D, generator=g)
    do = torch.randn(B, Hq, seq_len, D, generator=g)
    qg, kg, vg = (t.to(DEV).requires_grad_(True) for t in (q, k, v))
    A.adasplash_v2(qg, kg, vg, niter=10).backward(do.to(DEV))
    for name, got, w in zip(("dq", "dk", "dv"), (qg.grad, kg.grad, vg.grad),
                            exact.dense_entmax_attention_grads(q, k, v, do, 1.5, True)):
        assert got.shape == w.shape
        assert (got.double().cpu() - w).abs().max().item() < 1e-4, name


@pytest.mark.parametrize("seq_len", [16384, 32768])
def test_fp32_long_context_forward_and_backward(seq_len):
    """tests/test_adasplash_v2.py:182-241 (B=1, H=1, D=64, fp32, seed 42, niter=10, 1e-4).  The dense oracle over all
    rows would need the whole score matrix in fp64; the output is held to it on 96 sampled rows, and the gradients with
    an upstream gradient that is non-zero on those rows only, for which dq (on the rows), dk and dv (everywhere) follow
    from the sampled rows' probabilities alone."""
    g = torch.Generator().manual_seed(42)
    N, D = seq_len, 64
    q, k, v = (torch.randn(1, 1, N, D, generator=g) for _ in range(3))
    rows = sorted(set([0, 1, 63, 64, 127, 128, 129, N // 2, N - 2, N - 1] + torch.randint(0, N, (86,), generator=g).tolist()))
    do = torch.zeros(1, 1, N, D)
    do[0, 0, rows] = torch.randn(len(rows), D, generator=g)
    qg, kg, vg = (t.to(DEV).requires_grad_(True) for t in (q, k, v))
    out = A.adasplash_v2(qg, kg, vg, niter=10)
    out.backward(do.to(DEV))
    z, tau, probs = _oracle_rows(q, k, 0, 0, rows, 1.5, True, N)
    kd, vd, dod, qd = k[0, 0].double(), v[0, 0].double(), do[0, 0, rows].double(), q[0, 0, rows].double()
    assert (out[0, 0, rows].detach().double().cpu() - probs @ vd).abs().max().item() < 1e-4
    u = probs.sqrt()
    dp = dod @ vd.t()
    dx = u * (dp - (u * dp).sum(-1, keepdim=True) / u.sum(-1, keepdim=True))
    sm = 1.0 / math.sqrt(D)
    assert (qg.grad[0, 0, rows].double().cpu() - dx @ kd * sm).abs().max().item() < 1e-4
    rest = torch.ones(N, dtype=torch.bool)
    rest[rows] = False
    assert (qg.grad[0, 0][rest.to(DEV)] == 0).all()  # rows without an upstream gradient
    assert (kg.grad[0, 0].double().cpu() - dx.t() @ qd * sm).abs().max().item() < 1e-4
    assert (vg.grad[0, 0].double().cpu() - probs.t() @ dod).abs().max().item() < 1e-4


def test_bf16_longest_context_backward_on_the_supports():
    """N = 65536, the longest sequence the sparse-support kernels take (16-bit key indices; the dK/dV kernel's table of
    pieces is filled more than once per key block here), D = 64, bf16, causal: forward and backward with an upstream
    gradient that is non-zero on 96 sampled rows only, so that dq on those rows and dk, dv everywhere follow from the
    sampled rows' probabilities alone (as in the fp32 long-context test above).  2e-2 / 4e-2 on the magnitude-aware scale."""
    g = torch.Generator().manual_seed(5)
    N, D = 65536, 64
    q, k, v = (torch.randn(1, 1, N, D, generator=g).to(torch.bfloat16) for _ in range(3))
    rows = sorted(set([0, 1, 127, 128, N // 2, N - 129, N - 2, N - 1] + torch.randint(0, N, (88,), generator=g).tolist()))
    do = torch.zeros(1, 1, N, D, dtype=torch.bfloat16)
    do[0, 0, rows] = torch.randn(len(rows), D, generator=g).to(torch.bfloat16)
    qg, kg, vg = (t.to(DEV).requires_grad_(True) for t in (q, k, v))
    out = A.adasplash_v2(qg, kg, vg, niter=1)
    out.backward(do.to(DEV))
    z, tau, probs = _oracle_rows(q, k, 0, 0, rows, 1.5, True, N)
    kd, vd, dod, qd = k[0, 0].double(), v[0, 0].double(), do[0, 0, rows].double(), q[0, 0, rows].double()
    assert max_err(out[0, 0, rows].detach(), probs @ vd) < 2e-2
    u = probs.sqrt()
    dp = dod @ vd.t()
    dx = u * (dp - (u * dp).sum(-1, keepdim=True) / u.sum(-1, keepdim=True))
    sm = 1.0 / math.sqrt(D)
    assert max_err(qg.grad[0, 0, rows], dx @ kd * sm) < 4e-2
    rest = torch.ones(N, dtype=torch.bool)
    rest[rows] = False
    assert (qg.grad[0, 0][rest.to(DEV)] == 0).all()  # rows without an upstream gradient
    assert max_err(kg.grad[0, 0], dx.t() @ qd * sm) < 4e-2
    assert max_err(vg.grad[0, 0], probs.t() @ dod) < 4e-2


def test_headline_workload_is_bit_reproducible():
    """Forward and backward of the headline shapes, three times on the same inputs: the same bits every time (which
    kernel serves a row block is decided by the inputs alone, and no sum depends on the order in which workgroups run)."""
    g = torch.Generator().manual_seed(42)
    B, Hq, Hkv, N, D = 8, 32, 8, 8192, 128
    q = torch.randn(B, Hq, N, D, generator=g).to(torch.bfloat16).to(DEV)
    k = torch.randn(B, Hkv, N, D, generator=g).to(torch.bfloat16).to(DEV)
    v = torch.randn(B, Hkv, N, D, generator=g).to(torch.bfloat16).to(DEV)
    do = torch.randn(B, Hq, N, D, generator=g).to(torch.bfloat16).to(DEV)
    lens = torch.randint(N // 4, N + 1, (B,), generator=g, dtype=torch.int32).to(DEV)
    runs = []
    for _ in range(3):
        qg, kg, vg = (t.clone().requires_grad_(True) for t in (q, k, v))
        out = A.adasplash_v2(qg, kg, vg, niter=1, varlen=lens)
        out.backward(do)
        torch.cuda.synchronize()
        runs.append((out.detach(), qg.grad, kg.grad, vg.grad))
        del qg, kg, vg, out
    for other in runs[1:]:
        for name, a, b in zip(("out", "dq", "dk", "dv"), other, runs[0]):
            assert torch.equal(a, b), name
