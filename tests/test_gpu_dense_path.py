"""The dense example path (ALiBi, left padding, q_len != k_len) on the GPU against the loop oracle.

Mirrors what ``examples/attention.py:34-91`` offers beyond the fused kernels; the entmax of every score row is
the HIP rows kernel, the two products are library GEMMs.  Tolerance: 1e-4 in fp32 (the rows kernel's bar),
2e-2 in bf16.
"""
import pytest
import torch

from adasplash_amd import dense
from oracle import exact
from tests.gpu_util import DEV

pytestmark = pytest.mark.gpu


def _qkv(B, H, Nq, Nk, D, dtype, seed=42):
    g = torch.Generator().manual_seed(seed)
    return tuple(torch.randn(B, H, n, D, generator=g).to(dtype) for n in (Nq, Nk, Nk))


def _check(q, k, v, tol, **kw):
    got = dense.slow_entmax_attention(q.to(DEV), k.to(DEV), v.to(DEV), niter=10, **{
        key: (val.to(DEV) if torch.is_tensor(val) else val) for key, val in kw.items()})
    want = exact.dense_entmax_attention_general(q, k, v, kw.get("alpha", 1.5), kw.get("is_causal", False),
                                                varlen=kw.get("varlen"), padding=kw.get("padding", "right"),
                                                alibi_slopes=kw.get("alibi_slopes"))
    assert got.shape == q.shape and got.dtype == q.dtype
    assert (got.double().cpu() - want).abs().max().item() < tol


@pytest.mark.parametrize("alpha", [1.333, 1.5, 2.0])
@pytest.mark.parametrize("is_causal", [False, True])
def test_alibi_slopes(alpha, is_causal):
    q, k, v = _qkv(2, 4, 48, 48, 16, torch.float32)
    slopes = torch.tensor([2.0 ** -(i + 1) for i in range(4)])
    _check(q, k, v, 1e-4, alpha=alpha, is_causal=is_causal, alibi_slopes=slopes)


@pytest.mark.parametrize("padding", ["right", "left"])
@pytest.mark.parametrize("is_causal", [False, True])
def test_padding_sides(padding, is_causal):
    q, k, v = _qkv(3, 2, 40, 40, 16, torch.float32)
    varlen = torch.tensor([40, 17, 1])
    _check(q, k, v, 1e-4, is_causal=is_causal, varlen=varlen, padding=padding,
           alibi_slopes=torch.tensor([0.25, 0.0625]))
    got = dense.slow_entmax_attention(q.to(DEV), k.to(DEV), v.to(DEV), varlen=varlen.to(DEV), padding=padding)
    dead = slice(17, None) if padding == "right" else slice(0, 40 - 17)
    assert (got[1, :, dead] == 0).all()


@pytest.mark.parametrize("q_len", [1, 5])
def test_fewer_queries_than_keys_bottom_right_causal(q_len):
    q, k, v = _qkv(2, 2, q_len, 33, 16, torch.float32)
    _check(q, k, v, 1e-4, is_causal=True, alibi_slopes=torch.tensor([0.5, 0.1]))
    _check(q, k, v, 1e-4, is_causal=True, varlen=torch.tensor([33, 20]), padding="left")


def test_bf16_inputs():
    """16-bit inputs: the score matrix is formed in fp32, the probabilities are rounded to the input type for the
    second product; 2e-2 max-abs as for the fused kernels."""
    q, k, v = _qkv(1, 2, 64, 64, 32, torch.bfloat16)
    _check(q, k, v, 2e-2, is_causal=True, alibi_slopes=torch.tensor([0.25, 0.03125]))
    _check(q, k, v, 2e-2, is_causal=False)


@pytest.mark.parametrize("padding", ["left", "right"])
@pytest.mark.parametrize("is_causal", [False, True])
def test_gradients_with_alibi_and_padding(padding, is_causal):
    """dq, dk, dv through autograd with ALiBi slopes and a padded sequence, the reference's own case
    (tests/test_attention.py:50-77,103-107: B=1, H=2, N=64, D=32, fp32, varlen 48, slopes 0.1 / 0.2, niter=10; its
    bars: 1e-4 forward, 1e-3 gradients) against the loop oracle's gradients."""
    g = torch.Generator().manual_seed(42)
    q, k, v, do = (torch.randn(1, 2, 64, 32, generator=g) for _ in range(4))
    varlen = torch.tensor([48], dtype=torch.int32)
    alibi = torch.tensor([0.1, 0.2])
    qg, kg, vg = (t.to(DEV).requires_grad_(True) for t in (q, k, v))
    out = dense.slow_entmax_attention(qg, kg, vg, varlen=varlen.to(DEV), is_causal=is_causal, padding=padding, niter=10,
                                      alibi_slopes=alibi.to(DEV))
    dq, dk, dv = torch.autograd.grad(out, (qg, kg, vg), do.to(DEV))
    want = exact.dense_entmax_attention_general(q, k, v, 1.5, is_causal, varlen=varlen, padding=padding, alibi_slopes=alibi)
    wq, wk, wv = exact.dense_entmax_attention_general_grads(q, k, v, do, 1.5, is_causal, varlen=varlen, padding=padding,
                                                            alibi_slopes=alibi)
    assert (out.double().cpu() - want).abs().max().item() < 1e-4
    for name, got, w in (("dq", dq, wq), ("dk", dk, wk), ("dv", dv, wv)):
        assert (got.double().cpu() - w).abs().max().item() < 1e-3, name
    dead = slice(48, None) if padding == "right" else slice(0, 16)
    assert (dq[0, :, dead] == 0).all() and (dk[0, :, dead] == 0).all() and (dv[0, :, dead] == 0).all()


def test_gradients_with_fewer_queries_than_keys():
    g = torch.Generator().manual_seed(7)
    q = torch.randn(2, 2, 5, 16, generator=g)
    k, v = (torch.randn(2, 2, 33, 16, generator=g) for _ in range(2))
    do = torch.randn(2, 2, 5, 16, generator=g)
    slopes = torch.tensor([0.5, 0.1])
    qg, kg, vg = (t.to(DEV).requires_grad_(True) for t in (q, k, v))
    out = dense.slow_entmax_attention(qg, kg, vg, is_causal=True, niter=10, alibi_slopes=slopes.to(DEV))
    got = torch.autograd.grad(out, (qg, kg, vg), do.to(DEV))
    want = exact.dense_entmax_attention_general_grads(q, k, v, do, 1.5, True, alibi_slopes=slopes)
    for name, a, w in zip(("dq", "dk", "dv"), got, want):
        assert (a.double().cpu() - w).abs().max().item() < 1e-3, name


def test_argument_errors():
    q, k, v = (t.to(DEV) for t in _qkv(2, 2, 8, 8, 16, torch.float32))
    with pytest.raises(ValueError):
        dense.slow_entmax_attention(q[0], k, v)
    with pytest.raises(ValueError):
        dense.slow_entmax_attention(q, k, v[:, :, :4])
    with pytest.raises(ValueError):
        dense.slow_entmax_attention(q, k, v, alibi_slopes=torch.ones(3, device=DEV))
    with pytest.raises(ValueError):
        dense.slow_entmax_attention(q, k, v, varlen=torch.tensor([8, 8, 8], device=DEV))
    with pytest.raises(ValueError):
        dense.slow_entmax_attention(q, k, v, varlen=torch.tensor([8, 4], device=DEV), padding="middle")


def test_flash_name_routes_to_the_fused_kernels():
    q, k, v = (t.to(DEV) for t in _qkv(1, 2, 128, 128, 64, torch.float32))
    a = dense.flash_entmax_attention(q, k, v, niter=10)  # the default single step is good to ~1e-3 only
    b = dense.slow_entmax_attention(q, k, v, is_causal=True, niter=10)
    assert (a - b).abs().max().item() < 3e-4  # each side is within 1e-4 of the exact result
