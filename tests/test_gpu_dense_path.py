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
