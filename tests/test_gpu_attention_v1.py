"""GPU parity of the AdaSplash-1 (block-mask) forward -- any alpha in (1, 2], causal or not, varlen --
against the dense CPU oracle."""

import itertools

import numpy as np
import pytest
import torch

import adasplash_amd as A
from adasplash_amd.adasplash_block_mask import tile_sparsity
from oracle import exact
from tests.gpu_util import DEV, max_err, oracle_rows_of_attention, tol_for

pytestmark = pytest.mark.gpu


def run_v1(q, k, v, **kw):
    if kw.get("varlen") is not None:
        kw["varlen"] = kw["varlen"].to(DEV)
    return A.adasplash_v1(q.to(DEV), k.to(DEV), v.to(DEV), **kw)


def test_golden_fixture(golden_dir):
    g = np.load(golden_dir / "attn_v1_alphas.npz")
    q, k, v = (torch.tensor(g[n]) for n in "qkv")
    varlen = torch.tensor(g["varlen"])
    for alpha, causal in itertools.product((1.333, 1.5, 2.0), (False, True)):
        key = f"out_a{str(alpha).replace('.', 'p')}_{'causal' if causal else 'full'}"
        out = run_v1(q, k, v, alpha=alpha, is_causal=causal, varlen=varlen)
        assert max_err(out, torch.tensor(g[key])) < tol_for(torch.float32, alpha)
        # the dispatcher sends these to the same kernel
        out2 = A.adasplash(q.to(DEV), k.to(DEV), v.to(DEV), alpha=alpha, is_causal=causal, varlen=varlen.to(DEV),
                           niter=10 if (alpha != 1.5 or not causal) else 10)
        assert max_err(out2, torch.tensor(g[key])) < tol_for(torch.float32, alpha)


def test_smoke():
    # tests/test_adasplash.py:65-82 (varlen given as an int64 tensor)
    torch.manual_seed(42)
    q, k, v = (torch.randn(1, 1, 128, 32) for _ in range(3))
    varlen = torch.tensor([96])
    out = run_v1(q, k, v, alpha=1.5, varlen=varlen, is_causal=True)
    assert max_err(out, exact.dense_entmax_attention(q, k, v, 1.5, True, varlen)) < 1e-4


@pytest.mark.parametrize("B,H", [(1, 1), (2, 2)])
@pytest.mark.parametrize("N", [128, 256])
@pytest.mark.parametrize("D", [32, 64])
@pytest.mark.parametrize("alpha", [1.333, 1.5, 2.0])
@pytest.mark.parametrize("causal", [False, True])
def test_parameter_sweep(B, H, N, D, alpha, causal):
    # tests/test_adasplash.py:85-114 (random varlen, fp16 and fp32)
    torch.manual_seed(42)
    for dtype in (torch.float32, torch.float16, torch.bfloat16):
        q, k, v = (torch.randn(B, H, N, D).to(dtype) for _ in range(3))
        varlen = torch.randint(1, N + 1, (B,))
        out = run_v1(q, k, v, alpha=alpha, is_causal=causal, varlen=varlen)
        want = exact.dense_entmax_attention(q, k, v, alpha, causal, varlen)
        assert max_err(out, want) < tol_for(dtype, alpha)


def test_zero_scores_give_the_mean_of_v():
    # tests/test_adasplash.py:173-184
    for n in (64, 128):
        q = torch.zeros(1, 1, n, 64)
        out = run_v1(q, q.clone(), torch.ones(1, 1, n, 64), alpha=1.5)
        assert torch.allclose(out.cpu(), torch.ones(1, 1, n, 64), atol=1e-4)


def test_padding_rows_are_exactly_zero():
    # tests/test_adasplash.py:187-201
    torch.manual_seed(0)
    q, k, v = (torch.randn(2, 1, 256, 64) for _ in range(3))
    varlen = torch.tensor([128, 64])
    out = run_v1(q, k, v, varlen=varlen)
    for i in range(2):
        assert (out[i, :, int(varlen[i]):] == 0).all()
    assert max_err(out, exact.dense_entmax_attention(q, k, v, 1.5, False, varlen)) < 1e-4


@pytest.mark.parametrize("seq_len", [512, 1024])
def test_large_inputs_stay_finite(seq_len):
    # tests/test_adasplash.py:149-170
    torch.manual_seed(0)
    q, k, v = ((torch.randn(2, 2, seq_len, 64) * 100).half() for _ in range(3))
    out = run_v1(q, k, v, alpha=1.5)
    assert torch.isfinite(out).all() and out.abs().max().item() < 1e3


def test_high_sparsity_workload_downscaled():
    # the block-mask benchmark workload (q, k x3, alpha = 1.333, niter = 10, non-causal) at N = 2048
    torch.manual_seed(42)
    q, k = ((3 * torch.randn(1, 2, 2048, 64)).to(torch.bfloat16) for _ in range(2))
    v = torch.randn(1, 2, 2048, 64).to(torch.bfloat16)
    out, total, active = tile_sparsity(q.to(DEV), k.to(DEV), v.to(DEV), alpha=1.333, is_causal=False, niter=10)
    want, probs, _, _ = exact.dense_entmax_attention(q, k, v, 1.333, False, return_aux=True)
    assert max_err(out, want) < 2e-2
    assert total == 2 * 128 * 128
    true_active = int((probs > 0).view(1, 2, 128, 16, 128, 16).any(5).any(3).sum())
    assert abs(active - true_active) <= 0.02 * true_active + 2  # ties at the threshold may flip a tile
    assert active < 0.5 * total


def test_full_size_block_mask_workload_sampled_rows():
    g = torch.Generator().manual_seed(42)
    B, H, N, D = 2, 16, 16384, 64
    q = (3 * torch.randn(B, H, N, D, generator=g)).to(torch.bfloat16)
    k = (3 * torch.randn(B, H, N, D, generator=g)).to(torch.bfloat16)
    v = torch.randn(B, H, N, D, generator=g).to(torch.bfloat16)
    out = run_v1(q, k, v, alpha=1.333, is_causal=False, niter=10).cpu()
    assert torch.isfinite(out.float()).all()
    for b, h in ((0, 0), (1, 15)):
        rows = [0, 127, 128, 8191, 16383]
        want = oracle_rows_of_attention(q, k, v, b, h, rows, 1.333, False, N)
        assert max_err(out[b, h, rows], want) < 2e-2


# ---- several solver steps: the steps after a walk run on per-lane candidate lists when those fit -------------


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("alpha", [1.333, 1.5, 2.0])
@pytest.mark.parametrize("D,causal,scale", [(64, False, 3.0), (128, True, 2.0), (32, False, 2.0)])
def test_many_steps_on_peaked_scores(dtype, alpha, D, causal, scale):
    # few scores within 1 of a row's maximum: every block solves on its lists after the first walk
    g = torch.Generator().manual_seed(7)
    B, H, N = 2, 2, 1024
    q = (scale * torch.randn(B, H, N, D, generator=g)).to(dtype)
    k = (scale * torch.randn(B, H, N, D, generator=g)).to(dtype)
    v = torch.randn(B, H, N, D, generator=g).to(dtype)
    varlen = torch.tensor([N, 700])
    out = run_v1(q, k, v, alpha=alpha, is_causal=causal, niter=12, varlen=varlen).cpu()
    want = exact.dense_entmax_attention(q, k, v, alpha, causal, varlen=varlen)
    assert max_err(out, want) < tol_for(dtype, alpha)
    assert (out[1, :, 700:] == 0).all()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("alpha", [1.333, 1.5])
def test_flat_rows_beside_peaked_rows(dtype, alpha):
    # rows whose scores are all equal have as many candidates as keys: their lanes run out of list space and
    # the block keeps walking, with the same result for the peaked rows that share it
    g = torch.Generator().manual_seed(11)
    B, H, N, D = 1, 2, 2048, 64
    q = (3 * torch.randn(B, H, N, D, generator=g)).to(dtype)
    k = (3 * torch.randn(B, H, N, D, generator=g)).to(dtype)
    v = torch.randn(B, H, N, D, generator=g).to(dtype)
    flat = [5, 130, 131, 1000]
    q[:, :, flat] = 0
    out = run_v1(q, k, v, alpha=alpha, is_causal=False, niter=10).cpu()
    want = exact.dense_entmax_attention(q, k, v, alpha, False)
    assert max_err(out, want) < tol_for(dtype, alpha)
    mean_v = v.double().mean(2, keepdim=True)
    assert max_err(out[:, :, flat], mean_v.expand(-1, -1, len(flat), -1)) < tol_for(dtype, alpha)


@pytest.mark.parametrize("n_top", [9, 24, 40, 70, 200])
def test_rows_with_a_wide_top(n_top):
    # n_top keys tie for the maximum of every row: past 8 a lane draws further chunks, past 64 per lane (or when
    # the wave's chunks run out) the block falls back to walking
    g = torch.Generator().manual_seed(13)
    B, H, N, D = 1, 1, 1024, 64
    k = torch.zeros(B, H, N, D)
    k[..., 0] = -4.0
    k[:, :, :n_top, 0] = 4.0
    k[..., 1:] = 0.05 * torch.randn(B, H, N, D - 1, generator=g)
    q = torch.zeros(B, H, N, D)
    q[..., 0] = 8.0
    v = torch.randn(B, H, N, D, generator=g)
    for alpha in (1.5, 1.333):
        out = run_v1(q, k, v, alpha=alpha, is_causal=False, niter=10).cpu()
        want = exact.dense_entmax_attention(q, k, v, alpha, False)
        assert max_err(out, want) < tol_for(torch.float32, alpha)


def test_many_steps_match_between_versions():
    # adasplash_v2 with several steps takes the same list path behind the histogram
    g = torch.Generator().manual_seed(17)
    q = (3 * torch.randn(1, 4, 2048, 128, generator=g)).to(torch.bfloat16)
    k = (3 * torch.randn(1, 2, 2048, 128, generator=g)).to(torch.bfloat16)
    v = torch.randn(1, 2, 2048, 128, generator=g).to(torch.bfloat16)
    out = A.adasplash_v2(q.to(DEV), k.to(DEV), v.to(DEV), niter=4).cpu()
    kk, vv = k.repeat_interleave(2, 1), v.repeat_interleave(2, 1)
    want = exact.dense_entmax_attention(q, kk, vv, 1.5, True)
    assert max_err(out, want) < 2e-2


@pytest.mark.parametrize("alpha", [2.0, 1.5])
def test_one_dominant_key_converges_in_a_few_steps(alpha):
    # tau sits on the lower end of its bracket (row maximum - 1) when one key carries all the mass; at scores of
    # this size the spacing of floats exceeds the solver's eps, and a Newton step that lands exactly on that end
    # must be taken, not bisected towards
    g = torch.Generator().manual_seed(19)
    B, H, N, D = 1, 2, 1024, 64
    q = 3 * torch.randn(B, H, N, D, generator=g)
    k = 3 * torch.randn(B, H, N, D, generator=g)
    v = torch.randn(B, H, N, D, generator=g)
    out = run_v1(q, k, v, alpha=alpha, is_causal=False, niter=5).cpu()
    want = exact.dense_entmax_attention(q, k, v, alpha, False)
    assert max_err(out, want) < 1e-4


def test_many_steps_beyond_the_block_bit_limit():
    # past 128K keys the multi-step kernel keeps only the tile masks (no per-wave block bits); the candidate
    # lists still serve the later steps
    g = torch.Generator().manual_seed(23)
    B, H, N, D = 1, 1, 131072 + 2048, 64
    q = (3 * torch.randn(B, H, N, D, generator=g)).to(torch.bfloat16)
    k = (3 * torch.randn(B, H, N, D, generator=g)).to(torch.bfloat16)
    v = torch.randn(B, H, N, D, generator=g).to(torch.bfloat16)
    out = run_v1(q, k, v, alpha=1.5, is_causal=True, niter=6, varlen=torch.tensor([N])).cpu()
    assert torch.isfinite(out.float()).all()
    rows = [0, 63, 4097, 70000, N - 1]
    want = oracle_rows_of_attention(q, k, v, 0, 0, rows, 1.5, True, N)
    assert max_err(out[0, 0, rows], want) < 2e-2


def test_output_from_lists_matches_output_walk():
    # asking for tile statistics makes the kernel walk for the output; without them it gathers the V rows of the
    # listed keys: the same probabilities either way
    g = torch.Generator().manual_seed(29)
    q, k = ((3 * torch.randn(2, 2, 2048, 64, generator=g)).to(torch.bfloat16).to(DEV) for _ in range(2))
    v = torch.randn(2, 2, 2048, 64, generator=g).to(torch.bfloat16).to(DEV)
    varlen = torch.tensor([2048, 1500]).to(DEV)
    walked, _, _ = tile_sparsity(q, k, v, alpha=1.333, is_causal=False, niter=10, varlen=varlen)
    gathered = A.adasplash_v1(q, k, v, alpha=1.333, is_causal=False, niter=10, varlen=varlen)
    assert max_err(walked.cpu(), gathered.cpu().double()) < 2e-2  # one bf16 step: the walk rounds P to bf16 before its PV product
    want = exact.dense_entmax_attention(q.cpu(), k.cpu(), v.cpu(), 1.333, False, varlen=varlen.cpu())
    assert max_err(gathered.cpu(), want) < 2e-2


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("alpha,causal", [(1.5, False), (1.5, True), (1.333, False), (2.0, True)])
def test_no_block_mask_name_is_served_by_the_same_kernels(dtype, alpha, causal):
    """``adasplash_no_block_mask`` (adasplash/__init__.py:33-36, kernel file adasplash/adasplash_no_block_mask.py)
    computes the same function without the block mask; here the name is served by the block-mask kernels.  Parity
    against the dense oracle with and without variable lengths."""
    torch.manual_seed(3)
    q, k, v = (torch.randn(2, 2, 256, 64).to(dtype) for _ in range(3))  # (a power of two: the call without varlen asks for one)
    tol = tol_for(dtype, alpha)
    out = A.adasplash_no_block_mask(q.to(DEV), k.to(DEV), v.to(DEV), alpha=alpha, is_causal=causal)
    assert out.dtype == dtype
    assert max_err(out, exact.dense_entmax_attention(q, k, v, alpha, causal)) < tol
    varlen = torch.tensor([256, 131], dtype=torch.int32)
    out = A.adasplash_no_block_mask(q.to(DEV), k.to(DEV), v.to(DEV), alpha=alpha, is_causal=causal,
                                    varlen=varlen.to(DEV))
    assert max_err(out, exact.dense_entmax_attention(q, k, v, alpha, causal, varlen)) < tol
    assert (out[1, :, 131:] == 0).all()
