"""GPU test of the entry point that allocates nothing: adsp_attn_v2_fwd_noalloc takes its scratch memory from a device
array inside the library.  Its results are held against adsp_attn_v2_fwd's on the same inputs, on two calls in a row
(the second one smaller, so it finds the first call's leftovers in the shared scratch), through the C ABI."""

import pytest
import torch

from adasplash_amd import _lib
from oracle import exact
from tests.gpu_util import DEV, max_err

pytestmark = pytest.mark.gpu


def _call(entry, q, k, v, varlen, niter=1):
    lib = _lib.load()
    B, Hq, N, D = q.shape
    Hkv = k.shape[1]
    dt = _lib.dtype_code(q)
    out = torch.full_like(q, float("nan"))
    taus = torch.zeros((B, Hq, N), device=q.device, dtype=torch.float32)
    bmask = torch.zeros((B, Hq, lib.adsp_attn_bmask_words(N)), device=q.device, dtype=torch.int32)
    bits = 0 if varlen is None else 32
    stream = torch.cuda.current_stream().cuda_stream
    if entry == "noalloc":
        st = lib.adsp_attn_v2_fwd_noalloc(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), taus.data_ptr(),
                                          bmask.data_ptr(), _lib.ptr(varlen), bits, B, Hq, Hkv, N, D, dt, niter, stream)
    else:
        n = lib.adsp_attn_workspace_bytes(B, Hq, Hkv, N, D, dt)
        ws = torch.empty((max(n, 16),), device=q.device, dtype=torch.uint8)
        st = lib.adsp_attn_v2_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), taus.data_ptr(),
                                  bmask.data_ptr(), _lib.ptr(varlen), bits, B, Hq, Hkv, N, D, dt, niter,
                                  ws.data_ptr() if n else None, n, stream)
    torch.cuda.synchronize()
    return st, out, taus, bmask


def _inputs(B, Hq, Hkv, N, D, dtype, seed, lens=None, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    q = (scale * torch.randn(B, Hq, N, D, generator=g)).to(dtype)
    k = torch.randn(B, Hkv, N, D, generator=g).to(dtype)
    v = torch.randn(B, Hkv, N, D, generator=g).to(dtype)
    varlen = None if lens is None else torch.tensor(lens, dtype=torch.int32)
    return q, k, v, varlen


@pytest.mark.parametrize("dtype,tol", [(torch.bfloat16, 2e-2), (torch.float16, 2e-2), (torch.float32, 1e-4)])
def test_two_calls_in_a_row_match_the_entry_point_with_a_workspace(dtype, tol):
    # first a larger problem (sparse-support kernel and, for the flat batch item, the dense one), then a smaller one
    for case, (B, Hq, Hkv, N, D, lens, niter) in enumerate([(2, 4, 2, 2048, 128, [2048, 1500], 1),
                                                             (1, 2, 2, 320, 64, [300], 10)]):
        q, k, v, varlen = _inputs(B, Hq, Hkv, N, D, dtype, seed=case)
        if case == 0:
            q[1] *= 0.1  # a flat item: its heads go to the dense kernel
        dev = [t.to(DEV) if t is not None else None for t in (q, k, v, varlen)]
        st_a, out_a, tau_a, bm_a = _call("noalloc", *dev, niter=niter)
        st_b, out_b, tau_b, bm_b = _call("workspace", *dev, niter=niter)
        assert st_a == 0 and st_b == 0
        assert max_err(out_a, out_b.float().cpu()) < tol
        assert torch.equal(bm_a, bm_b)
        L = torch.tensor(lens)
        valid = (torch.arange(N)[None, :] < L[:, None])[:, None, :].expand(B, Hq, N)
        assert (tau_a.cpu() - tau_b.cpu())[valid].abs().max().item() < 1e-5
        want = exact.dense_entmax_attention(q, k, v, 1.5, True, varlen)
        assert max_err(out_a, want) < tol


def test_sizes_beyond_the_scratch_are_rejected():
    lib = _lib.load()
    cap = lib.adsp_attn_v2_fwd_noalloc_max_bytes()
    assert cap == 64 << 20
    B, Hq, Hkv, N, D = 8, 32, 8, 8192, 128
    assert lib.adsp_attn_workspace_bytes(B, Hq, Hkv, N, D, _lib.ADSP_BF16) > cap
    # rejected before any pointer is looked at
    st = lib.adsp_attn_v2_fwd_noalloc(16, 16, 16, 16, None, None, None, 0, B, Hq, Hkv, N, D, _lib.ADSP_BF16, 1, None)
    assert st == 8 and b"scratch" in lib.adsp_status_string(st)
