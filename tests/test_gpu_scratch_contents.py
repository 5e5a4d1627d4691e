"""GPU test: what the caller's scratch buffers hold before a call (the workspaces, the backward's delta and 1 / sum p
arrays, the outputs) must not matter.  Every buffer is filled with NaN bit patterns, with 0xff bytes or with zeros before
the call through the C ABI; both routes must return the same bits each time (which kernel serves a row block is
decided by the inputs alone, and a wave builds its lists in the order of its own candidate stream)."""

import os

import pytest
import torch

from adasplash_amd import _lib
from tests.gpu_util import DEV

pytestmark = pytest.mark.gpu


def _filled(shape, dtype, fill):
    t = torch.zeros(shape, device=DEV, dtype=dtype)
    if fill == "nan":
        t.fill_(0xff) if dtype == torch.uint8 else t.fill_(float("nan"))
    elif fill == "ones":
        t.fill_(0x3c) if dtype == torch.uint8 else t.fill_(1.0)
    return t


def _run(lib, q, k, v, dout, vl, fill):
    B, Hq, N, D = q.shape
    Hkv = k.shape[1]
    dt = _lib.dtype_code(q)
    stream = _lib.current_stream(q.device)
    out = _filled(q.shape, q.dtype, fill)
    taus = _filled((B, Hq, N), torch.float32, fill)
    bmask = torch.zeros((B, Hq, lib.adsp_attn_bmask_words(N)), device=DEV, dtype=torch.int32)
    nws = lib.adsp_attn_workspace_bytes(B, Hq, Hkv, N, D, dt)
    ws = _filled((max(nws, 16),), torch.uint8, fill)
    st = lib.adsp_attn_v2_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), taus.data_ptr(), bmask.data_ptr(),
                              _lib.ptr(vl), 32, B, Hq, Hkv, N, D, dt, 2, ws.data_ptr() if nws else None, nws, stream)
    assert st == 0
    dq, dk, dv = (_filled(t.shape, t.dtype, fill) for t in (q, k, v))
    delta = _filled((B, Hq, N), torch.float32, fill)
    zinv = _filled((B, Hq, N), torch.float32, fill)
    nbw = lib.adsp_attn_bwd_workspace_bytes(B, Hq, Hkv, N, D, dt)
    bws = _filled((max(nbw, 16),), torch.uint8, fill)
    st = lib.adsp_attn_bwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), dout.data_ptr(), taus.data_ptr(), bmask.data_ptr(),
                           _lib.ptr(vl), 32, dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), delta.data_ptr(), zinv.data_ptr(),
                           B, Hq, Hkv, N, D, dt, 1.5, 1, bws.data_ptr() if nbw else None, nbw, stream)
    assert st == 0
    torch.cuda.synchronize()
    return out, dq, dk, dv


@pytest.mark.parametrize("sparse", ["1", "0"])
@pytest.mark.parametrize("B,Hq,Hkv,N,D,lens", [
    (2, 4, 2, 512, 128, [512, 300]),
    (1, 4, 4, 1024, 64, [1000]),
    (2, 2, 1, 256, 32, [256, 77]),
])
def test_results_do_not_depend_on_what_the_buffers_held(sparse, B, Hq, Hkv, N, D, lens):
    old = os.environ.get("ADSP_SPARSE")
    os.environ["ADSP_SPARSE"] = sparse
    try:
        lib = _lib.load()
        g = torch.Generator().manual_seed(N + D)
        q = torch.randn(B, Hq, N, D, generator=g).bfloat16().to(DEV)
        k = torch.randn(B, Hkv, N, D, generator=g).bfloat16().to(DEV)
        v = torch.randn(B, Hkv, N, D, generator=g).bfloat16().to(DEV)
        dout = torch.randn(B, Hq, N, D, generator=g).bfloat16().to(DEV)
        vl = torch.tensor(lens, dtype=torch.int32).to(DEV)
        base = _run(lib, q, k, v, dout, vl, "zero")
        for fill in ("nan", "ones"):
            got = _run(lib, q, k, v, dout, vl, fill)
            for name, a, b in zip(("out", "dq", "dk", "dv"), got, base):
                for bi, l in enumerate(lens):  # (rows past the length: out, dq, dk, dv are zeros there on every path)
                    x, y = a[bi].float(), b[bi].float()
                    assert not torch.isnan(x).any(), f"{name}: NaN with buffers pre-filled with {fill}"
                    assert torch.equal(x, y), f"{name} depends on the buffers' contents ({fill})"
    finally:
        if old is None:
            os.environ.pop("ADSP_SPARSE", None)
        else:
            os.environ["ADSP_SPARSE"] = old


@pytest.mark.parametrize("scale", [1.0, 0.6])
def test_identical_calls_return_identical_bits(scale):
    """Forward and backward through the autograd functions, four times on the same inputs: peaked scores (every row block
    on the sparse-support kernels) and flatter ones (row blocks of both kinds in one launch) return the same bits."""
    import adasplash_amd as A

    g = torch.Generator().manual_seed(5)
    B, Hq, Hkv, N, D = 2, 8, 2, 2048, 128
    q = (scale * torch.randn(B, Hq, N, D, generator=g)).bfloat16().to(DEV)
    k = torch.randn(B, Hkv, N, D, generator=g).bfloat16().to(DEV)
    v = torch.randn(B, Hkv, N, D, generator=g).bfloat16().to(DEV)
    dout = torch.randn(B, Hq, N, D, generator=g).bfloat16().to(DEV)
    vl = torch.tensor([2048, 1500], dtype=torch.int32).to(DEV)
    runs = []
    for _ in range(4):
        qg, kg, vg = (t.clone().requires_grad_(True) for t in (q, k, v))
        out = A.adasplash_v2(qg, kg, vg, niter=1, varlen=vl)
        out.backward(dout)
        torch.cuda.synchronize()
        runs.append((out.detach(), qg.grad, kg.grad, vg.grad))
    for other in runs[1:]:
        for name, a, b in zip(("out", "dq", "dk", "dv"), other, runs[0]):
            assert torch.equal(a, b), name
