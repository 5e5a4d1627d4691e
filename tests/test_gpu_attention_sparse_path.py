"""GPU parity of the sparse-support forward (16-bit inputs, alpha in [1.125, 2], head dims 64 and 128) and of its hand-over
to the dense kernel: the same calls with the sparse-support kernel switched off (ADSP_SPARSE=0 in the environment,
read by the library on every call) must give the oracle's answer too, and the two must agree with each other."""

import os

import pytest
import torch

import adasplash_amd as A
from adasplash_amd import _attention
from oracle import exact
from tests.gpu_util import DEV, max_err, oracle_rows_of_attention

pytestmark = pytest.mark.gpu


@pytest.fixture
def sparse_switch():
    """Returns a function that sets the library's switch; the environment is restored afterwards."""
    old = os.environ.get("ADSP_SPARSE")

    def switch(on):
        os.environ["ADSP_SPARSE"] = "1" if on else "0"

    yield switch
    if old is None:
        os.environ.pop("ADSP_SPARSE", None)
    else:
        os.environ["ADSP_SPARSE"] = old


def forward(q, k, v, varlen=None, version=2, alpha=1.5, causal=True, niter=10):
    return _attention.launch_forward(q.to(DEV), k.to(DEV), v.to(DEV), version=version, alpha=alpha, is_causal=causal,
                                     niter=niter, varlen=None if varlen is None else varlen.to(DEV))


def qkv(B, Hq, Hkv, N, D, dtype, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    q = (scale * torch.randn(B, Hq, N, D, generator=g)).to(dtype)
    k = torch.randn(B, Hkv, N, D, generator=g).to(dtype)
    v = torch.randn(B, Hkv, N, D, generator=g).to(dtype)
    return q, k, v


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,Hq,Hkv,N,D,lens", [
    (1, 2, 2, 128, 64, None),
    (2, 4, 2, 512, 128, [512, 300]),
    (1, 4, 1, 2048, 128, [1999]),
    (2, 2, 2, 200, 64, [137, 200]),
    (1, 2, 1, 4096, 64, None),
    (3, 4, 4, 2304, 128, [2304, 65, 2100]),
])
def test_both_paths_match_the_oracle_and_each_other(sparse_switch, dtype, B, Hq, Hkv, N, D, lens):
    q, k, v = qkv(B, Hq, Hkv, N, D, dtype, seed=N + D)
    varlen = None if lens is None else torch.tensor(lens, dtype=torch.int32)
    want, probs, tau, _ = exact.dense_entmax_attention(q, k, v, 1.5, True, varlen, return_aux=True)
    sparse_switch(True)
    out_s, tau_s, bm_s = forward(q, k, v, varlen)
    sparse_switch(False)
    out_d, tau_d, bm_d = forward(q, k, v, varlen)
    assert max_err(out_s, want) < 2e-2 and max_err(out_d, want) < 2e-2
    assert max_err(out_s, out_d.float().cpu()) < 2e-2
    # thresholds of the valid rows: both paths converge (the list path always does, in fp32; the dense one ran ten
    # steps, whose sums over 16-bit inputs are taken in packed f16: a few 1e-4)
    valid = torch.ones(B, N, dtype=torch.bool) if lens is None else torch.arange(N)[None, :] < varlen[:, None].long()
    valid = valid[:, None, :].expand(B, Hq, N)
    assert (tau_s.double().cpu() - tau)[valid].abs().max().item() < 2e-4
    assert (tau_d.double().cpu() - tau)[valid].abs().max().item() < 1e-3
    # the tile mask covers every non-zero probability on both paths
    nm, nk = (N + 127) // 128, (N + 63) // 64
    pad_r, pad_k = nm * 128 - N, nk * 64 - N
    live = (probs > 0) & valid[..., None]  # rows past a sequence's length are outside the domain
    act = torch.nn.functional.pad(live, (0, pad_k, 0, pad_r)).view(B, Hq, nm, 128, nk, 64).any(5).any(3)
    for bm in (bm_s, bm_d):
        words = bm.cpu().view(B, Hq, nm, -1)
        bits = torch.stack([(words[..., c // 32] >> (c % 32)) & 1 for c in range(nk)], dim=-1).bool()
        assert (bits | ~act).all()


def test_flat_scores_are_left_to_the_dense_kernel(sparse_switch):
    """q / 8: supports of hundreds of keys.  The sparse-support kernel must give every row block up (N = 1024: in its
    walks; N = 4096: the probe marks the heads before it starts), so the result is the dense kernel's: the same bits
    on two calls, and within a solver step's effect of the dense kernel serving the call alone (which takes the
    reference's extra update)."""
    for n in (1024, 4096):
        q, k, v = qkv(1, 4, 4, n, 64, torch.bfloat16, seed=3, scale=0.125)
        sparse_switch(True)
        out_s = forward(q, k, v, niter=1)[0]
        assert torch.equal(out_s, forward(q, k, v, niter=1)[0])
        sparse_switch(False)
        out_d = forward(q, k, v, niter=1)[0]
        assert max_err(out_s, out_d.float().cpu()) < 2e-2
        rows = [0, 77, n // 2, n - 1]
        assert max_err(out_s[0, 1, rows].cpu(), oracle_rows_of_attention(q, k, v, 0, 1, rows, 1.5, True, n)) < 2e-2


@pytest.mark.parametrize("scale", [0.3, 0.5])
def test_supports_that_outgrow_the_lists_fall_back_row_block_by_row_block(sparse_switch, scale):
    """Scores between flat and peaked: a hundred or more candidates per row.  Short row blocks still fit the lists,
    long ones overflow them while the second walk is under way and are redone by the dense kernel."""
    q, k, v = qkv(1, 2, 1, 1536, 128, torch.bfloat16, seed=11, scale=scale)
    varlen = torch.tensor([1500], dtype=torch.int32)
    want = exact.dense_entmax_attention(q, k, v, 1.5, True, varlen)
    sparse_switch(True)
    assert max_err(forward(q, k, v, varlen)[0], want) < 2e-2


def test_heads_of_one_batch_can_go_different_ways(sparse_switch):
    """One flat and one peaked sequence in a batch, long enough for the probe (N >= 2048)."""
    q, k, v = qkv(2, 2, 2, 2048, 64, torch.float16, seed=5)
    q[0] *= 0.1
    want = exact.dense_entmax_attention(q, k, v, 1.5, True)
    sparse_switch(True)
    assert max_err(forward(q, k, v)[0], want) < 2e-2


@pytest.mark.parametrize("dtype,qscale,kscale", [
    (torch.bfloat16, 600.0, 1.0),     # q beyond the one-byte format's largest value: saturated in the first walk
    (torch.bfloat16, 1.0, 1000.0),    # the same for the copy of K
    (torch.bfloat16, 30.0, 1.0 / 512),  # k below the format's smallest value: the copy of K is all zeros
    (torch.float16, 1.0 / 300, 40.0),   # q vanishes in one byte, k does not
    (torch.float16, 16.0, 16.0),        # large but representable
])
def test_badly_scaled_inputs_only_cost_speed(sparse_switch, dtype, qscale, kscale):
    """The first walk reads q and k rounded to one byte (e4m3: largest value 448, smallest 2^-9) and only chooses
    keys; whatever it chooses, the bound it leads to is valid, so inputs far outside that range must still give the
    oracle's answer (through more candidates or through the dense kernel).  The products q k stay of order one or
    larger here, so the supports are short."""
    q, k, v = qkv(1, 2, 1, 1024, 128, dtype, seed=21)
    q = (q.float() * qscale).to(dtype)
    k = (k.float() * kscale).to(dtype)
    varlen = torch.tensor([1000], dtype=torch.int32)
    want = exact.dense_entmax_attention(q, k, v, 1.5, True, varlen)
    sparse_switch(True)
    out = forward(q, k, v, varlen)[0]
    assert torch.isfinite(out.float()).all()
    assert max_err(out, want) < 2e-2


@pytest.mark.parametrize("alpha,causal", [(1.5, False), (2.0, False), (2.0, True), (1.333, False), (1.333, True), (1.75, True), (1.15, False)])
def test_block_mask_entry_point_takes_the_same_path(sparse_switch, alpha, causal):
    q, k, v = qkv(2, 2, 2, 640, 64, torch.bfloat16, seed=7, scale=2.0)
    varlen = torch.tensor([640, 333], dtype=torch.int32)
    want = exact.dense_entmax_attention(q, k, v, alpha, causal, varlen)
    sparse_switch(True)
    out_s = forward(q, k, v, varlen, version=1, alpha=alpha, causal=causal, niter=20)[0]
    sparse_switch(False)
    out_d = forward(q, k, v, varlen, version=1, alpha=alpha, causal=causal, niter=20)[0]
    assert max_err(out_s, want) < 2e-2 and max_err(out_d, want) < 2e-2


def test_backward_takes_thresholds_and_tile_mask_of_the_sparse_path(sparse_switch):
    sparse_switch(True)
    q, k, v = qkv(2, 4, 2, 384, 128, torch.bfloat16, seed=9)
    varlen = torch.tensor([384, 250], dtype=torch.int32)
    dout = torch.randn(q.shape, generator=torch.Generator().manual_seed(1)).to(torch.bfloat16)
    qg, kg, vg = (t.to(DEV).requires_grad_(True) for t in (q, k, v))
    out = A.adasplash_v2(qg, kg, vg, varlen=varlen.to(DEV))
    out.backward(dout.to(DEV))
    want = exact.dense_entmax_attention_grads(q, k, v, dout, 1.5, True, varlen)
    for got, ref in zip((qg.grad, kg.grad, vg.grad), want):
        assert max_err(got, ref) < 4e-2


def test_padding_rows_may_hold_anything(sparse_switch):
    sparse_switch(True)
    q, k, v = qkv(1, 2, 2, 256, 64, torch.bfloat16, seed=13)
    varlen = torch.tensor([150], dtype=torch.int32)
    want = exact.dense_entmax_attention(q, k, v, 1.5, True, varlen)
    for t in (q, k, v):
        t[:, :, 150:] = float("nan")
    out = forward(q, k, v, varlen)[0]
    assert max_err(out, want) < 2e-2 and (out[:, :, 150:] == 0).all()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,Hq,Hkv,N,D,lens,alpha,causal,version", [
    (2, 4, 2, 512, 128, [512, 300], 1.5, True, 2),
    (1, 4, 1, 2048, 128, [1999], 1.5, True, 2),
    (2, 2, 2, 200, 64, [137, 200], 1.5, True, 2),
    (1, 2, 2, 512, 64, None, 2.0, False, 1),
    (2, 2, 2, 384, 128, [384, 129], 1.5, False, 1),
    (2, 2, 2, 384, 128, [384, 129], 1.333, False, 1),
    (1, 2, 2, 1024, 64, [1000], 1.75, True, 1),
])
def test_sparse_and_dense_dq_agree_with_the_oracle(sparse_switch, dtype, B, Hq, Hkv, N, D, lens, alpha, causal, version):
    """The backward's dQ comes from the rows' supports (sparse-support dQ kernel) or from the dense kernel
    (ADSP_SPARSE=0); dK and dV always come from the dense kernel, which reads delta and 1 / sum p from whichever of the
    two wrote them.  All three gradients against the oracle on both settings, dQ of the two against each other."""
    q, k, v = qkv(B, Hq, Hkv, N, D, dtype, seed=N + D + 1, scale=2.0 if alpha >= 1.75 else (1.5 if alpha < 1.5 else 1.0))
    varlen = None if lens is None else torch.tensor(lens, dtype=torch.int32)
    dout = torch.randn(q.shape, generator=torch.Generator().manual_seed(2)).to(dtype)
    want = exact.dense_entmax_attention_grads(q, k, v, dout, alpha, causal, varlen)
    grads = {}
    for on in (True, False):
        sparse_switch(on)
        qg, kg, vg = (t.to(DEV).requires_grad_(True) for t in (q, k, v))
        vl = None if varlen is None else varlen.to(DEV)
        if version == 2:
            out = A.adasplash_v2(qg, kg, vg, varlen=vl)
        else:
            out = A.adasplash_v1(qg, kg, vg, alpha=alpha, is_causal=causal, varlen=vl, niter=20)
        out.backward(dout.to(DEV))
        grads[on] = (qg.grad, kg.grad, vg.grad)
        for got, ref in zip(grads[on], want):
            assert max_err(got, ref) < 4e-2
    assert max_err(grads[True][0], grads[False][0].float().cpu()) < 4e-2
    if lens is not None:
        for b, l in enumerate(lens):
            assert (grads[True][0][b, :, l:] == 0).all()


def test_dense_supports_go_back_to_the_dense_backward_kernels(sparse_switch):
    """Flat scores: the sparse-support backward kernels give up the row blocks and key blocks whose lists overflow
    (most of them; the last key blocks, which few queries see, may still fit) and the dense kernels redo those.  The
    result agrees with the dense kernels' alone and with the oracle."""
    q, k, v = qkv(1, 4, 4, 1024, 64, torch.bfloat16, seed=3, scale=0.125)
    dout = torch.randn(q.shape, generator=torch.Generator().manual_seed(4)).to(torch.bfloat16)
    want = exact.dense_entmax_attention_grads(q, k, v, dout, 1.5, True, None)
    grads = {}
    for on in (True, False):
        sparse_switch(on)
        qg, kg, vg = (t.to(DEV).requires_grad_(True) for t in (q, k, v))
        A.adasplash_v2(qg, kg, vg, niter=10).backward(dout.to(DEV))
        grads[on] = (qg.grad, kg.grad, vg.grad)
        for got, ref in zip(grads[on], want):
            assert max_err(got, ref) < 4e-2
    for a, b in zip(grads[True], grads[False]):
        assert max_err(a, b.float().cpu()) < 4e-2
