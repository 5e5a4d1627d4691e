"""GPU parity of the attention backward (dq, dk, dv) against the oracle's closed-form entmax gradients,
which tests/test_oracle.py pins by finite differences of the forward oracle.

Tolerances on max |got - oracle|: fp32 1e-4 (what the reference asks of its own kernels against
entmax_bisect's autograd, tests/test_adasplash_v2.py:146-179; it has no 16-bit gradient test), 16-bit types
4e-2 on the magnitude-aware scale of tests/gpu_util.max_err: P and dX are rounded to the element type before
their MFMA, as the reference does (adasplash/adasplash_v2.py:1066-1068), and the sums run over hundreds of
such terms with |g| up to ~10."""

import pytest
import torch

import adasplash_amd as A
from oracle import exact
from tests.gpu_util import DEV, max_err

pytestmark = pytest.mark.gpu


def grad_tol(dtype):
    return 1e-4 if dtype == torch.float32 else 4e-2


def run_case(alpha, causal, B, Hq, Hkv, N, D, dtype, varlen=None, version=1, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    q = (scale * torch.randn(B, Hq, N, D, generator=g)).to(dtype)
    k = (scale * torch.randn(B, Hkv, N, D, generator=g)).to(dtype)
    v = torch.randn(B, Hkv, N, D, generator=g).to(dtype)
    do = torch.randn(B, Hq, N, D, generator=g).to(dtype)
    qg, kg, vg = (t.to(DEV).requires_grad_(True) for t in (q, k, v))
    vl = varlen.to(DEV) if varlen is not None else None
    if version == 2:
        out = A.adasplash_v2(qg, kg, vg, niter=10, varlen=vl)
    else:
        out = A.adasplash_v1(qg, kg, vg, alpha=alpha, is_causal=causal, varlen=vl, niter=20)
    out.backward(do.to(DEV))
    want = exact.dense_entmax_attention_grads(q, k, v, do, alpha, causal, varlen)
    return (qg.grad, kg.grad, vg.grad), want


def check(got, want, dtype, tol_scale=1.0):
    for name, g, w in zip(("dq", "dk", "dv"), got, want):
        assert g.dtype == dtype and g.shape == w.shape
        assert torch.isfinite(g).all(), name
        assert max_err(g, w) < tol_scale * grad_tol(dtype), name


@pytest.mark.parametrize("N,D", [(128, 64), (256, 128), (512, 32), (128, 16), (128, 256)])
def test_v2_backward_fp32(N, D):
    got, want = run_case(1.5, True, 1, 2, 2, N, D, torch.float32, version=2)
    check(got, want, torch.float32)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("N,D", [(256, 64), (512, 128), (256, 256)])
def test_v2_backward_16bit(dtype, N, D):
    got, want = run_case(1.5, True, 1, 2, 2, N, D, dtype, version=2)
    check(got, want, dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_v2_backward_gqa_and_varlen(dtype):
    # adasplash/adasplash_v2.py:1180-1188: dk / dv accumulate over the query heads of a K/V head;
    # lengths that end inside a 128-row block, inside a 64-key tile, and a full one
    varlen = torch.tensor([300, 77, 384], dtype=torch.int32)
    got, want = run_case(1.5, True, 3, 8, 2, 384, 64, dtype, varlen=varlen, version=2)
    check(got, want, dtype)
    for b, L in enumerate(varlen.tolist()):
        for g in got:
            assert (g[b, :, L:] == 0).all()  # padded rows get exactly zero gradient


def test_v2_backward_matches_reference_test_shape():
    # tests/test_adasplash_v2.py:146-179 at its smallest length
    got, want = run_case(1.5, True, 2, 2, 2, 1024, 64, torch.float32, version=2, seed=42)
    check(got, want, torch.float32)


@pytest.mark.parametrize("alpha", [1.333, 1.5, 2.0])
@pytest.mark.parametrize("causal", [False, True])
def test_v1_backward_alphas(alpha, causal):
    got, want = run_case(alpha, causal, 1, 2, 2, 256, 64, torch.float32)
    check(got, want, torch.float32)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_v1_backward_varlen_and_sparse_rows(dtype):
    # a higher temperature makes most tiles drop out of the forward's mask, which the backward reuses
    varlen = torch.tensor([512, 200], dtype=torch.int64)
    got, want = run_case(1.333, False, 2, 2, 2, 512, 64, dtype, varlen=varlen, scale=2.0)
    check(got, want, dtype)


def test_zero_upstream_gradient_gives_zero():
    q, k, v = (torch.randn(1, 2, 128, 64, device=DEV, requires_grad=True) for _ in range(3))
    out = A.adasplash(q, k, v)
    out.backward(torch.zeros_like(out))
    assert all((t.grad == 0).all() for t in (q, k, v))


def test_gradient_of_the_sum_vanishes_for_q_and_k():
    # rows of P sum to one, so with v = const the output does not depend on q and k
    q, k = (torch.randn(1, 2, 256, 64, device=DEV, requires_grad=True) for _ in range(2))
    v = torch.ones(1, 2, 256, 64, device=DEV, requires_grad=True)
    out = A.adasplash_v1(q, k, v, alpha=1.5, is_causal=True, niter=20)
    out.backward(torch.randn(1, 2, 256, 64, device=DEV))
    assert q.grad.abs().max() < 1e-4 and k.grad.abs().max() < 1e-4


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("version", [1, 2])
def test_padding_rows_may_hold_anything(dtype, version, D):
    # the reference never reads past a sequence's valid length (masked loads, adasplash/adasplash_v2.py:
    # 1030-1033, 1194-1207): NaNs parked in the padding of q, k, v and of the upstream gradient must not leak
    g = torch.Generator().manual_seed(5)
    B, H, N = 2, 2, 256
    varlen = torch.tensor([150, 256], dtype=torch.int32)
    q, k, v, do = (torch.randn(B, H, N, D, generator=g).to(dtype) for _ in range(4))
    dirty = [t.clone() for t in (q, k, v, do)]
    for t in dirty:
        t[0, :, 150:] = float("nan")

    def run(ts):
        qg, kg, vg = (t.to(DEV).requires_grad_(True) for t in ts[:3])
        if version == 2:
            out = A.adasplash_v2(qg, kg, vg, niter=10, varlen=varlen.to(DEV))
        else:
            out = A.adasplash_v1(qg, kg, vg, alpha=1.5, is_causal=False, varlen=varlen.to(DEV), niter=20)
        out.backward(ts[3].to(DEV))
        return out.detach(), qg.grad, kg.grad, vg.grad

    clean, soiled = run((q, k, v, do)), run(dirty)
    for a, b in zip(clean, soiled):
        assert torch.isfinite(b).all()
        assert torch.equal(a, b)


@pytest.mark.parametrize("version,alpha", [(1, 1.333), (1, 2.0), (2, 1.5)])
@pytest.mark.parametrize("dtype,D", [(torch.float32, 64), (torch.bfloat16, 128)])
def test_backward_after_a_forward_on_candidate_lists(version, alpha, dtype, D):
    # peaked scores: the forward's later solver steps and its output run on the per-lane lists, and the tile mask
    # the backward consumes comes from the listed keys
    causal = version == 2
    got, want = run_case(alpha, causal, 1, 2, 2, 1024, D, dtype, version=version, seed=3, scale=2.0)
    # dq and dk are linear in k and q, which are twice the size the 16-bit tolerance was set for
    check(got, want, dtype, tol_scale=1.0 if dtype == torch.float32 else 2.0)


@pytest.mark.parametrize("sparse", ["1", "0"])
@pytest.mark.parametrize("B,H,N,D,dtype,qscale,lens,causal,seed", [
    (2, 2, 200, 64, torch.bfloat16, 0.3, [160, 185], False, 12),
    (1, 2, 1024, 128, torch.float16, 1.0, None, False, 0),
    (2, 2, 777, 64, torch.float16, 1.0, [640, 651], False, 33),
])
def test_sparsemax_gradients_on_flat_scores(sparse, B, H, N, D, dtype, qscale, lens, causal, seed):
    """alpha = 2 weighs every member of a support alike in the backward (u = 1), so a threshold that is 1e-4 off --
    harmless to the output -- moves a key in or out of a support and changes that row's gradient by O(1).  With flat
    scores (small q) the supports are long and the dense kernels serve the rows (ADSP_SPARSE=0: all of them): their
    solver walk keeps fp32 sums for alpha = 2 so that the threshold converges to the oracle's (it was 2e-4 off with the
    packed f16 sums that alpha = 1.5 uses, and single rows of dq and dk were off by 1 to 5)."""
    import os
    old = os.environ.get("ADSP_SPARSE")
    os.environ["ADSP_SPARSE"] = sparse
    try:
        g = torch.Generator().manual_seed(seed)
        q = (qscale * torch.randn(B, H, N, D, generator=g)).to(dtype)
        k = torch.randn(B, H, N, D, generator=g).to(dtype)
        v = torch.randn(B, H, N, D, generator=g).to(dtype)
        do = torch.randn(B, H, N, D, generator=g).to(dtype)
        varlen = None if lens is None else torch.tensor(lens, dtype=torch.int32)
        qg, kg, vg = (t.to(DEV).requires_grad_(True) for t in (q, k, v))
        out = A.adasplash_v1(qg, kg, vg, alpha=2.0, is_causal=causal, varlen=None if varlen is None else varlen.to(DEV))
        out.backward(do.to(DEV))
        want = exact.dense_entmax_attention_grads(q, k, v, do, 2.0, causal, varlen)
        check((qg.grad, kg.grad, vg.grad), want, dtype)
    finally:
        if old is None:
            os.environ.pop("ADSP_SPARSE", None)
        else:
            os.environ["ADSP_SPARSE"] = old


@pytest.mark.parametrize("alpha,causal,B,Hq,Hkv,N,D,dtype,lens,version,scale", [
    (1.5, True, 2, 4, 2, 1024, 128, torch.bfloat16, [1024, 700], 2, 1.0),
    (1.5, True, 1, 2, 1, 3000, 64, torch.float16, [2777], 2, 1.0),
    (2.0, False, 2, 2, 2, 640, 64, torch.bfloat16, [640, 333], 1, 1.0),
    (1.5, True, 1, 4, 4, 2048, 128, torch.bfloat16, None, 1, 0.55),  # rows with long supports: some row blocks go to the dense kernels
])
def test_dkdv_from_the_dq_kernels_streams_and_from_its_own_walk(alpha, causal, B, Hq, Hkv, N, D, dtype, lens, version, scale):
    """The sparse-support dK/dV kernel takes the supports from the streams the dQ kernel left (default) or finds them
    with a score walk of its own (ADSP_BWD_STREAMS=0).  Both must meet the oracle, and they must agree with each other
    far inside the tolerance: the same members with scores that differ by a rounding at most."""
    import os
    varlen = None if lens is None else torch.tensor(lens, dtype=torch.int32)
    old = os.environ.get("ADSP_BWD_STREAMS")
    got = {}
    try:
        for mode in ("1", "0"):
            os.environ["ADSP_BWD_STREAMS"] = mode
            got[mode], want = run_case(alpha, causal, B, Hq, Hkv, N, D, dtype, varlen=varlen, version=version, seed=5, scale=scale)
            check(got[mode], want, dtype)
    finally:
        if old is None:
            os.environ.pop("ADSP_BWD_STREAMS", None)
        else:
            os.environ["ADSP_BWD_STREAMS"] = old
    for a, b in zip(got["1"], got["0"]):
        # (the kernel on the streams takes each member's two weights in the element type, the walking one in fp32)
        assert max_err(a, b.float().cpu(), report=False) < grad_tol(dtype)


@pytest.mark.parametrize("B,Hq,Hkv,N,D,dtype,lens,with_oracle,scale", [
    (2, 8, 2, 1024, 64, torch.bfloat16, [1024, 700], True, 1.0),   # 4 heads x 1024 rows: one 16-bit list entry names any of them
    (1, 4, 1, 3000, 128, torch.float16, [2777], True, 1.0),
    (1, 4, 2, 2048, 128, torch.bfloat16, [2048], True, 0.55),      # long supports: some row blocks, and their key blocks, go to the dense kernels
    (1, 16, 1, 4224, 64, torch.bfloat16, [4100], False, 1.0),      # 16 x 4224 > 65536: head after head, sums in the scratch slot
])
def test_late_key_blocks_served_for_all_query_heads_at_once(B, Hq, Hkv, N, D, dtype, lens, with_oracle, scale):
    """With a causal mask the dK/dV kernel on the streams serves the key blocks from 5/16 of a sequence on with one item
    for all query heads of a K/V head and writes dK and dV itself (ADSP_DKDV_MERGE256, default 80); the earlier blocks
    go per query head through fp32 partial rows and the reduction.  0 turns the merging off, 1 merges every block but
    the first (long items that are worked off in parts).  All three must agree -- the same members and weights, summed
    in another order -- and meet the oracle where it is affordable."""
    import os
    varlen = torch.tensor(lens, dtype=torch.int32)
    old = os.environ.get("ADSP_DKDV_MERGE256")
    got = {}
    want = None
    try:
        for mode in ("80", "0", "1"):
            os.environ["ADSP_DKDV_MERGE256"] = mode
            if with_oracle:
                got[mode], want = run_case(1.5, True, B, Hq, Hkv, N, D, dtype, varlen=varlen, version=2, seed=11, scale=scale)
                check(got[mode], want, dtype)
            else:
                g = torch.Generator().manual_seed(11)
                q = torch.randn(B, Hq, N, D, generator=g).to(dtype)
                k = torch.randn(B, Hkv, N, D, generator=g).to(dtype)
                v = torch.randn(B, Hkv, N, D, generator=g).to(dtype)
                do = torch.randn(B, Hq, N, D, generator=g).to(dtype)
                qg, kg, vg = (t.to(DEV).requires_grad_(True) for t in (q, k, v))
                A.adasplash_v2(qg, kg, vg, niter=10, varlen=varlen.to(DEV)).backward(do.to(DEV))
                got[mode] = (qg.grad, kg.grad, vg.grad)
                assert all(torch.isfinite(t).all() for t in got[mode])
    finally:
        if old is None:
            os.environ.pop("ADSP_DKDV_MERGE256", None)
        else:
            os.environ["ADSP_DKDV_MERGE256"] = old
    for mode in ("0", "1"):
        for a, b in zip(got["80"], got[mode]):
            # (fp32 sums of the same terms in another order, rounded once to the element type)
            assert max_err(a, b.float().cpu(), report=False) < 0.25 * grad_tol(dtype), mode
    from adasplash_amd import _lib
    lib = _lib.load()
    dt = _lib.dtype_code(got["80"][0])
    assert lib.adsp_attn_bwd_workspace_bytes_causal(B, Hq, Hkv, N, D, dt, 1) < lib.adsp_attn_bwd_workspace_bytes(B, Hq, Hkv, N, D, dt)
    assert lib.adsp_attn_bwd_workspace_bytes_causal(B, Hq, Hkv, N, D, dt, 0) == lib.adsp_attn_bwd_workspace_bytes(B, Hq, Hkv, N, D, dt)


@pytest.mark.parametrize("alpha,causal,B,Hq,Hkv,N,D,dtype,lens,version,scale,sparse", [
    (1.5, True, 2, 4, 2, 1024, 128, torch.bfloat16, [1024, 700], 2, 1.0, "1"),
    (1.5, True, 1, 2, 1, 3000, 64, torch.float16, [2777], 2, 1.0, "1"),
    (2.0, False, 2, 2, 2, 640, 64, torch.bfloat16, [640, 333], 1, 1.0, "1"),
    (1.5, True, 1, 4, 4, 2048, 128, torch.bfloat16, None, 1, 0.55, "1"),  # some row blocks go to the dense kernels: no supports kept for them
    (1.5, True, 2, 2, 2, 512, 64, torch.bfloat16, [512, 300], 2, 1.0, "0"),   # the dense forward keeps nothing: every flag is cleared
    (1.333, False, 1, 2, 2, 1500, 128, torch.bfloat16, [1400], 1, 1.5, "1"),  # any alpha in [1.125, 2) takes the same kernels
    (1.8, True, 2, 2, 2, 768, 64, torch.float16, [768, 500], 1, 1.5, "1"),
])
def test_backward_with_and_without_the_supports_the_forward_kept(alpha, causal, B, Hq, Hkv, N, D, dtype, lens, version, scale, sparse):
    """With a gradient asked for the forward keeps the supports it found and the dQ kernel takes them from there
    (``set_keep_supports("always")``; "auto" does the same up to a size); "never" makes it find them again with its
    score walk.  Both must meet the oracle and agree with each other (the same members up to scores that differ by a
    rounding)."""
    import os
    varlen = None if lens is None else torch.tensor(lens, dtype=torch.int32)
    old = os.environ.get("ADSP_SPARSE")
    old_mode = A.set_keep_supports("always")
    got = {}
    try:
        os.environ["ADSP_SPARSE"] = sparse
        for mode in ("always", "never"):
            A.set_keep_supports(mode)
            got[mode], want = run_case(alpha, causal, B, Hq, Hkv, N, D, dtype, varlen=varlen, version=version, seed=6, scale=scale)
            check(got[mode], want, dtype)
    finally:
        A.set_keep_supports(old_mode)
        if old is None:
            os.environ.pop("ADSP_SPARSE", None)
        else:
            os.environ["ADSP_SPARSE"] = old
    for a, b in zip(got["always"], got["never"]):
        # (the kernel on the streams takes each member's two weights in the element type, the walking one in fp32)
        assert max_err(a, b.float().cpu(), report=False) < grad_tol(dtype)


def _both_routes(q, k, v, do, fn):
    """(dq, dk, dv) on the device from the sparse-support kernels (default) and from the dense kernels alone."""
    import os
    old = os.environ.get("ADSP_SPARSE")
    res = {}
    try:
        for mode in ("1", "0"):
            os.environ["ADSP_SPARSE"] = mode
            qg, kg, vg = (t.clone().requires_grad_(True) for t in (q, k, v))
            fn(qg, kg, vg).backward(do)
            res[mode] = (qg.grad, kg.grad, vg.grad)
    finally:
        if old is None:
            os.environ.pop("ADSP_SPARSE", None)
        else:
            os.environ["ADSP_SPARSE"] = old
    return res["1"], res["0"]


def _scaled_diff_on_device(a, b):
    a, b = a.float(), b.float()
    return ((a - b).abs() / torch.clamp(b.abs() / 2, min=1.0)).max().item()


def test_full_size_gqa_varlen_backward():
    """The headline workload's backward at full size (B=8, Hq=32, Hkv=8, N=8192, D=128, bf16, ragged lengths): the
    gradients of padded rows and keys are zero; one whole K/V head of the shortest sequence (its four query heads)
    meets the oracle; and the two independent routes - fp32 arithmetic on the kept supports, the dense MFMA kernels -
    agree everywhere within twice the bound each is held to against the oracle.  niter = 1, the API's default: the
    sparse route solves to convergence whatever niter is, and the dense kernel serving a call alone takes the
    reference's extra update behind its niter steps (adasplash/adasplash_v2.py:617-681)."""
    g = torch.Generator().manual_seed(11)
    B, Hq, Hkv, N, D = 8, 32, 8, 8192, 128
    dt = torch.bfloat16
    q = torch.randn(B, Hq, N, D, generator=g).to(dt).to(DEV)
    k = torch.randn(B, Hkv, N, D, generator=g).to(dt).to(DEV)
    v = torch.randn(B, Hkv, N, D, generator=g).to(dt).to(DEV)
    do = torch.randn(B, Hq, N, D, generator=g).to(dt).to(DEV)
    lens = [7297, 6553, 5730, 1500, 6310, 4494, 8192, 4555]
    vl = torch.tensor(lens, dtype=torch.int32, device=DEV)
    sparse, dense = _both_routes(q, k, v, do, lambda a, b, c: A.adasplash_v2(a, b, c, niter=1, varlen=vl))
    for got in (sparse, dense):
        for t in got:
            assert torch.isfinite(t.float()).all()
            for b, L in enumerate(lens):
                assert (t[b, :, L:] == 0).all()
    b, kvh, L = 3, 5, 1500
    hs = slice(4 * kvh, 4 * kvh + 4)
    want = exact.dense_entmax_attention_grads(q[b:b + 1, hs, :L].cpu(), k[b:b + 1, kvh:kvh + 1, :L].cpu(),
                                              v[b:b + 1, kvh:kvh + 1, :L].cpu(), do[b:b + 1, hs, :L].cpu(), 1.5, True)
    for got in (sparse, dense):
        part = (got[0][b:b + 1, hs, :L], got[1][b:b + 1, kvh:kvh + 1, :L], got[2][b:b + 1, kvh:kvh + 1, :L])
        check(part, want, dt)
    for name, a_, b_ in zip(("dq", "dk", "dv"), sparse, dense):
        d = _scaled_diff_on_device(a_, b_)
        print(name, "sparse against dense route, magnitude-scaled:", d)
        assert d < 2 * grad_tol(dt), name


def test_full_size_block_mask_backward_two_routes():
    """The block-mask workload's backward at full size (B=2, H=16, N=16384, D=64, bf16, alpha = 1.333, non-causal, q
    and k scaled by 3): the sparse-support kernels' generic-alpha instances against the dense kernels', each of which
    the smaller cases hold to the oracle."""
    g = torch.Generator().manual_seed(12)
    B, H, N, D = 2, 16, 16384, 64
    dt = torch.bfloat16
    q = (3 * torch.randn(B, H, N, D, generator=g)).to(dt).to(DEV)
    k = (3 * torch.randn(B, H, N, D, generator=g)).to(dt).to(DEV)
    v = torch.randn(B, H, N, D, generator=g).to(dt).to(DEV)
    do = torch.randn(B, H, N, D, generator=g).to(dt).to(DEV)
    sparse, dense = _both_routes(q, k, v, do,
                                 lambda a, b, c: A.adasplash_v1(a, b, c, alpha=1.333, is_causal=False, niter=10))
    for name, a_, b_ in zip(("dq", "dk", "dv"), sparse, dense):
        assert torch.isfinite(a_.float()).all() and torch.isfinite(b_.float()).all()
        d = _scaled_diff_on_device(a_, b_)
        print(name, "sparse against dense route, magnitude-scaled:", d)
        assert d < 2 * grad_tol(dt), name
