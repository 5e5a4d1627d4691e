"""GPU test of the dense kernels' block numbering (xcd_block_map in csrc/common.h): the workgroups of a launch are dealt
to (K/V head, block, member of the group) by a rule that depends on the number of heads, of blocks per head and on
the mask.  Whatever the rule, a batch must give what its items give one by one: a block that the numbering left out,
or dealt to the wrong place, shows as a row block that differs."""

import os

import pytest
import torch

from adasplash_amd import _attention
from tests.gpu_util import DEV

pytestmark = pytest.mark.gpu


@pytest.fixture
def dense_only():
    old = os.environ.get("ADSP_SPARSE")
    os.environ["ADSP_SPARSE"] = "0"
    yield
    if old is None:
        os.environ.pop("ADSP_SPARSE", None)
    else:
        os.environ["ADSP_SPARSE"] = old


# (B, Hq, Hkv, N, D, causal): heads per XCD 1, 2, 3 and a count that is no multiple of 8; sets of several heads, of
# one head, and a last set that is smaller than the others (24 heads of 128 blocks: sets of two, three per XCD)
CASES = [
    (1, 8, 8, 512, 64, True),
    (2, 8, 8, 1024, 64, True),
    (3, 8, 8, 256, 64, True),
    (3, 32, 8, 4096, 64, True),
    (1, 6, 3, 512, 64, True),
    (2, 16, 8, 2048, 128, True),
    (2, 8, 8, 1024, 64, False),
]


@pytest.mark.parametrize("B,Hq,Hkv,N,D,causal", CASES)
def test_a_batch_equals_its_items_forward_and_backward(dense_only, B, Hq, Hkv, N, D, causal):
    g = torch.Generator().manual_seed(B * 1000 + N + D)
    q = torch.randn(B, Hq, N, D, generator=g).bfloat16().to(DEV)
    k = torch.randn(B, Hkv, N, D, generator=g).bfloat16().to(DEV)
    v = torch.randn(B, Hkv, N, D, generator=g).bfloat16().to(DEV)
    dout = torch.randn(B, Hq, N, D, generator=g).bfloat16().to(DEV)
    version, alpha = (2, 1.5) if causal else (1, 1.5)

    def run(qq, kk, vv, dd):
        out, taus, bmask = _attention.launch_forward(qq, kk, vv, version=version, alpha=alpha, is_causal=causal, niter=2, varlen=None)
        dq, dk, dv = _attention.launch_backward(qq, kk, vv, dd, taus, bmask, alpha=alpha, is_causal=causal, varlen=None)[:3]
        return out, taus, dq, dk, dv

    whole = run(q, k, v, dout)
    for b in range(B):
        one = run(q[b:b + 1].contiguous(), k[b:b + 1].contiguous(), v[b:b + 1].contiguous(), dout[b:b + 1].contiguous())
        for name, w, o in zip(("out", "taus", "dq", "dk", "dv"), whole, one):
            assert torch.equal(w[b], o[0]), f"{name}: batch item {b} differs from the item run alone"
