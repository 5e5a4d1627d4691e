"""Writes the golden fixtures of tests/golden/ from the CPU oracle (``oracle.exact``).

The reference stores no vectors for this path, so the fixtures freeze the oracle's answers on the
reference's own CPU-sized configuration (B=1, H=8, N=128, D=64 fp32 causal alpha=1.5; entmax rows on
[128, 256] fp32, alpha in {1.5, 2}) plus two small GQA / varlen / generic-alpha cases, all from seed 42.
Run from the repository root:  python tests/golden/make_golden.py
"""

import sys
from pathlib import Path

import numpy as np
import torch

ROOT = Path(__file__).resolve().parents[2]
sys.path.insert(0, str(ROOT))
from oracle import exact  # noqa: E402

OUT = Path(__file__).resolve().parent


def main():
    g = torch.Generator().manual_seed(42)
    x = torch.randn(128, 256, generator=g)
    np.savez_compressed(OUT / "entmax_rows_128x256.npz", x=x.numpy(),
                        y15=exact.entmax_rows(x, 1.5).float().numpy(),
                        y20=exact.entmax_rows(x, 2.0).float().numpy(),
                        y1333=exact.entmax_rows(x, 1.333).float().numpy())

    q, k, v = (torch.randn(1, 8, 128, 64, generator=g) for _ in range(3))
    out = exact.dense_entmax_attention(q, k, v, 1.5, True)
    np.savez_compressed(OUT / "attn_v2_b1h8n128d64.npz", q=q.numpy(), k=k.numpy(), v=v.numpy(),
                        out=out.float().numpy())

    q = torch.randn(2, 4, 128, 32, generator=g)
    k = torch.randn(2, 2, 128, 32, generator=g)
    v = torch.randn(2, 2, 128, 32, generator=g)
    varlen = torch.tensor([100, 65], dtype=torch.int32)
    out = exact.dense_entmax_attention(q, k, v, 1.5, True, varlen)
    np.savez_compressed(OUT / "attn_v2_gqa_varlen.npz", q=q.numpy(), k=k.numpy(), v=v.numpy(), varlen=varlen.numpy(),
                        out=out.float().numpy())

    q, k, v = (torch.randn(1, 2, 128, 32, generator=g) for _ in range(3))
    varlen = torch.tensor([96], dtype=torch.int64)
    outs = {}
    for alpha in (1.333, 1.5, 2.0):
        for causal in (False, True):
            key = f"out_a{str(alpha).replace('.', 'p')}_{'causal' if causal else 'full'}"
            outs[key] = exact.dense_entmax_attention(q, k, v, alpha, causal, varlen).float().numpy()
    np.savez_compressed(OUT / "attn_v1_alphas.npz", q=q.numpy(), k=k.numpy(), v=v.numpy(), varlen=varlen.numpy(), **outs)


if __name__ == "__main__":
    main()
