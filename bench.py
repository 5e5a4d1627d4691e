#!/usr/bin/env python3
"""Benchmark of the sparse entmax attention hot path on one MI355X.

``python bench.py --gpus 1 --steps K --warmup W`` runs W untimed and K timed forward passes of the
headline workload and prints ONE JSON line.  A step is one ``adasplash_v2`` causal forward on one batch
of synthetic inputs that are already resident in HBM.

Workloads (``--workload``):
  c4   adasplash_v2 causal GQA + varlen, B=8 Hq=32 Hkv=8 N=8192 D=128 bf16   (headline, default)
  c3   adasplash_v2 causal MHA, B=4 H=16 N=4096 D=64 bf16, q pre-scaled by 1/sqrt(D)
  c5   adasplash_v1 non-causal alpha=1.333 niter=10, B=2 H=16 N=16384 D=64 bf16, q,k x3
  c2   entmax rows x[16384, 8192] = 4*N(0,1), bf16 and fp32, alpha in {1.5, 2}
  c2_bwd  entmax rows backward on the same shape (reads y, writes dx, reads dy on the support only)
  c4_bwd, c3_bwd, c5_bwd   dq, dk, dv of the c4 / c3 / c5 forward (2.5 x its dense-equivalent FLOPs per step)
The default run also times c3, c5, the entmax rows workloads (c2, c2_bwd) and the c4 backward and reports them under
``extra``, with the v2 tile statistics of the headline workload (key tiles of 128 rows x 64 keys inside the causal /
valid domain, those the block mask keeps, and the share of row blocks the sparse-support kernel served).

Dense-equivalent FLOPs of causal attention = 2 * Hq * D * sum_b L_b^2 (QK^T and PV, each halved by
causality); non-causal = 4 * B * H * N^2 * D.  Rows bytes = rows * cols * (sizeof(in) + sizeof(out)).
Peaks are MI355X's published ones: bf16 dense MFMA 2500 TFLOP/s, HBM 8000 GB/s.
"""

import argparse
import json
import os
import sys
import time

import torch

MFMA_BF16_PEAK_TFLOPS = 2500.0
HBM_PEAK_GBS = 8000.0

# HBM bytes per launch of the dominant kernel, from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of these
# same workloads, each counter scaled by what it reads for a plain 1 GiB copy (FETCH_SIZE x 2.0,
# WRITE_SIZE x 1.0); the summaries are in profiles/.  None = not measured.
MEASURED_HBM_TRAFFIC_BYTES = {"c4": 2.467e9, "c3": 0.5076e9, "c5": 0.556e9, "c2_f32": 1.0739e9, "c2_bf16": 0.5370e9,
                              "c2_bwd_f32": 1.0847e9, "c2_bwd_bf16": 0.5476e9,
                              "c4_bwd": 12.57e9,
                              "c5_bwd": 0.795e9}  # c4_bwd: sparse dq kernel 3.21e9 + dk/dv kernel on its streams 8.75e9 + reduction 0.61e9


# The kernel that dominates a forward step of each workload.  A 16-bit step of the v2 entry point is four launches: a
# probe of the score distribution, the one-byte copy of K, the sparse-support kernel and the dense kernel, of which the
# last returns at once unless the sparse-support kernel left row blocks over (c3: the probe marks every head dense, the
# copy of K and the sparse-support kernel step aside and the dense kernel does all the work).
FWD_KERNELS = {"c4": "attn_fwd_sparse_kernel<bf16, 128> (step = probe + fp8 copy of K + this + attn_fwd_kernel on leftovers)",
               "c3": "attn_fwd_kernel<bf16, 64, single step> (step = probe + sparse-support kernel stepping aside + this)",
               "c5": "attn_fwd_sparse_kernel<bf16, 64, generic alpha> (step = probe + fp8 copy of K + this + attn_fwd_kernel on leftovers)"}
_BWD_SPARSE = "attn_bwd_dq_sparse_kernel + attn_bwd_dkdv_stream_kernel"
BWD_KERNELS = {"c4_bwd": _BWD_SPARSE + " + dkdv_reduce_kernel", "c3_bwd": "attn_bwd_dq_kernel + attn_bwd_dkdv_kernel",
               "c5_bwd": _BWD_SPARSE + " (generic alpha; one query head per K/V head: no reduction)"}


def _events_ms(fn, steps, warmup):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record()
    for _ in range(steps):
        fn()
    stop.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    return start.elapsed_time(stop) / steps, wall_ms / steps


def make_c4(device, seed=42):
    g = torch.Generator().manual_seed(seed)
    B, Hq, Hkv, N, D = 8, 32, 8, 8192, 128
    q = torch.randn(B, Hq, N, D, generator=g).to(torch.bfloat16).to(device)
    k = torch.randn(B, Hkv, N, D, generator=g).to(torch.bfloat16).to(device)
    v = torch.randn(B, Hkv, N, D, generator=g).to(torch.bfloat16).to(device)
    varlen = torch.randint(N // 4, N + 1, (B,), generator=g, dtype=torch.int32)
    flops = 2.0 * Hq * D * float((varlen.double() ** 2).sum())
    cfg = {"workload": "c4: adasplash_v2 causal GQA+varlen fwd", "B": B, "Hq": Hq, "Hkv": Hkv, "N": N, "D": D,
           "alpha": 1.5, "niter": 1, "varlen": varlen.tolist()}
    return (q, k, v, varlen.to(device)), flops, cfg


def make_c3(device, seed=42):
    g = torch.Generator().manual_seed(seed)
    B, H, N, D = 4, 16, 4096, 64
    q = (torch.randn(B, H, N, D, generator=g) / 8.0).to(torch.bfloat16).to(device)
    k = torch.randn(B, H, N, D, generator=g).to(torch.bfloat16).to(device)
    v = torch.randn(B, H, N, D, generator=g).to(torch.bfloat16).to(device)
    flops = 2.0 * H * D * B * float(N) ** 2
    cfg = {"workload": "c3: adasplash_v2 causal MHA fwd, q pre-scaled 1/sqrt(D)", "B": B, "Hq": H, "Hkv": H, "N": N,
           "D": D, "alpha": 1.5, "niter": 1}
    return (q, k, v, None), flops, cfg


def make_c5(device, seed=42):
    g = torch.Generator().manual_seed(seed)
    B, H, N, D = 2, 16, 16384, 64
    q = (3.0 * torch.randn(B, H, N, D, generator=g)).to(torch.bfloat16).to(device)
    k = (3.0 * torch.randn(B, H, N, D, generator=g)).to(torch.bfloat16).to(device)
    v = torch.randn(B, H, N, D, generator=g).to(torch.bfloat16).to(device)
    flops = 4.0 * B * H * float(N) ** 2 * D
    cfg = {"workload": "c5: adasplash_v1 block-mask non-causal fwd, q,k x3", "B": B, "H": H, "N": N, "D": D,
           "alpha": 1.333, "niter": 10}
    return (q, k, v), flops, cfg


def v2_tile_stats(q, k, v, varlen):
    """Tile statistics of one adasplash_v2 forward, from the block mask it writes: a tile is 128 query rows x 64 keys.
    `grid` counts all tiles of the padded problem, `domain` those that hold a valid (row, key) pair under the causal
    mask and the sequence lengths (the difference is excluded by causality or padding, not by tau), `kept` those in
    which some row has a non-zero probability; `skipped_by_tau` = domain - kept."""
    from adasplash_amd import _attention

    B, Hq, N, _ = q.shape
    _, _, bmask = _attention.launch_forward(q, k, v, version=2, alpha=1.5, is_causal=True, niter=1, varlen=varlen)
    n_blk, n_tile = (N + 127) // 128, (N + 63) // 64
    lens = varlen.cpu().long() if varlen is not None else torch.full((B,), N, dtype=torch.long)
    m0 = torch.arange(n_blk) * 128
    row_hi = torch.minimum(m0[None, :] + 128, lens[:, None])  # [B, n_blk]
    domain_per_blk = torch.where(m0[None, :] < lens[:, None], (row_hi + 63) // 64, torch.zeros_like(row_hi))
    domain = int(domain_per_blk.sum()) * Hq
    words = bmask.view(B, Hq, n_blk, -1).cpu()
    kept = 0
    for w in range(words.shape[-1]):
        x = words[..., w].to(torch.int64) & 0xFFFFFFFF
        for bit in range(32):
            kept += int(((x >> bit) & 1).sum())
    grid = B * Hq * n_blk * n_tile
    return {"tile": "128 rows x 64 keys", "tiles_grid": grid, "tiles_domain": domain, "tiles_kept": kept,
            "tiles_excluded_by_causality_or_padding": grid - domain, "tiles_skipped_by_tau": domain - kept,
            "tiles_skipped_frac_of_domain": (domain - kept) / domain if domain else None}


def bench_attention(name, steps, warmup, device, backward=False):
    import adasplash_amd as A

    if name == "c4":
        (q, k, v, varlen), flops, cfg = make_c4(device)
        fn = lambda: A.adasplash_v2(q, k, v, niter=1, varlen=varlen)  # noqa: E731
    elif name == "c3":
        (q, k, v, varlen), flops, cfg = make_c3(device)
        fn = lambda: A.adasplash_v2(q, k, v, niter=1)  # noqa: E731
    else:
        (q, k, v), flops, cfg = make_c5(device)
        fn = lambda: A.adasplash_v1(q, k, v, alpha=1.333, is_causal=False, niter=10)  # noqa: E731
    if backward:
        # one step = dq, dk, dv for a fixed upstream gradient (the forward runs once, outside the timed region);
        # dense-equivalent work: S recomputed, dP, dV, dK, dQ = 2.5 x the forward's two products
        from adasplash_amd import _attention

        # (as the autograd function does: the forward keeps the supports it found for the backward)
        if name == "c5":
            kw, varlen = dict(alpha=1.333, is_causal=False), None
            fwd_kw = dict(version=1, niter=10, **kw)
        else:
            kw = dict(alpha=1.5, is_causal=True)
            fwd_kw = dict(version=2, niter=1, **kw)
        out, taus, bmask, supports = _attention.launch_forward(q, k, v, varlen=varlen, keep_supports=True, **fwd_kw)
        cfg = dict(cfg, supports_kept_bytes=0 if supports is None else supports.numel())
        dout = torch.randn(q.shape, generator=torch.Generator().manual_seed(7)).to(q.dtype).to(device)
        fn = lambda: _attention.launch_backward(q, k, v, dout, taus, bmask, varlen=varlen,  # noqa: E731
                                                supports=supports, **kw)
        flops = 2.5 * flops
        cfg = dict(cfg, workload=cfg["workload"].replace("fwd", "bwd (dq, dk, dv)"))
    if (name == "c3" and not backward) or (name == "c5" and backward):
        # a step of 0.35 ms (0.66 ms): a short run would be timed while the clocks still ramp (the rows workloads do the same)
        steps, warmup = max(steps, 100), max(warmup, 300)
    ms, wall_ms = _events_ms(fn, steps, warmup)
    tflops = flops / (ms * 1e-3) / 1e12
    res = {"ms_per_step": ms, "wall_ms_per_step": wall_ms, "eff_tflops": tflops, "flops_per_step": flops,
           "frac_mfma_peak": tflops / MFMA_BF16_PEAK_TFLOPS, "config": cfg, "steps": steps, "warmup": warmup}
    if name == "c4" and not backward:
        # the same forward as the autograd function runs it when a gradient is asked for: it also keeps the supports
        # it found for the backward (its candidate streams go to a buffer of their own instead of the workspace)
        from adasplash_amd import _attention

        keep_fn = lambda: _attention.launch_forward(q, k, v, version=2, alpha=1.5, is_causal=True, niter=1,  # noqa: E731
                                                    varlen=varlen, keep_supports="always")
        kms, _ = _events_ms(keep_fn, steps, warmup)
        kept = keep_fn()[3]
        res["forward_keeping_supports"] = {"ms_per_step": kms, "supports_bytes": 0 if kept is None else kept.numel(),
                                           "steps": steps, "warmup": warmup}
        del kept
    if name in ("c4", "c3") and not backward:
        res["tiles"] = v2_tile_stats(q, k, v, varlen)
    if name == "c5" and not backward:
        from adasplash_amd.adasplash_block_mask import tile_sparsity

        _, total, active = tile_sparsity(q, k, v, alpha=1.333, is_causal=False, niter=10)
        res["tiles_16x16_total"] = total
        res["tiles_16x16_active"] = active
        res["tiles_skipped_frac"] = (1.0 - active / total) if total else None
    return res


def bench_c4_sweep(steps, warmup, device, scales=(0.25, 0.5, 0.75, 1.0, 2.0)):
    env_scales = os.environ.get("ADSP_BENCH_SWEEP_SCALES")
    if env_scales:
        scales = tuple(float(x) for x in env_scales.split(","))
    """The headline shapes with q scaled: from flat score distributions (supports of hundreds of keys, the dense
    kernel's case) to peaked ones (the sparse-support kernel's).  Per scale: the step as the library routes it, the step
    with every K/V head left to the dense kernel by the probe (ADSP_PROBE_MAX_SUPPORT=0: the dense kernel as it runs
    behind the sparse-support kernel), and the share of row blocks the sparse-support kernel served (the library's
    control word counts the row blocks it left to the dense kernel).  The lengths and
    the dense-equivalent FLOPs are the headline workload's."""
    from adasplash_amd import _lib

    lib = _lib.load()
    (q0, k, v, varlen), flops, _ = make_c4(device)
    B, Hq, N, D = q0.shape
    Hkv = k.shape[1]
    dt = _lib.dtype_code(q0)
    out = torch.empty_like(q0)
    taus = torch.empty((B, Hq, N), device=device, dtype=torch.float32)
    bmask = torch.empty((B, Hq, lib.adsp_attn_bmask_words(N)), device=device, dtype=torch.int32)
    nws = lib.adsp_attn_workspace_bytes(B, Hq, Hkv, N, D, dt)
    ws = torch.zeros((nws,), device=device, dtype=torch.uint8)
    stream = _lib.current_stream(device)
    items = B * Hq * ((N + 127) // 128)
    steps, warmup = max(steps, 5), max(warmup, 5)
    points = []
    old = os.environ.get("ADSP_PROBE_MAX_SUPPORT")
    try:
        for sc in scales:
            q = (q0.float() * sc).to(q0.dtype)

            def fn():
                st = lib.adsp_attn_v2_fwd(q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), taus.data_ptr(),
                                          bmask.data_ptr(), varlen.data_ptr(), 32, B, Hq, Hkv, N, D, dt, 1,
                                          ws.data_ptr(), nws, stream)
                assert st == 0

            os.environ.pop("ADSP_PROBE_MAX_SUPPORT", None)
            if old is not None:
                os.environ["ADSP_PROBE_MAX_SUPPORT"] = old
            ms, _ = _events_ms(fn, steps, warmup)
            # eight work counters, then {row blocks left to the dense kernel, all dense, left after work was spent on them}
            ctrl = ws[:64].view(torch.int32).cpu()
            left = items if int(ctrl[9]) != 0 else int(ctrl[8])
            gave_up = 0 if int(ctrl[9]) != 0 else int(ctrl[10])
            os.environ["ADSP_PROBE_MAX_SUPPORT"] = "0"
            ms_dense, _ = _events_ms(fn, steps, warmup)
            points.append({"q_scale": sc, "ms": ms, "ms_dense_kernel_only": ms_dense,
                           "frac_mfma_peak": flops / (ms * 1e-3) / 1e12 / MFMA_BF16_PEAK_TFLOPS,
                           "row_blocks_served_by_sparse_kernel": 1.0 - left / items,
                           "row_blocks_given_up_by_sparse_kernel": gave_up / items,
                           "ms_over_dense_only": ms / ms_dense})
            del q
    finally:
        if old is None:
            os.environ.pop("ADSP_PROBE_MAX_SUPPORT", None)
        else:
            os.environ["ADSP_PROBE_MAX_SUPPORT"] = old
    return {"steps": steps, "warmup": warmup, "points": points}


def bench_rows(steps, warmup, device, rows=16384, cols=8192):
    """Entmax rows: rotate over several input/output pairs so every read comes from HBM, not the
    256 MB last-level cache."""
    from adasplash_amd import _lib

    lib = _lib.load()
    out = {}
    g = torch.Generator().manual_seed(42)
    base = 4.0 * torch.randn(rows, cols, generator=g)
    for dt, dname in ((torch.bfloat16, "bf16"), (torch.float32, "f32")):
        nbuf = 4
        xs = [base.roll(i, 0).to(dt).to(device) for i in range(nbuf)]
        # Outputs are allocated once and the launches go through the C ABI, so that the timed region holds kernel
        # launches only (a launch lasts 0.08-0.18 ms; the Python wrapper adds about 13 us of host time per call).
        # 200 untimed launches first (20-40 ms): the first few milliseconds after an idle period run at lower clocks.
        ys = [torch.empty_like(x) for x in xs]
        nbytes = rows * cols * 2 * xs[0].element_size()
        stream = _lib.current_stream(device)
        for alpha in (1.5, 2.0):
            state = {"i": 0}

            def fn():
                i = state["i"] % nbuf
                st = lib.adsp_entmax_rows_fwd(xs[i].data_ptr(), ys[i].data_ptr(), rows, cols, _lib.dtype_code(xs[i]),
                                              alpha, 2, 1, 0, stream)
                assert st == 0
                state["i"] += 1

            ms, _ = _events_ms(fn, max(steps, 100), max(warmup, 200))
            gbs = nbytes / (ms * 1e-3) / 1e9
            out[f"{dname}_alpha{alpha}"] = {"ms": ms, "GBps": gbs, "frac_hbm_peak": gbs / HBM_PEAK_GBS,
                                            "bytes": nbytes, "steps": max(steps, 100), "warmup": max(warmup, 200)}
        del xs, ys
        torch.cuda.empty_cache()
    return out


def bench_rows_backward(steps, warmup, device, rows=16384, cols=8192):
    """Entmax rows backward on the forward's own outputs; buffers rotated as in ``bench_rows``.  The kernel
    reads y, writes dx, and reads dy only where y is non-zero (a fraction of a percent of these rows), so the
    algorithmic bytes are 2 * rows * cols * sizeof(dtype); counting dy in full would put the kernel above the
    HBM peak."""
    import adasplash_amd as A
    from adasplash_amd import _lib

    lib = _lib.load()
    out = {}
    g = torch.Generator().manual_seed(42)
    base = 4.0 * torch.randn(rows, cols, generator=g)
    for dt, dname in ((torch.bfloat16, "bf16"), (torch.float32, "f32")):
        nbuf = 4
        ys = [A.triton_entmax(base.roll(i, 0).to(dt).to(device), alpha=1.5) for i in range(nbuf)]
        dys = [torch.randn(rows, cols, generator=g).to(dt).to(device) for _ in range(nbuf)]
        dxs = [torch.empty_like(y) for y in ys]
        nbytes = rows * cols * 2 * ys[0].element_size()
        stream = _lib.current_stream(device)
        state = {"i": 0}

        def fn():
            i = state["i"] % nbuf
            st = lib.adsp_entmax_rows_bwd(ys[i].data_ptr(), dys[i].data_ptr(), dxs[i].data_ptr(), rows, cols,
                                          _lib.dtype_code(ys[i]), 1.5, stream)
            assert st == 0
            state["i"] += 1

        ms, _ = _events_ms(fn, max(steps, 100), max(warmup, 200))
        gbs = nbytes / (ms * 1e-3) / 1e9
        out[f"{dname}_alpha1.5"] = {"ms": ms, "GBps": gbs, "frac_hbm_peak": gbs / HBM_PEAK_GBS, "bytes": nbytes,
                                    "steps": max(steps, 100), "warmup": max(warmup, 200)}
        del ys, dys, dxs
        torch.cuda.empty_cache()
    return out


def cpu_baseline():
    """Dense exact-entmax attention (the oracle) on the host cores, fp32 torch ops, on a bounded slice
    of the headline workload: B=1, Hq=4, Hkv=1, N=4096, D=128, causal, alpha=1.5."""
    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
    from oracle import exact

    g = torch.Generator().manual_seed(42)
    B, Hq, Hkv, N, D = 1, 4, 1, 4096, 128
    q = torch.randn(B, Hq, N, D, generator=g).to(torch.bfloat16)
    k = torch.randn(B, Hkv, N, D, generator=g).to(torch.bfloat16)
    v = torch.randn(B, Hkv, N, D, generator=g).to(torch.bfloat16)
    flops = 2.0 * Hq * D * B * float(N) ** 2
    exact.dense_entmax_attention(q, k, v, 1.5, True, dtype=torch.float32)  # warm-up
    times = []
    t_end = time.perf_counter() + 20.0
    while len(times) < 3 or (time.perf_counter() < t_end and len(times) < 10):
        t0 = time.perf_counter()
        exact.dense_entmax_attention(q, k, v, 1.5, True, dtype=torch.float32)
        times.append(time.perf_counter() - t0)
    times.sort()
    med = times[len(times) // 2]
    return {"value": flops / med / 1e12, "unit": "TFLOP/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"oracle.exact.dense_entmax_attention fp32, B={B} Hq={Hq} Hkv={Hkv} N={N} D={D} causal "
                      f"alpha=1.5, median of {len(times)} runs ({med * 1e3:.0f} ms each), host cpu_count="
                      f"{os.cpu_count()}"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="c4", choices=["c4", "c3", "c5", "c2", "copy", "c4_bwd", "c3_bwd", "c5_bwd", "c2_bwd", "c4_sweep"])
    ap.add_argument("--no-extra", action="store_true", help="skip the entmax-rows and CPU-baseline legs")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (the op shards over batch and "
              "KV-head groups without communication); run with --gpus 1.", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py needs a ROCm GPU (no CPU fallback exists for the kernels).", file=sys.stderr)
        sys.exit(1)
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)

    from adasplash_amd import _lib

    line = {"metric": "v2 fwd ms + eff. TFLOPS/%MFMA peak (N=8192,D=128,GQA); entmax rows GB/s",
            "build_id": _lib.build_id(), "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "higher_is_better": True, "scaling": "weak",
            "vs_baseline": None, "data": "synthetic"}
    if args.workload == "copy":
        # plain device copy of known size: the reference point for scaling rocprofv3's FETCH_SIZE / WRITE_SIZE
        x = torch.empty(1 << 30, dtype=torch.uint8, device=device).random_(0, 255)
        y = torch.empty_like(x)
        ms, _ = _events_ms(lambda: y.copy_(x), args.steps, args.warmup)
        line.update({"value": 2 * x.numel() / (ms * 1e-3) / 1e9, "unit": "GB/s", "ms_per_step": ms, "dtype": "u8",
                     "config": {"workload": "copy: torch copy_ of 1 GiB (reads 1 GiB, writes 1 GiB)"}})
        print(json.dumps(line))
        return
    if args.workload == "c4_sweep":
        sweep = bench_c4_sweep(args.steps, args.warmup, device)
        unit = next((pt for pt in sweep["points"] if pt["q_scale"] == 1.0), sweep["points"][-1])
        line.update({"value": unit["frac_mfma_peak"] * MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s", "ms_per_step": unit["ms"],
                     "dtype": "bf16", "config": {"workload": "c4_sweep: the headline shapes with q scaled by 0.25 .. 2"},
                     "extra": {"c4_sweep": sweep}})
        print(json.dumps(line))
        return
    if args.workload == "c2_bwd":
        rows = bench_rows_backward(args.steps, args.warmup, device)
        best = rows["f32_alpha1.5"]
        line.update({"value": best["GBps"], "unit": "GB/s", "ms_per_step": best["ms"], "dtype": "f32",
                     "config": {"workload": "c2_bwd: entmax rows backward [16384, 8192] fp32 alpha=1.5"},
                     "roofline": {"bound": "hbm", "achieved": best["GBps"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                  "frac": best["frac_hbm_peak"], "traffic": MEASURED_HBM_TRAFFIC_BYTES.get("c2_bwd_f32"),
                                  "kernel": "entmax_rows_bwd_reg_kernel", "bytes_per_launch": best["bytes"]},
                     "extra": {"entmax_rows_backward": rows}})
    elif args.workload == "c2":
        rows = bench_rows(args.steps, args.warmup, device)
        best = rows["f32_alpha1.5"]
        line.update({"value": best["GBps"], "unit": "GB/s", "ms_per_step": best["ms"], "dtype": "f32",
                     "config": {"workload": "c2: entmax rows [16384, 8192] fp32 alpha=1.5, hist init, n_iter=2"},
                     "roofline": {"bound": "hbm", "achieved": best["GBps"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                  "frac": best["frac_hbm_peak"], "traffic": MEASURED_HBM_TRAFFIC_BYTES["c2_f32"],
                                  "kernel": "entmax_rows_reg_kernel", "bytes_per_launch": best["bytes"]},
                     "extra": {"entmax_rows": rows}})
    else:
        bwd = args.workload.endswith("_bwd")
        res = bench_attention(args.workload[:2], args.steps, args.warmup, device, backward=bwd)
        line.update({"value": res["eff_tflops"], "unit": "TFLOP/s", "ms_per_step": res["ms_per_step"],
                     "dtype": "bf16", "config": res["config"],
                     "roofline": {"bound": "mfma", "achieved": res["eff_tflops"], "peak": MFMA_BF16_PEAK_TFLOPS,
                                  "unit": "TFLOP/s", "frac": res["frac_mfma_peak"],
                                  "traffic": MEASURED_HBM_TRAFFIC_BYTES.get(args.workload),
                                  "kernel": BWD_KERNELS[args.workload] if bwd else FWD_KERNELS[args.workload],
                                  "flops_per_launch": res["flops_per_step"]},
                     "extra": {k: v for k, v in res.items() if k.startswith("tiles") or k in ("wall_ms_per_step", "forward_keeping_supports")}})
        if bwd and args.workload != "c3_bwd":
            # with the supports kept the sparse kernels issue no matrix products at all: the dense-equivalent rate
            # says how fast a dense implementation would have to be, and may exceed the matrix pipe's peak
            line["roofline"]["note"] = ("dense-equivalent FLOPs over time; the sparse-support kernels do this work on "
                                        "the vector pipe and are bound by their gathers, so frac is not a utilisation")
        if "tiles" in res:
            line["tiles"] = res["tiles"]
        if not args.no_extra:
            del res
            torch.cuda.empty_cache()
            line["extra"]["entmax_rows"] = bench_rows(args.steps, args.warmup, device)
            line["extra"]["entmax_rows_backward"] = bench_rows_backward(args.steps, args.warmup, device)
            if args.workload == "c4":
                for other in ("c3", "c5"):
                    r = bench_attention(other, args.steps, args.warmup, device)
                    line["extra"][other] = {k: r[k] for k in r if k != "wall_ms_per_step"}
                    line["extra"][other]["kernel"] = FWD_KERNELS[other]
                    del r
                    torch.cuda.empty_cache()
                line["extra"]["c4_sweep"] = bench_c4_sweep(args.steps // 2, 5, device)
                torch.cuda.empty_cache()
                b = bench_attention("c4", max(3, args.steps // 2), 5, device, backward=True)
                line["extra"]["attention_backward"] = {k: b[k] for k in ("ms_per_step", "eff_tflops", "frac_mfma_peak",
                                                                         "flops_per_step", "steps", "warmup")}
                line["extra"]["attention_backward"]["supports_kept_bytes"] = b["config"]["supports_kept_bytes"]
                del b
                torch.cuda.empty_cache()
    if not args.no_extra:
        line["cpu_baseline"] = cpu_baseline()
    print(json.dumps(line))


if __name__ == "__main__":
    main()
