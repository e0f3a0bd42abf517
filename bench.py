#!/usr/bin/env python3
"""Benchmark of the IVFPQ search hot path on one MI355X.

A "step" is one search of the whole query batch (coarse probe -> LUT -> ADC scan -> top-k) with
queries and results resident in HBM.  Default workload: 10M x 128-d float32 L2, Gaussian mixture of
1024 components (sigma 0.25), trained on a 500k sample, nlist=16384, M=32 x 8 bit, 10k queries,
nprobe=64, k=100, fp32 LUT.  Prints ONE JSON line.
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0


def log(msg):
    print(f"[bench] {msg}", file=sys.stderr, flush=True)


def gen_mixture_gpu(torch, seed, n, d, comp, sigma, centres=None, chunk=1 << 20):
    """Gaussian-mixture rows generated on the device in chunks (centres ~ N(0, I))."""
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    if centres is None:
        centres = torch.randn(comp, d, generator=g, device="cuda", dtype=torch.float32)
    out = torch.empty(n, d, device="cuda", dtype=torch.float32)
    for s in range(0, n, chunk):
        e = min(n, s + chunk)
        which = torch.randint(0, comp, (e - s,), generator=g, device="cuda")
        out[s:e] = centres[which] + sigma * torch.randn(e - s, d, generator=g, device="cuda", dtype=torch.float32)
    return out, centres


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--n", type=int, default=10_000_000, help="base vectors (default: the 10M workload)")
    ap.add_argument("--nq", type=int, default=10_000)
    ap.add_argument("--ntrain", type=int, default=500_000)
    ap.add_argument("--nlist", type=int, default=16384)
    ap.add_argument("--nprobe", type=int, default=64)
    ap.add_argument("--k", type=int, default=100)
    ap.add_argument("--niter", type=int, default=10, help="k-means iterations used to build the index")
    ap.add_argument("--layout", type=int, default=-1)
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="target CPU time of the baseline sample")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run a 1 GiB plain copy kernel (yardstick for rocprofv3 traffic counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures ONE GPU: this build has no multi-GPU path (one MI355X holds the whole index); "
              "run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch

    import indexsdk_amd as ix
    from indexsdk_amd import _capi

    if not torch.cuda.is_available():
        print("bench.py needs a GPU (no CPU fallback exists)", file=sys.stderr)
        sys.exit(2)
    lib = _capi.load()
    d, M, comp, sigma = 128, 32, 1024, 0.25
    n, nq, k, nprobe, nlist = args.n, args.nq, args.k, args.nprobe, args.nlist

    t0 = time.time()
    base, centres = gen_mixture_gpu(torch, 1236, n, d, comp, sigma)
    queries, _ = gen_mixture_gpu(torch, 99, nq, d, comp, sigma, centres=centres)
    train = base[torch.randperm(n, device="cuda", generator=torch.Generator(device="cuda").manual_seed(5))[
        : min(args.ntrain, n)]].contiguous()
    torch.cuda.synchronize()
    log(f"data on device in {time.time() - t0:.1f}s")

    cfg = ix.AscendIndexIVFPQConfig(niter=args.niter, train_samples_per_list=1 << 20, code_layout=args.layout)
    index = ix.AscendIndexIVFPQ(d, ix.METRIC_L2, nlist, M, 8, cfg)
    t0 = time.time()
    _capi.check(lib.ivfpq_train_device(index._h, train.shape[0], ctypes.c_void_p(train.data_ptr())))
    log(f"trained (nlist={nlist}, M={M}, {train.shape[0]} samples, {args.niter} iters) in {time.time() - t0:.1f}s")
    t0 = time.time()
    _capi.check(lib.ivfpq_add_with_ids_device(index._h, n, ctypes.c_void_p(base.data_ptr()), None))
    t_add = time.time() - t0
    log(f"added {n} vectors in {t_add:.1f}s ({n / t_add / 1e6:.2f} M vec/s)")
    del base, train
    torch.cuda.empty_cache()
    index.setNumProbes(nprobe)

    D = torch.empty(nq, k, device="cuda", dtype=torch.float32)
    I = torch.empty(nq, k, device="cuda", dtype=torch.int64)

    def step():
        _capi.check(lib.ivfpq_search_device(index._h, nq, ctypes.c_void_p(queries.data_ptr()), k,
                                            ctypes.c_void_p(D.data_ptr()), ctypes.c_void_p(I.data_ptr())))

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    scan_ms, coarse_ms = [], []
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
        s = index.last_search_stats()
        scan_ms.append(s["ms_scan"])
        coarse_ms.append(s["ms_coarse"])
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    stats = index.last_search_stats()
    ms_per_step = elapsed / args.steps * 1e3
    qps = nq * args.steps / elapsed
    scan_bytes = stats["scanned_codes"] * M          # algorithmic bytes: code bytes only
    scan_ms_avg = float(np.mean(scan_ms))
    achieved = scan_bytes / (scan_ms_avg * 1e-3) / 1e9
    log(f"step {ms_per_step:.3f} ms (coarse {np.mean(coarse_ms):.3f} ms, scan {scan_ms_avg:.3f} ms), "
        f"{qps:.0f} QPS, scan {achieved:.0f} GB/s")

    if args.copy_probe:
        src = torch.zeros(1 << 28, device="cuda", dtype=torch.float32)
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        _capi.check(lib.ixa_copy_probe(ctypes.c_void_p(src.data_ptr()), ctypes.c_void_p(dst.data_ptr()), 1 << 30))
        del src, dst

    result = {
        "metric": "queries/sec and ADC-scan GB/s (% HBM peak) at k=100 on 1 MI355X",
        "value": qps, "unit": "queries/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "u8 codes -> f32 LUT sums", "data": "synthetic",
        "config": {"workload": f"IVFPQ L2 {n}x{d} f32, {comp}-component Gaussian mixture sigma {sigma}, "
                               f"nlist={nlist}, M={M}x8bit, nq={nq}, nprobe={nprobe}, k={k}, fp32 LUT",
                   "code_layout": "rot32" if (args.layout != 0) else "row", "ntrain": int(min(args.ntrain, n)),
                   "kmeans_iters": args.niter},
        "adc_scan_GBps": achieved, "adc_scan_pct_hbm_peak": 100.0 * achieved / HBM_PEAK_GBPS,
        "ms_coarse": float(np.mean(coarse_ms)), "ms_scan": scan_ms_avg, "scanned_codes_per_step": stats["scanned_codes"],
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBPS, "traffic": None,
                     "kernel": "ivfpq_scan_kernel", "bytes_per_launch": scan_bytes, "ms_per_launch": scan_ms_avg},
    }

    if not args.no_cpu:
        from oracle import oracle as orc
        t0 = time.time()
        cent, cb = index.get_trained()
        lens = np.array([index.getListLength(l) for l in range(nlist)], dtype=np.int64)
        off = np.zeros(nlist + 1, dtype=np.int64)
        np.cumsum(lens, out=off[1:])
        codes = np.empty((int(off[-1]), M), dtype=np.uint8)
        ids = np.empty(int(off[-1]), dtype=np.int64)
        for l in range(nlist):
            if lens[l]:
                c, i = index.getListCodesAndIds(l)
                codes[off[l]:off[l + 1]] = c
                ids[off[l]:off[l + 1]] = i
        ref = orc.CsrIndex(d, M, orc.METRIC_L2, cent, cb, off, codes, ids)
        log(f"index copied to host for the CPU baseline in {time.time() - t0:.1f}s")
        qh = queries.cpu().numpy()
        probe_n = min(nq, 200)
        t0 = time.perf_counter()
        Dr, Ir = ref.search(qh[:probe_n], k, nprobe)
        t_probe = time.perf_counter() - t0
        sample = int(min(nq, max(probe_n, args.cpu_seconds / max(t_probe / probe_n, 1e-9))))
        t0 = time.perf_counter()
        Dr, Ir = ref.search(qh[:sample], k, nprobe)
        t_cpu = time.perf_counter() - t0
        cpu_qps = sample / t_cpu
        Ih, Dh = I[:sample].cpu().numpy(), D[:sample].cpu().numpy()
        same = float((Ih == Ir).mean())
        dist_ok = bool(np.all(np.abs(Dh - Dr) <= 1e-4 * np.maximum(np.abs(Dr), 1e-30)))
        log(f"CPU oracle: {sample} queries in {t_cpu:.2f}s on {orc.num_threads()} threads = {cpu_qps:.0f} QPS; "
            f"GPU ids equal at {same:.6f} of positions, distances within 1e-4: {dist_ok}")
        result["cpu_baseline"] = {"value": cpu_qps, "unit": "queries/s", "cores": orc.num_threads(), "kind": "port",
                                  "sample": f"first {sample} of the {nq} queries, same index, OpenMP over queries, "
                                            f"{t_cpu:.1f}s", "adc_scan_GBps": ref.last_scanned * M / t_cpu / 1e9}
        result["parity_sample"] = {"queries": sample, "ids_equal_frac": same, "dist_within_1e-4": dist_ok}
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
