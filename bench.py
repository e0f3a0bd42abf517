#!/usr/bin/env python3
"""Benchmark of the IVFPQ search hot path on one MI355X.

A "step" is one search of the whole query batch (coarse probe -> LUT -> ADC scan -> top-k) with
queries and results resident in HBM.  Default workload: 10M x 128-d float32 L2, Gaussian mixture of
1024 components (sigma 0.25), trained on a 500k sample, nlist=16384, M=32 x 8 bit, 10k queries,
nprobe=64, k=100, fp32 LUT.  Prints ONE JSON line.
"""
import argparse
import ctypes
import hashlib
import json
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0


def log(msg):
    print(f"[bench] {msg}", file=sys.stderr, flush=True)


PROFILES = os.path.join(ROOT, "profiles")
SCAN_SOURCES = ("scan.hip", "scan.h", "topk.h")
FLAT_I8_SOURCES = ("flat_i8.hip", "flat_i8.h", "resident_tile.h")


def source_hash(names):
    """sha256 over kernel sources: a counter figure measured on other sources is stale."""
    h = hashlib.sha256()
    for name in names:
        with open(os.path.join(ROOT, "indexsdk_amd", "csrc", name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()


def scan_source_hash():
    return source_hash(SCAN_SOURCES)


def tracked_lines(tag):
    """Every line `<tag>: key=value ...` of the tracked profiles, as (file name, dict)."""
    out = []
    try:
        names = sorted(os.listdir(PROFILES))
    except OSError:
        return out
    for name in names:
        if not name.endswith(".md"):
            continue
        try:
            text = open(os.path.join(PROFILES, name)).read()
        except OSError:
            continue
        for m in re.finditer(r"^%s:(.*)$" % re.escape(tag), text, re.M):
            try:
                out.append((name, dict(item.split("=", 1) for item in m.group(1).split())))
            except ValueError:
                pass
    return out


def measured_traffic(workload, layout_name, locality, lut_fp16, overridden):
    """HBM bytes per byte of scanned code and bytes written per launch, as the rocprofv3 FETCH_SIZE / WRITE_SIZE
    runs recorded in a tracked profile found them -- or None when no profile was taken on this workload with these
    knobs and these kernel sources (the `bench-traffic:` line it is read from names all of them)."""
    if overridden:
        return None
    for name, kv in tracked_lines("bench-traffic"):
        same = (kv.get("workload") == workload and kv.get("layout") == layout_name and
                kv.get("locality") == str(locality) and kv.get("lut") == ("fp16" if lut_fp16 else "fp32") and
                kv.get("scan_source_sha256") == scan_source_hash())
        if same:
            return float(kv["fetch_per_algorithmic_byte"]), float(kv["write_bytes"]), "profiles/" + name
    return None


def measured_issue(workload, layout_name, lut_fp16, overridden):
    """What the SQ counters of a tracked profile say bounds the scan kernel of this workload (`bench-issue:` line,
    same keys as `bench-traffic:`): VALU issue time and LDS activity as fractions of the launch, the share of LDS
    cycles lost to bank conflicts, and the time the LDS gathers alone would take."""
    if overridden:
        return None
    for name, kv in tracked_lines("bench-issue"):
        if (kv.get("workload") == workload and kv.get("layout") == layout_name and
                kv.get("lut") == ("fp16" if lut_fp16 else "fp32") and kv.get("scan_source_sha256") == scan_source_hash()):
            out = {k: float(v) for k, v in kv.items() if k in ("valu_issue_frac", "lds_active_frac", "lds_conflict_frac",
                                                                "lds_floor_ms", "shader_clock_ghz")}
            out["source"] = "profiles/" + name
            return out
    return None


def cpu_model():
    """Model name of the host CPU the baseline leg runs on (/proc/cpuinfo), or "unknown"."""
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.lower().startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def gen_mixture_gpu(torch, seed, n, d, comp, sigma, centres=None, chunk=1 << 20, weights=None, unit=False,
                    out=None):
    """Mixture rows generated on the device in chunks: centres ~ N(0, I) (normalised when ``unit``),
    within-cluster N(0, sigma^2) noise, rows renormalised when ``unit``; ``weights`` skews the cluster sizes."""
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    if centres is None:
        centres = torch.randn(comp, d, generator=g, device="cuda", dtype=torch.float32)
        if unit:
            centres /= centres.norm(dim=1, keepdim=True)
    if out is None:
        out = torch.empty(n, d, device="cuda", dtype=torch.float32)
    for s in range(0, n, chunk):
        e = min(n, s + chunk)
        if weights is None:
            which = torch.randint(0, comp, (e - s,), generator=g, device="cuda")
        else:
            which = torch.multinomial(weights, e - s, replacement=True, generator=g)
        out[s:e] = centres[which] + sigma * torch.randn(e - s, d, generator=g, device="cuda", dtype=torch.float32)
        if unit:
            out[s:e] /= out[s:e].norm(dim=1, keepdim=True)
    return out, centres


# The five benchmark configurations; "C2" is the one the headline metric is quoted on.
WORKLOADS = {
    "C1": dict(n=100_000, nq=1000, d=128, comp=64, sigma=0.3, nlist=256, M=16, nprobe=16, k=10, metric="L2",
               lut_fp16=0, ntrain=100_000, seed=1235),
    "C2": dict(n=10_000_000, nq=10_000, d=128, comp=1024, sigma=0.25, nlist=16384, M=32, nprobe=64, k=100,
               metric="L2", lut_fp16=0, ntrain=500_000, seed=1236),
    "C3": dict(n=20_000_000, nq=4096, d=768, comp=4096, sigma=0.05, nlist=32768, M=96, nprobe=128, k=100,
               metric="IP", lut_fp16=1, ntrain=1_310_720, seed=1237, unit=True),
    # the shape the reference's design document states its latency targets on (10M x 128, nlist 1024, M 4, k 300,
    # batches of 1..64, nprobe 32 / 64 / 128: 880 / 1350 / 2340 us on its hardware,
    # docs/rfc/26.1.0/IVFPQ...RFC.md:84-93); `--latency-sweep` reports those cells
    "RFC": dict(n=10_000_000, nq=64, d=128, comp=1024, sigma=0.25, nlist=1024, M=4, nprobe=64, k=300,
                metric="L2", lut_fp16=0, ntrain=500_000, seed=1240),
    "C5": dict(n=100_000_000, nq=1024, d=96, comp=256, sigma=0.25, nlist=65536, M=48, nprobe=256, k=1024,
               metric="L2", lut_fp16=0, ntrain=2_621_440, seed=1239, zipf=1.1),
}


def run_flat_i8(args, torch, ix, _capi, lib, steps, warmup, cpu_leg):
    """Config 4: Flat int8, 10M x 512 uniform in [-127, 127], 2048 queries, exact int32 L2, k = 100."""
    import numpy as np
    n, nq, d, k = args.n or 10_000_000, args.nq or 2048, 512, args.k or 100
    g = torch.Generator(device="cuda")
    g.manual_seed(1238)
    index = ix.AscendIndexInt8Flat(d, ix.METRIC_L2, scratch_bytes=2 << 30)
    t0 = time.time()
    for s in range(0, n, 1 << 21):
        e = min(n, s + (1 << 21))
        chunk = torch.randint(-127, 128, (e - s, d), generator=g, device="cuda", dtype=torch.int8)
        torch.cuda.synchronize()
        _capi.check(lib.flat_i8_add_with_ids_device(index._h, e - s, ctypes.c_void_p(chunk.data_ptr()), None))
    queries = torch.randint(-127, 128, (nq, d), generator=g, device="cuda", dtype=torch.int8)
    torch.cuda.synchronize()
    log(f"flat int8 base {n}x{d} on device in {time.time() - t0:.1f}s")
    D = torch.empty(nq, k, device="cuda", dtype=torch.int32)
    I = torch.empty(nq, k, device="cuda", dtype=torch.int64)

    def step():
        _capi.check(lib.flat_i8_search_device(index._h, nq, ctypes.c_void_p(queries.data_ptr()), k,
                                              ctypes.c_void_p(D.data_ptr()), ctypes.c_void_p(I.data_ptr())))

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms = elapsed / steps * 1e3
    ops = 2.0 * nq * n * d
    stats = index.last_search_stats()
    # HBM bytes of a search as the tracked FETCH_SIZE / WRITE_SIZE runs found them, when they were taken on these
    # kernel sources
    traffic, traffic_src = None, None
    if not (args.n or args.nq or args.k):
        for name, kv in tracked_lines("bench-traffic"):
            if kv.get("workload") == "C4" and kv.get("flat_i8_source_sha256") == source_hash(FLAT_I8_SOURCES):
                traffic, traffic_src = float(kv["fetch_bytes"]) + float(kv["write_bytes"]), "profiles/" + name
    result = {
        "metric": "queries/sec (Flat int8 brute force, exact int32 L2) at k=100 on 1 MI355X",
        "value": nq * steps / elapsed, "unit": "queries/s", "n_gpus": 1, "steps": steps,
        "warmup": warmup, "ms_per_step": ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int8 -> int32", "data": "synthetic",
        "config": {"workload": f"C4 Flat int8 {n}x{d} uniform[-127,127], nq={nq}, k={k}, exact int32 L2"},
        "roofline": {"bound": "mfma", "achieved": ops / (ms * 1e-3) / 1e12, "peak": 5000.0, "unit": "TOP/s",
                     "frac": ops / (ms * 1e-3) / 1e12 / 5000.0, "traffic": traffic, "traffic_source": traffic_src,
                     "basis": "2 * nq * n * d int8 operations of the WHOLE search (seed stretch, bound-filtered score "
                              "launches, candidate merges) / wall time of a search; peak = dense int8 matrix rate at "
                              "the 2.4 GHz boost clock",
                     "kernel": "resident_i8_kernel (query tile resident in LDS) + selection kernels",
                     "device_ms": stats["ms_total"]},
    }
    if cpu_leg:
        from oracle import oracle as orc
        sample_q, sample_n = min(nq, 64), min(n, 1_000_000)
        base_h = index.getBase(0, sample_n)
        qh = queries[:sample_q].cpu().numpy()
        t0 = time.perf_counter()
        Dr, Ir = orc.flat_i8(base_h, qh, k)
        t_cpu = time.perf_counter() - t0
        # exactness on the sampled sub-problem: search the same rows on the GPU
        sub = ix.AscendIndexInt8Flat(d, ix.METRIC_L2)
        sub.add(base_h)
        Dg, Ig = sub.search_int32(qh, k)
        exact = bool(np.array_equal(Dg, Dr) and np.array_equal(Ig, Ir))
        cpu_ops = 2.0 * sample_q * sample_n * d
        result["cpu_baseline"] = {"value": sample_q / t_cpu * (sample_n / n), "unit": "queries/s", "cores": orc.num_threads(),
                                  "kind": "port", "cpu_model": cpu_model(), "host_cpus": os.cpu_count(),
                                  "sample": f"{sample_q} queries x first {sample_n} base rows in {t_cpu:.1f}s, "
                                  f"scaled by {sample_n}/{n} to the full base; {cpu_ops / t_cpu / 1e9:.1f} GOP/s"}
        result["parity_sample"] = {"queries": sample_q, "rows": sample_n, "bit_exact": exact}
        log(f"CPU oracle flat int8: {t_cpu:.2f}s for {sample_q}x{sample_n}; GPU bit-exact on the sample: {exact}")
        del sub
    log(f"C4 step {ms:.2f} ms, {result['value']:.0f} QPS, {result['roofline']['achieved']:.1f} TOP/s")
    if args.copy_probe:
        src = torch.zeros(1 << 28, device="cuda", dtype=torch.float32)
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        _capi.check(lib.ixa_copy_probe(ctypes.c_void_p(src.data_ptr()), ctypes.c_void_p(dst.data_ptr()), 1 << 30))
        del src, dst
    del index, queries, D, I
    torch.cuda.empty_cache()
    return result


def host_copy_of_lists(index, np, orc, d, M, metric, nlist, lists=None):
    """The index as the oracle's CSR structure in host memory: every list, or only `lists` (the others stay empty:
    an oracle search that probes one of them returns other results than the GPU's, and the parity check says so)."""
    cent, cb = index.get_trained()
    lens = np.zeros(nlist, dtype=np.int64)
    wanted = range(nlist) if lists is None else lists
    for l in wanted:
        lens[l] = index.getListLength(int(l))
    off = np.zeros(nlist + 1, dtype=np.int64)
    np.cumsum(lens, out=off[1:])
    codes = np.empty((int(off[-1]), M), dtype=np.uint8)
    ids = np.empty(int(off[-1]), dtype=np.int64)
    for l in wanted:
        if lens[l]:
            c, i = index.getListCodesAndIds(int(l))
            codes[off[l]:off[l + 1]] = c
            ids[off[l]:off[l + 1]] = i
    return orc.CsrIndex(d, M, metric, cent, cb, off, codes, ids)


def run_ivfpq(name, args, torch, ix, _capi, lib, steps, warmup, min_seconds, headline):
    """One IVFPQ workload: build the index from synthetic data on the device, time `steps` searches of the whole batch
    (queries and results resident in HBM), keep stepping for `min_seconds`, check a sample against the oracle.  The
    headline workload also gets the host-pointer figure, the streaming-read yardstick and the full CPU leg."""
    import numpy as np
    w = dict(WORKLOADS[name])
    for key in ("n", "nq", "ntrain", "nlist", "nprobe", "k"):
        if getattr(args, key):
            w[key] = getattr(args, key)
    if args.m:
        w["M"] = args.m
    d, M, comp, sigma = w["d"], w["M"], w["comp"], args.sigma or w["sigma"]
    n, nq, k, nprobe, nlist = w["n"], w["nq"], w["k"], w["nprobe"], w["nlist"]
    metric = ix.METRIC_L2 if w["metric"] == "L2" else ix.METRIC_INNER_PRODUCT
    unit = bool(w.get("unit"))
    weights = None
    if w.get("zipf"):
        weights = 1.0 / torch.arange(1, comp + 1, device="cuda", dtype=torch.float64) ** w["zipf"]
        weights = (weights / weights.sum()).float()

    # the base is generated and added in chunks so that the raw vectors never have to be resident at once
    t0 = time.time()
    ntrain = min(w["ntrain"], n)
    train, centres = gen_mixture_gpu(torch, w["seed"] + 7, ntrain, d, comp, sigma, weights=weights, unit=unit)
    queries, _ = gen_mixture_gpu(torch, 99, nq, d, comp, sigma, centres=centres, weights=weights, unit=unit)
    if args.same_queries:
        queries = queries[:1].repeat(nq, 1).contiguous()
    torch.cuda.synchronize()
    cfg = ix.AscendIndexIVFPQConfig(niter=args.niter, train_samples_per_list=1 << 20, code_layout=args.layout,
                                    lut_fp16=w["lut_fp16"], scan_locality=args.locality, spherical=1 if metric == ix.METRIC_INNER_PRODUCT else 0,
                                    **({"scratch_bytes": args.scratch_mb << 20} if args.scratch_mb else {}))
    index = ix.AscendIndexIVFPQ(d, metric, nlist, M, 8, cfg)
    _capi.check(lib.ivfpq_train_device(index._h, ntrain, ctypes.c_void_p(train.data_ptr())))
    log(f"{name}: trained (nlist={nlist}, M={M}, {ntrain} samples, {args.niter} iters) in {time.time() - t0:.1f}s")
    del train
    t0 = time.time()
    chunk_rows = max(1 << 20, min(n, (2 << 30) // (4 * d)))
    buf = torch.empty(min(chunk_rows, n), d, device="cuda", dtype=torch.float32)
    for ci, s in enumerate(range(0, n, chunk_rows)):
        e = min(n, s + chunk_rows)
        gen_mixture_gpu(torch, w["seed"] + 1000 + ci, e - s, d, comp, sigma, centres=centres, weights=weights, unit=unit,
                        out=buf[: e - s])
        torch.cuda.synchronize()
        _capi.check(lib.ivfpq_add_with_ids_device(index._h, e - s, ctypes.c_void_p(buf.data_ptr()), None))
    t_add = time.time() - t0
    log(f"{name}: generated + added {n} vectors in {t_add:.1f}s ({n / t_add / 1e6:.2f} M vec/s)")
    del buf
    torch.cuda.empty_cache()
    index.setNumProbes(nprobe)
    index.set_stage_timings(1)   # the steps below report their coarse / scan split, whatever the batch size

    D = torch.empty(nq, k, device="cuda", dtype=torch.float32)
    I = torch.empty(nq, k, device="cuda", dtype=torch.int64)

    def step():
        _capi.check(lib.ivfpq_search_device(index._h, nq, ctypes.c_void_p(queries.data_ptr()), k,
                                            ctypes.c_void_p(D.data_ptr()), ctypes.c_void_p(I.data_ptr())))

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    scan_ms, coarse_ms = [], []
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
        ms_c, ms_s = index.last_search_timings()     # HIP events on the library's stream; no device work
        scan_ms.append(ms_s)
        coarse_ms.append(ms_c)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    stats = index.last_search_stats()
    ms_per_step = elapsed / steps * 1e3
    qps = nq * steps / elapsed
    # the K steps above are the measurement; they are followed by more of the same until min_seconds have been timed,
    # each step on its own clock, so that mean and median of a stretch at steady-state clocks stand beside it
    wall = []
    extra_scan, extra_coarse = list(scan_ms), list(coarse_ms)
    spent = elapsed
    while spent < min_seconds and len(wall) < 100000:
        t1 = time.perf_counter()
        step()
        dt = time.perf_counter() - t1
        ms_c, ms_s = index.last_search_timings()
        wall.append(dt * 1e3)
        extra_scan.append(ms_s)
        extra_coarse.append(ms_c)
        spent += dt
    tail = extra_scan[len(extra_scan) // 2:]    # the second half of the stretch: clocks have settled
    sustained = {"steps": steps + len(wall), "seconds": spent,
                 "ms_per_step_mean": (elapsed * 1e3 + sum(wall)) / (steps + len(wall)),
                 "ms_per_step_median": float(np.median(wall)) if wall else ms_per_step,
                 "ms_scan_median": float(np.median(extra_scan)), "ms_scan_mean": float(np.mean(extra_scan)),
                 "ms_scan_median_second_half": float(np.median(tail)),
                 "ms_coarse_median": float(np.median(extra_coarse))}
    scan_bytes = stats["scanned_codes"] * M          # algorithmic bytes: code bytes only
    scan_ms_avg = float(np.mean(scan_ms))
    achieved = scan_bytes / (scan_ms_avg * 1e-3) / 1e9
    log(f"{name}: step {ms_per_step:.3f} ms (coarse {np.mean(coarse_ms):.3f} ms, scan {scan_ms_avg:.3f} ms), "
        f"{qps:.0f} QPS, scan {achieved:.0f} GB/s, coarse fp32 rerun {int(stats.get('coarse_reruns', 0))}; "
        f"sustained {sustained['seconds']:.1f}s: step median {sustained['ms_per_step_median']:.3f} ms")

    layout_name = {0: "row", 1: "rot32", 2: "xor48"}[index.code_layout()]
    # HBM traffic of the scan kernel per launch: rocprofv3 FETCH_SIZE / WRITE_SIZE runs scaled by the copy probe,
    # recorded in a tracked profile together with the workload, the knobs and the hash of the kernel's sources
    # they were taken on.  Anything else than exactly that gets null: a factor from another kernel is no figure.
    overridden = any(getattr(args, key) for key in ("n", "nq", "nlist", "nprobe", "k", "m", "scratch_mb")) or args.same_queries \
        or bool(args.sigma)
    locality_used = 1 if stats.get("ordered") == 2 else 0
    factors = measured_traffic(name, layout_name, locality_used, w["lut_fp16"], overridden)
    traffic = None if factors is None else factors[0] * scan_bytes + factors[1]
    issue = measured_issue(name, layout_name, w["lut_fp16"], overridden)
    frac = achieved / HBM_PEAK_GBPS
    roofline = {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": frac, "traffic": traffic,
                "basis": "achieved = ALGORITHMIC bytes (code bytes of every (query, list) visit) / launch time; "
                         "queries that share lists find part of them in L2, so the bytes that leave the fabric "
                         "(traffic) can be fewer: hbm_frac = traffic / launch time / peak",
                "hbm_GBps": None if traffic is None else traffic / (scan_ms_avg * 1e-3) / 1e9,
                "hbm_frac": None if traffic is None else traffic / (scan_ms_avg * 1e-3) / 1e9 / HBM_PEAK_GBPS,
                "traffic_source": None if factors is None else factors[2],
                "kernel": "ivfpq_scan_kernel", "bytes_per_launch": scan_bytes, "ms_per_launch": scan_ms_avg,
                "coarse_plan": int(stats.get("coarse_plan", 0))}
    if frac > 1.0 or (traffic is not None and traffic < 0.9 * scan_bytes):
        # more algorithmic bytes per second than the memory can deliver: part of them came out of the L2s, and
        # the launch is held by what the issue counters show, not by HBM
        roofline["bound_by_counters"] = "LDS gathers and VALU issue; a share of the code bytes is served by the XCD L2s " \
                                        "(cache-assisted: `frac` is not an HBM fraction, `hbm_frac` is)"
    if issue is not None:
        roofline["issue"] = issue
    result = {
        "metric": "queries/sec and ADC-scan GB/s (% HBM peak) at k=100 on 1 MI355X",
        "value": qps, "unit": "queries/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "value_basis": "whole-batch search with queries and results resident in HBM (ivfpq_search_device); the same "
                       "batch through host pointers is `host_io`",
        "dtype": "u8 codes -> f16 LUT, f32 sums" if w["lut_fp16"] else "u8 codes -> f32 LUT sums",
        "data": "synthetic" if not args.same_queries else "synthetic, DIAGNOSTIC: all queries identical (lists L2-resident)",
        "config": {"workload": f"{name}: IVFPQ {w['metric']} {n}x{d} f32, {comp}-component "
                               f"{'unit-norm ' if unit else ''}mixture sigma {sigma}"
                               f"{' Zipf(%s) sizes' % w['zipf'] if w.get('zipf') else ''}, nlist={nlist}, M={M}x8bit, "
                               f"nq={nq}, nprobe={nprobe}, k={k}, {'fp16' if w['lut_fp16'] else 'fp32'} LUT",
                   "code_layout": layout_name, "scan_order": {2: "locality", 1: "heaviest first"}.get(int(stats.get("ordered", 0)), "input"),
                   "ntrain": int(ntrain), "kmeans_iters": args.niter},
        "adc_scan_GBps": achieved, "adc_scan_pct_hbm_peak": 100.0 * achieved / HBM_PEAK_GBPS,
        "ms_coarse": float(np.mean(coarse_ms)), "ms_scan": scan_ms_avg, "scanned_codes_per_step": stats["scanned_codes"],
        "roofline": roofline, "sustained": sustained,
    }

    if headline:
        # What this GPU's memory system delivers to a plain streaming read of 8 GiB, measured in the same run: the
        # practical ceiling beside the published peak (the roofline fraction stays relative to the peak).
        probe = torch.zeros(2 << 30, device="cuda", dtype=torch.float32)
        torch.cuda.synchronize()
        probe_ms = ctypes.c_double()
        _capi.check(lib.ixa_read_probe(ctypes.c_void_p(probe.data_ptr()), probe.numel() * 4, 10, ctypes.byref(probe_ms)))
        stream_read = probe.numel() * 4 / (probe_ms.value * 1e-3) / 1e9
        del probe
        log(f"plain streaming read of 8 GiB: {stream_read:.0f} GB/s")
        roofline["streaming_read_GBps"] = stream_read
        roofline["frac_of_streaming_read"] = achieved / stream_read
        if args.copy_probe:
            src = torch.zeros(1 << 28, device="cuda", dtype=torch.float32)
            dst = torch.empty_like(src)
            torch.cuda.synchronize()
            _capi.check(lib.ixa_copy_probe(ctypes.c_void_p(src.data_ptr()), ctypes.c_void_p(dst.data_ptr()), 1 << 30))
            del src, dst

        # The same batch through the host-pointer entry point (queries and results in pageable host memory, as a
        # caller of the reference's API holds them): reported beside `value`, never as `value`.
        qh_io = queries.cpu().numpy()
        Dh_io = np.zeros((nq, k), dtype=np.float32)    # the caller's result arrays, allocated (and touched) once,
        Ih_io = np.zeros((nq, k), dtype=np.int64)      # as the reference's API has them: pageable host memory

        def host_step():
            _capi.check(lib.ivfpq_search(index._h, nq, qh_io.ctypes.data_as(ctypes.c_void_p), k,
                                         Dh_io.ctypes.data_as(ctypes.c_void_p), Ih_io.ctypes.data_as(ctypes.c_void_p)))

        host_step()
        reps = 20
        t0 = time.perf_counter()
        for _ in range(reps):
            host_step()
        host_io_ms = (time.perf_counter() - t0) / reps * 1e3
        host_c, host_s = index.last_search_timings()   # stage times of the last host-pointer search
        # the Python wrapper allocates new result arrays on every call: their first touch (page faults) is the caller's
        # cost, shown beside
        index.search(qh_io, k)
        t0 = time.perf_counter()
        for _ in range(5):
            index.search(qh_io, k)
        fresh_ms = (time.perf_counter() - t0) / 5 * 1e3
        result["host_io"] = {"ms_per_step": host_io_ms, "queries_per_s": nq / (host_io_ms * 1e-3),
                             "ms_coarse": host_c, "ms_scan": host_s,
                             "ms_per_step_fresh_result_arrays": fresh_ms,
                             "note": "ivfpq_search with host pointers (pageable numpy arrays, result arrays reused "
                                     "between calls): H2D of the queries and D2H of the results included; the "
                                     "end-to-end figure of a caller that keeps queries and results in host memory"}
        log(f"host-pointer search: {host_io_ms:.3f} ms per batch, {nq / (host_io_ms * 1e-3):.0f} QPS "
            f"(coarse {host_c:.3f} ms, scan {host_s:.3f} ms; {fresh_ms:.3f} ms when every call allocates new result "
            f"arrays)")

    if headline and args.latency_sweep:
        # one search call per cell, synchronised, 40 calls after 5 warm-up calls: the median wall time of a call
        sweep = {}
        index.set_stage_timings(-1)   # the library's default: small batches record no stage events
        for np_ in (32, 64, 128):
            if np_ > nlist:
                continue
            index.setNumProbes(np_)
            for b in (1, 2, 4, 8, 16, 32, 64):
                if b > nq:
                    continue
                qd = queries[:b].contiguous()
                qh_b = qd.cpu().numpy()
                cell = {}
                for kind in ("device", "host"):
                    ts = []
                    for it in range(45):
                        torch.cuda.synchronize()
                        t1 = time.perf_counter()
                        if kind == "device":
                            _capi.check(lib.ivfpq_search_device(index._h, b, ctypes.c_void_p(qd.data_ptr()), k,
                                                                ctypes.c_void_p(D.data_ptr()), ctypes.c_void_p(I.data_ptr())))
                        else:
                            index.search(qh_b, k)
                        ts.append((time.perf_counter() - t1) * 1e6)
                    cell[kind + "_us"] = float(np.median(ts[5:]))
                st = index.last_search_stats()
                cell["nsplit"] = int(st.get("nsplit", 0))
                sweep[f"nprobe{np_}_batch{b}"] = cell
                log(f"latency nprobe {np_:4d} batch {b:3d}: device {cell['device_us']:8.1f} us, host pointers "
                    f"{cell['host_us']:8.1f} us (nsplit {cell['nsplit']})")
        index.setNumProbes(nprobe)
        index.set_stage_timings(1)
        step()   # D and I hold the full batch again for the parity check below
        torch.cuda.synchronize()
        result["latency_sweep"] = sweep

    if not args.no_cpu:
        from oracle import oracle as orc
        from tests.parity import assert_topk_parity
        lut16 = bool(w["lut_fp16"])
        tol = 1e-2 if lut16 else 1e-4
        qh = queries.cpu().numpy()
        t0 = time.time()
        if headline:
            ref = host_copy_of_lists(index, np, orc, d, M, metric, nlist)
            sel = np.arange(nq)
        else:
            # a sample of the batch against the oracle on the lists those queries probe (the probe lists come from the
            # library and are checked like everything else: the oracle selects its own)
            sel = np.unique(np.linspace(0, nq - 1, min(nq, args.parity_queries)).astype(np.int64))
            probed, _ = index.coarse_probe(qh[sel])
            lists = np.unique(probed[probed >= 0])
            ref = host_copy_of_lists(index, np, orc, d, M, metric, nlist, lists)
        log(f"{name}: {'index' if headline else '%d probed lists' % len(lists)} copied to host for the oracle in "
            f"{time.time() - t0:.1f}s")
        qs = qh[sel]
        probe_n = min(len(sel), 200)
        t0 = time.perf_counter()
        Dr, Ir = ref.search(qs[:probe_n], k, nprobe, lut_fp16=lut16)
        t_probe = time.perf_counter() - t0
        cpu_seconds = args.cpu_seconds if headline else min(args.cpu_seconds, 2.0)
        sample = int(min(len(sel), max(probe_n, cpu_seconds / max(t_probe / probe_n, 1e-9))))
        # repeat the sample until about cpu_seconds of CPU work have been timed (the probe above ran cold and
        # overestimates a pass, so the clock decides, not a count fixed in advance); report the median pass
        times = []
        while sum(times) < cpu_seconds and len(times) < 200:
            t0 = time.perf_counter()
            Dr, Ir = ref.search(qs[:sample], k, nprobe, lut_fp16=lut16)
            times.append(time.perf_counter() - t0)
        passes = len(times)
        t_cpu = float(np.median(times))
        cpu_qps = sample / t_cpu
        rows = torch.as_tensor(sel[:sample], device="cuda")
        Ih, Dh = I[rows].cpu().numpy(), D[rows].cpu().numpy()
        same = float((Ih == Ir).mean())
        # the tie-aware rule of the parity tests: distances within tol at every rank; where ids differ, the
        # GPU's id must be a candidate whose oracle distance ties with the oracle's entry at that rank
        try:
            exempt = assert_topk_parity(orc, ref, qs[:sample], Dh, Ih, Dr, Ir, tol, lut_fp16=lut16)
            parity_ok, parity_msg = True, ""
        except AssertionError as e:
            exempt, parity_ok, parity_msg = None, False, str(e)[:200]
        log(f"{name}: CPU oracle: {sample} queries x {passes} passes, median {t_cpu:.2f}s on {orc.num_threads()} threads = "
            f"{cpu_qps:.0f} QPS; parity with the oracle (tolerance {tol}, ties exempt): {parity_ok}, ids equal at "
            f"{same:.6f} of positions, {exempt} positions differ between tied candidates {parity_msg}")
        result["cpu_baseline"] = {"value": cpu_qps, "unit": "queries/s", "cores": orc.num_threads(), "kind": "port",
                                  "cpu_model": cpu_model(), "host_cpus": os.cpu_count(),
                                  "sample": f"{sample} of the {nq} queries ({'the first' if headline else 'evenly spaced'}), same "
                                            f"index, OpenMP over queries, median of {passes} passes of {t_cpu:.1f}s",
                                  "adc_scan_GBps": ref.last_scanned * M / t_cpu / 1e9}
        result["parity_sample"] = {"queries": sample, "rule": "tests/parity.py: distances within tol at every rank, "
                                   "id differences only between candidates whose oracle distances tie within tol",
                                   "ok": parity_ok, "ids_equal_frac": same, "tie_exempt_positions": exempt,
                                   "dist_within_tol": parity_ok, "tol": tol}
        del ref
    del index, queries, D, I
    torch.cuda.empty_cache()
    return result


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="", choices=["", "C1", "C2", "C3", "C4", "C5", "RFC"],
                    help="run ONE benchmark configuration; without it: C2, the one the metric is quoted on, as the "
                         "headline, and the other four configurations as entries of `workloads`")
    ap.add_argument("--no-others", action="store_true", help="default run: the headline workload only")
    ap.add_argument("--n", type=int, default=0, help="override the number of base vectors")
    ap.add_argument("--nq", type=int, default=0)
    ap.add_argument("--ntrain", type=int, default=0)
    ap.add_argument("--nlist", type=int, default=0)
    ap.add_argument("--nprobe", type=int, default=0)
    ap.add_argument("--k", type=int, default=0)
    ap.add_argument("--m", type=int, default=0, help="override the number of sub-quantizers")
    ap.add_argument("--sigma", type=float, default=0.0,
                    help="override the within-cluster standard deviation of the synthetic mixture (centres are N(0, 1))")
    ap.add_argument("--min-seconds", type=float, default=5.0,
                    help="after the K timed steps, keep stepping until this much time has been measured in all "
                         "(reported under 'sustained'; 'value' stays the K steps)")
    ap.add_argument("--niter", type=int, default=10, help="k-means iterations used to build the index")
    ap.add_argument("--layout", type=int, default=-1)
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="target CPU time of the baseline sample")
    ap.add_argument("--parity-queries", type=int, default=64,
                    help="queries of each `workloads` entry that are checked against the oracle")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--locality", type=int, default=-1,
                    help="scan workgroups ordered by locality: 1, 0, -1 = library default")
    ap.add_argument("--scratch-mb", type=int, default=0,
                    help="score scratch of the coarse stage in MiB (the reference's resourceSize); 0 = library default")
    ap.add_argument("--same-queries", action="store_true",
                    help="diagnostic: every query is a copy of the first, so the scanned lists stay in L2 "
                         "(the scan kernel's own ceiling, without HBM); not the benchmark")
    ap.add_argument("--latency-sweep", action="store_true",
                    help="also report the median latency of one search call for batches of 1..64 queries at "
                         "nprobe 32 / 64 / 128 (device-resident queries and results, and through host pointers)")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run a 1 GiB plain copy kernel (yardstick for rocprofv3 traffic counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures ONE GPU: this build has no multi-GPU path (one MI355X holds the whole index); "
              "run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch

    import indexsdk_amd as ix
    from indexsdk_amd import _capi

    if not torch.cuda.is_available():
        print("bench.py needs a GPU (no CPU fallback exists)", file=sys.stderr)
        sys.exit(2)
    lib = _capi.load()
    if args.workload == "C4":
        result = run_flat_i8(args, torch, ix, _capi, lib, args.steps, args.warmup, not args.no_cpu)
    elif args.workload:
        result = run_ivfpq(args.workload, args, torch, ix, _capi, lib, args.steps, args.warmup, args.min_seconds, True)
    else:
        result = run_ivfpq("C2", args, torch, ix, _capi, lib, args.steps, args.warmup, args.min_seconds, True)
        overridden = any(getattr(args, key) for key in ("n", "nq", "ntrain", "nlist", "nprobe", "k", "m")) or args.sigma
        if not args.no_others and not overridden and not args.same_queries:
            # the other four configurations, each built and timed in this same run: fewer steps, a second of sustained
            # stepping, a sample of the queries against the oracle
            others = {}
            for name in ("C1", "C3", "C4", "C5"):
                t0 = time.time()
                if name == "C4":
                    r = run_flat_i8(args, torch, ix, _capi, lib, 5, 2, not args.no_cpu)
                else:
                    r = run_ivfpq(name, args, torch, ix, _capi, lib, 20 if name == "C1" else 10, 3,
                                  min(args.min_seconds, 1.0), False)
                r["queries_per_s"] = r.pop("value")
                for key in ("metric", "unit", "n_gpus", "higher_is_better", "scaling", "vs_baseline", "data", "value_basis"):
                    r.pop(key, None)
                r["wall_seconds_incl_build"] = time.time() - t0
                others[name] = r
            result["workloads"] = others
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
