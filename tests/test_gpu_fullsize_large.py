"""The two large IVFPQ configurations at their full sizes, through properties that need no full-size
reference run, plus oracle parity on a sample of the queries against the index copied back to the host:

* inner product on unit vectors: 20M x 768, nlist 32768, M 96, fp16 LUT, 4096 queries, nprobe 128, k 100
  (half LUT under the `rot32` code layout; tolerance 1e-2);
* large k over skewed lists: 100M x 96 with Zipf(1.1) cluster sizes, nlist 65536, M 48, 1024 queries,
  nprobe 256, k 1024 (shared selection pool, `xor48` code layout, queries ordered by work; tolerance 1e-4).

The base is generated on the device in chunks and added from device memory, so the raw vectors are never
resident at once (61 GB and 38 GB of float32)."""
import ctypes

import numpy as np
import pytest

from tests.parity import assert_topk_parity

pytestmark = pytest.mark.gpu


def _mixture(torch, gen, n, centres, sigma, weights, unit, out):
    """Rows of a Gaussian mixture written into out[:n] (device tensor), 1M rows at a time."""
    comp = centres.shape[0]
    for s in range(0, n, 1 << 20):
        e = min(n, s + (1 << 20))
        if weights is None:
            which = torch.randint(0, comp, (e - s,), generator=gen, device="cuda")
        else:
            which = torch.multinomial(weights, e - s, replacement=True, generator=gen)
        out[s:e] = centres[which] + sigma * torch.randn(e - s, centres.shape[1], generator=gen, device="cuda")
        if unit:
            out[s:e] /= out[s:e].norm(dim=1, keepdim=True)
    return out[:n]


def _build(n, d, comp, sigma, nlist, M, metric_name, lut_fp16, ntrain, nq, seed, zipf=None, unit=False, keep=0):
    import torch

    import indexsdk_amd as ix
    from indexsdk_amd import _capi
    lib = _capi.load()
    gen = torch.Generator(device="cuda")
    gen.manual_seed(seed)
    centres = torch.randn(comp, d, generator=gen, device="cuda")
    if unit:
        centres /= centres.norm(dim=1, keepdim=True)
    weights = None
    if zipf:
        weights = 1.0 / torch.arange(1, comp + 1, device="cuda", dtype=torch.float64) ** zipf
        weights = (weights / weights.sum()).float()
    metric = ix.METRIC_L2 if metric_name == "L2" else ix.METRIC_INNER_PRODUCT
    cfg = ix.AscendIndexIVFPQConfig(niter=4, train_samples_per_list=1 << 20, lut_fp16=lut_fp16,
                                    spherical=1 if metric == ix.METRIC_INNER_PRODUCT else 0)
    index = ix.AscendIndexIVFPQ(d, metric, nlist, M, 8, cfg)
    train = _mixture(torch, gen, ntrain, centres, sigma, weights, unit, torch.empty(ntrain, d, device="cuda"))
    torch.cuda.synchronize()
    _capi.check(lib.ivfpq_train_device(index._h, ntrain, ctypes.c_void_p(train.data_ptr())))
    del train
    rows = max(1 << 20, (2 << 30) // (4 * d))
    buf = torch.empty(min(rows, n), d, device="cuda")
    kept = None
    for s in range(0, n, rows):
        e = min(n, s + rows)
        _mixture(torch, gen, e - s, centres, sigma, weights, unit, buf)
        torch.cuda.synchronize()
        if s == 0 and keep:
            kept = buf[:keep].cpu().numpy()               # database vectors 0..keep-1, used as queries later
        _capi.check(lib.ivfpq_add_with_ids_device(index._h, e - s, ctypes.c_void_p(buf.data_ptr()), None))
    q = _mixture(torch, gen, nq, centres, sigma, weights, unit, torch.empty(nq, d, device="cuda")).cpu().numpy()
    del buf
    torch.cuda.empty_cache()
    return ix, index, q, kept


def _host_copy(oracle, ix, index, d, M, nlist, n):
    cent, cb = index.get_trained()
    lens = np.array([index.getListLength(l) for l in range(nlist)], dtype=np.int64)
    assert lens.sum() == n
    off = np.zeros(nlist + 1, dtype=np.int64)
    np.cumsum(lens, out=off[1:])
    codes = np.empty((n, M), dtype=np.uint8)
    ids = np.empty(n, dtype=np.int64)
    for l in np.flatnonzero(lens):
        codes[off[l]:off[l + 1]], ids[off[l]:off[l + 1]] = index.getListCodesAndIds(int(l))
    seen = np.zeros(n, dtype=bool)
    seen[ids] = True
    assert seen.all()                                     # every id 0..n-1 exactly once
    return oracle.CsrIndex(d, M, index.metric_type, cent, cb, off, codes, ids), lens


def _properties(index, q, k, nprobe, fewer, n, lens, best_is_smallest):
    Dm, Im = index.search(q, k)
    st = index.last_search_stats()
    real = Im >= 0
    assert (Im[real] < n).all()
    # padding only at the end of a row, and with the sentinel of the metric
    assert (np.diff(real.astype(np.int8), axis=1) <= 0).all()
    sentinel = np.float32(np.finfo(np.float32).max) * (1 if best_is_smallest else -1)
    assert (Dm[~real] == sentinel).all()
    step = np.diff(Dm, axis=1)
    assert (step >= 0).all() if best_is_smallest else (step <= 0).all()       # best first
    srt = np.sort(np.where(real, Im, -1 - np.arange(Im.shape[1])[None, :]), axis=1)
    assert (np.diff(srt, axis=1) > 0).all()                                    # no id twice
    D2, I2 = index.search(q, k)                                                # idempotence
    assert np.array_equal(I2, Im) and np.array_equal(D2.view(np.uint32), Dm.view(np.uint32))
    D10, I10 = index.search(q, 10)                                             # k = 10 is a prefix
    assert np.array_equal(I10, Im[:, :10]) and np.array_equal(D10.view(np.uint32), Dm[:, :10].view(np.uint32))
    probes, _ = index.coarse_probe(q)
    assert (np.diff(np.sort(probes, axis=1), axis=1) > 0).all()                # no list twice
    assert st["scanned_codes"] == lens[probes].sum()
    # a row is padded exactly when its probed lists hold fewer than k vectors
    assert np.array_equal(real.sum(axis=1), np.minimum(lens[probes].sum(axis=1), k))
    index.setNumProbes(fewer)                                                  # fewer probes: k-th never better
    Df, _ = index.search(q, k)
    index.setNumProbes(nprobe)
    assert (Df[:, k - 1] >= Dm[:, k - 1]).all() if best_is_smallest else (Df[:, k - 1] <= Dm[:, k - 1]).all()
    return Dm, Im


def test_full_size_inner_product_half_lut(oracle):
    n, d, nlist, M, nq, nprobe, k = 20_000_000, 768, 32768, 96, 4096, 128, 100
    ix, index, q, _ = _build(n, d, 4096, 0.05, nlist, M, "IP", 1, 1_310_720, nq, seed=1237, unit=True)
    index.setNumProbes(nprobe)
    assert index.ntotal == n
    ref, lens = _host_copy(oracle, ix, index, d, M, nlist, n)
    Dm, Im = _properties(index, q, k, nprobe, 32, n, lens, best_is_smallest=False)
    sel = np.arange(0, nq, 16)
    Dr, Ir = ref.search(q[sel], k, nprobe, lut_fp16=True)
    exempt = assert_topk_parity(oracle, ref, q[sel], Dm[sel], Im[sel], Dr, Ir, 1e-2, lut_fp16=True)
    assert exempt <= 0.002 * Ir.size + 5
    pi, pd = index.coarse_probe(q[sel])
    oi, od = oracle.coarse_probe(q[sel], ref.cent, nprobe, ix.METRIC_INNER_PRODUCT)
    assert np.array_equal(pi, oi) and np.array_equal(pd.view(np.uint32), od.view(np.uint32))


def test_full_size_large_k_over_skewed_lists(oracle):
    n, d, nlist, M, nq, nprobe, k = 100_000_000, 96, 65536, 48, 1024, 256, 1024
    ix, index, q, kept = _build(n, d, 256, 0.25, nlist, M, "L2", 0, 2_621_440, nq, seed=1239, zipf=1.1, keep=1000)
    index.setNumProbes(nprobe)
    assert index.ntotal == n
    ref, lens = _host_copy(oracle, ix, index, d, M, nlist, n)
    print(f"list lengths: mean {lens.mean():.0f}, max {lens.max()}, empty {(lens == 0).sum()}", flush=True)
    assert lens.max() > 2 * lens.mean()                                        # the lists really are skewed
    Dm, Im = _properties(index, q, k, nprobe, 64, n, lens, best_is_smallest=True)
    sel = np.arange(0, nq, 8)
    Dr, Ir = ref.search(q[sel], k, nprobe)
    exempt = assert_topk_parity(oracle, ref, q[sel], Dm[sel], Im[sel], Dr, Ir, 1e-4, lut_fp16=False)
    assert exempt <= 0.01 * Ir.size + 5
    pi, pd = index.coarse_probe(q[sel])
    oi, od = oracle.coarse_probe(q[sel], ref.cent, nprobe, ix.METRIC_L2)
    assert np.array_equal(pi, oi) and np.array_equal(pd.view(np.uint32), od.view(np.uint32))
    # database vectors as queries: a vector's own code minimises every term of its ADC sum and its own list
    # is its first probe, so it comes back first unless another vector of a probed list has the same code
    # (FR/test/ascend/TestAscendIndexIVFPQ.cpp:150-166)
    Ds, Is = index.search(kept, 5)
    own = np.arange(len(kept))
    for i in np.flatnonzero(Is[:, 0] != own):
        at = np.flatnonzero(Is[i] == own[i])
        if len(at):
            assert Ds[i, at[0]] == Ds[i, 0]
        else:                                              # six or more vectors share the code
            assert Ds[i, 4] == Ds[i, 0]
