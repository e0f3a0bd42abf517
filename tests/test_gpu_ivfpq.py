"""GPU parity tests of the IVFPQ path: HIP library (through the C ABI) against the CPU oracle.

Bars: coarse assignment, probe lists and PQ codes bit-exact; distances within 1e-4 relative with
an fp32 LUT (1e-2 with an fp16 LUT); top-k ids identical except where oracle distances tie within
that tolerance.
"""
import numpy as np
import pytest

from tests.parity import FLT_MAX, assert_topk_parity

pytestmark = pytest.mark.gpu

TOL_FP32 = 1e-4
TOL_FP16 = 1e-2


@pytest.fixture(scope="module")
def ix():
    import indexsdk_amd
    return indexsdk_amd


def make_data(seed, n, nq, d, comp=32, sigma=0.3):
    rng = np.random.default_rng(seed)
    centres = rng.standard_normal((comp, d)).astype(np.float32)
    x = (centres[rng.integers(0, comp, n)] + sigma * rng.standard_normal((n, d))).astype(np.float32)
    q = (centres[rng.integers(0, comp, nq)] + sigma * rng.standard_normal((nq, d))).astype(np.float32)
    return x, q


def build_pair(ix, oracle, seed, n, nq, d, nlist, M, metric, layout=-1, lut_fp16=0, niter=4):
    """Oracle-trained quantizers injected into both sides; base added through the GPU add path."""
    x, q = make_data(seed, n, nq, d)
    if metric == ix.METRIC_INNER_PRODUCT:
        x /= np.linalg.norm(x, axis=1, keepdims=True)
        q /= np.linalg.norm(q, axis=1, keepdims=True)
    cent, _ = oracle.kmeans(x[: min(n, 20 * nlist)], nlist, niter=niter, seed=seed)
    cb = oracle.train_pq(x[: min(n, 5000)], M, niter=niter, seed=seed)
    ids = np.random.default_rng(seed + 1).permutation(10 * n)[:n].astype(np.int64)
    ref = oracle.CsrIndex.build(d, M, metric, cent, cb, x, ids)
    cfg = ix.AscendIndexIVFPQConfig(code_layout=layout, lut_fp16=lut_fp16)
    gpu = ix.AscendIndexIVFPQ(d, metric, nlist, M, 8, cfg)
    gpu.set_trained(cent, cb)
    gpu.add_with_ids(x, ids)
    return gpu, ref, x, q, ids


def test_assign_encode_lists_bit_exact(ix, oracle):
    gpu, ref, x, q, ids = build_pair(ix, oracle, 21, 20000, 10, 128, 64, 16, ix.METRIC_L2)
    assert gpu.ntotal == 20000
    assert np.array_equal(gpu.assign(x[:3000]), oracle.assign(x[:3000], ref.cent))
    assert np.array_equal(gpu.encode(x[:3000]), oracle.pq_encode(x[:3000], ref.codebook))
    total = 0
    for l in range(ref.nlist):
        codes, lid = gpu.getListCodesAndIds(l)
        b, e = ref.list_off[l], ref.list_off[l + 1]
        assert gpu.getListLength(l) == e - b
        assert np.array_equal(lid, ref.ids[b:e]), f"list {l}: ids / insertion order differ"
        assert np.array_equal(codes, ref.codes[b:e]), f"list {l}: codes differ"
        total += e - b
    assert total == 20000


@pytest.mark.parametrize("metric_name", ["L2", "IP"])
@pytest.mark.parametrize("nprobe", [1, 8, 64])
def test_coarse_probe_bit_exact(ix, oracle, metric_name, nprobe):
    metric = ix.METRIC_L2 if metric_name == "L2" else ix.METRIC_INNER_PRODUCT
    gpu, ref, x, q, ids = build_pair(ix, oracle, 22, 6000, 300, 96, 200, 8, metric)
    gpu.setNumProbes(nprobe)
    gi, gd = gpu.coarse_probe(q)
    oi, od = oracle.coarse_probe(q, ref.cent, nprobe, metric)
    assert np.array_equal(gi, oi)
    assert np.array_equal(gd.view(np.uint32), od.view(np.uint32))


@pytest.mark.parametrize("metric_name", ["L2", "IP"])
@pytest.mark.parametrize("nlist,nprobe", [(5003, 64), (5003, 150), (4096, 300), (20000, 32)])
def test_coarse_probe_bit_exact_with_thousands_of_lists(ix, oracle, metric_name, nlist, nprobe):
    """Probe selection over score rows long enough for the register-based row selection (every group
    count, a ragged last segment, two segments)."""
    metric = ix.METRIC_L2 if metric_name == "L2" else ix.METRIC_INNER_PRODUCT
    d, M, nq = 64, 8, 200
    rng = np.random.default_rng(nlist + nprobe)
    centres = rng.standard_normal((40, d)).astype(np.float32)
    cent = (centres[rng.integers(0, 40, nlist)] + 0.4 * rng.standard_normal((nlist, d))).astype(np.float32)
    q = (centres[rng.integers(0, 40, nq)] + 0.4 * rng.standard_normal((nq, d))).astype(np.float32)
    if metric == ix.METRIC_INNER_PRODUCT:
        cent /= np.linalg.norm(cent, axis=1, keepdims=True)
        q /= np.linalg.norm(q, axis=1, keepdims=True)
    cb = rng.standard_normal((M, 256, d // M)).astype(np.float32)
    gpu = ix.AscendIndexIVFPQ(d, metric, nlist, M, 8, ix.AscendIndexIVFPQConfig())
    gpu.set_trained(cent, cb)
    gpu.setNumProbes(nprobe)
    gi, gd = gpu.coarse_probe(q)
    oi, od = oracle.coarse_probe(q, cent, nprobe, metric)
    assert np.array_equal(gi, oi)
    assert np.array_equal(gd.view(np.uint32), od.view(np.uint32))
    # the search path refines only the boundary of the probe set: same set of lists
    x = (centres[rng.integers(0, 40, 30000)] + 0.4 * rng.standard_normal((30000, d))).astype(np.float32)
    if metric == ix.METRIC_INNER_PRODUCT:
        x /= np.linalg.norm(x, axis=1, keepdims=True)
    gpu.add(x)
    ref = oracle.CsrIndex.build(d, M, metric, cent, cb, x, np.arange(30000, dtype=np.int64))
    D, I = gpu.search(q, 20)
    Dr, Ir = ref.search(q, 20, nprobe)
    assert_topk_parity(oracle, ref, q, D, I, Dr, Ir, TOL_FP32)
    assert gpu.last_search_stats()["scanned_codes"] == ref.last_scanned


@pytest.mark.parametrize("d,M,nlist,layout", [(128, 16, 64, 0), (128, 32, 64, 0), (128, 32, 64, 1), (96, 48, 32, 0),
                                              (64, 8, 16, 0), (60, 12, 16, 0), (192, 96, 16, 1), (128, 64, 16, 1)])
def test_search_l2_fp32(ix, oracle, d, M, nlist, layout):
    gpu, ref, x, q, ids = build_pair(ix, oracle, 23, 12000, 150, d, nlist, M, ix.METRIC_L2, layout=layout)
    for nprobe, k in ((4, 10), (nlist, 100)):
        gpu.setNumProbes(nprobe)
        D, I = gpu.search(q, k)
        Dr, Ir = ref.search(q, k, nprobe)
        assert_topk_parity(oracle, ref, q, D, I, Dr, Ir, TOL_FP32)
        if layout == 0:
            # row layout accumulates m = 0..M-1 like the oracle: distances are bit-identical
            assert np.array_equal(D.view(np.uint32), Dr.view(np.uint32))
        assert gpu.last_search_stats()["scanned_codes"] == ref.last_scanned


def test_search_ip_fp16_lut(ix, oracle):
    gpu, ref, x, q, ids = build_pair(ix, oracle, 24, 8000, 100, 192, 32, 96, ix.METRIC_INNER_PRODUCT, lut_fp16=1)
    gpu.setNumProbes(8)
    D, I = gpu.search(q, 50)
    Dr, Ir = ref.search(q, 50, 8, lut_fp16=True)
    assert np.all(np.diff(D, axis=1) <= 0)
    assert_topk_parity(oracle, ref, q, D, I, Dr, Ir, TOL_FP16)


def test_search_ip_sums_that_cancel_to_almost_nothing(ix, oracle):
    """Inner product with one dimension per sub-quantizer: 96 terms of both signs, many results within
    1e-4 of zero.  There the association order of the fp32 sum shows at the scale of the terms, which is
    what the parity rule measures against; ids and ranks still have to match."""
    gpu, ref, x, q, ids = build_pair(ix, oracle, 31241, 300, 65, 96, 16, 96, ix.METRIC_INNER_PRODUCT, niter=2)
    gpu.setNumProbes(16)
    D, I = gpu.search(q, 1000)
    Dr, Ir = ref.search(q, 1000, 16)
    assert (np.abs(Dr[:, :300]) < 1e-4).sum() > 20           # the case is what it claims to be
    assert_topk_parity(oracle, ref, q, D, I, Dr, Ir, TOL_FP32)
    # the rule is no blank cheque: an error of 1e-3 of the terms' scale is still caught
    Dbad = D.copy()
    Dbad[0, 5] += 1e-3
    with pytest.raises(AssertionError):
        assert_topk_parity(oracle, ref, q, Dbad, I, Dr, Ir, TOL_FP32)


def test_search_sentinels_k_larger_than_candidates(ix, oracle):
    gpu, ref, x, q, ids = build_pair(ix, oracle, 25, 600, 20, 64, 32, 8, ix.METRIC_L2)
    gpu.setNumProbes(2)
    D, I = gpu.search(q, 200)
    Dr, Ir = ref.search(q, 200, 2)
    assert (Ir == -1).any()
    assert_topk_parity(oracle, ref, q, D, I, Dr, Ir, TOL_FP32)
    assert np.all(D[I == -1] == FLT_MAX)


def test_search_empty_index_and_single_query(ix, oracle):
    gpu, ref, x, q, ids = build_pair(ix, oracle, 26, 3000, 5, 64, 16, 8, ix.METRIC_L2)
    D, I = gpu.search(q[:1], 7)      # one query -> the scan splits the probes over several workgroups
    Dr, Ir = ref.search(q[:1], 7, gpu.getNumProbes())
    assert_topk_parity(oracle, ref, q[:1], D, I, Dr, Ir, TOL_FP32)
    gpu.reset()
    assert gpu.ntotal == 0 and gpu.is_trained
    D, I = gpu.search(q, 5)
    assert np.all(I == -1) and np.all(D == FLT_MAX)


def test_stage_timings_are_recorded_for_large_pages_or_on_request(ix, oracle):
    """ms_coarse / ms_scan come from events around the stages: recorded for pages of 256 queries or more, for
    smaller ones only on request (they cost a small batch several microseconds); results never depend on it."""
    gpu, ref, x, q, ids = build_pair(ix, oracle, 29, 6000, 300, 32, 16, 4, ix.METRIC_L2)
    gpu.setNumProbes(4)
    D8, I8 = gpu.search(q[:8], 5)
    assert gpu.last_search_timings() == (0.0, 0.0)
    st = gpu.last_search_stats()
    assert st["ms_total"] == 0.0 and st["scanned_codes"] > 0
    gpu.search(q, 5)
    c, s = gpu.last_search_timings()
    assert c > 0 and s > 0 and gpu.last_search_stats()["ms_scan"] > 0
    gpu.set_stage_timings(1)
    D8t, I8t = gpu.search(q[:8], 5)
    assert min(gpu.last_search_timings()) > 0
    assert np.array_equal(I8, I8t) and np.array_equal(D8.view(np.uint32), D8t.view(np.uint32))
    gpu.set_stage_timings(0)
    gpu.search(q, 5)
    assert gpu.last_search_timings() == (0.0, 0.0)
    with pytest.raises(ix.IndexSdkError):
        gpu.set_stage_timings(2)
    never = ix.AscendIndexIVFPQ(32, ix.METRIC_L2, 16, 4, 8, ix.AscendIndexIVFPQConfig(stage_timings=1))
    never.set_trained(ref.cent, ref.codebook)
    never.add_with_ids(x, ids)
    never.setNumProbes(4)
    never.search(q[:2], 5)
    assert min(never.last_search_timings()) > 0


def test_large_k(ix, oracle):
    gpu, ref, x, q, ids = build_pair(ix, oracle, 27, 30000, 40, 96, 32, 48, ix.METRIC_L2)
    gpu.setNumProbes(16)
    D, I = gpu.search(q, 1024)
    Dr, Ir = ref.search(q, 1024, 16)
    assert_topk_parity(oracle, ref, q, D, I, Dr, Ir, TOL_FP32)


def test_add_in_two_calls_add_codes_and_remove(ix, oracle):
    gpu, ref, x, q, ids = build_pair(ix, oracle, 28, 5000, 30, 64, 16, 32, ix.METRIC_L2)
    cfg = ix.AscendIndexIVFPQConfig()
    g2 = ix.AscendIndexIVFPQ(64, ix.METRIC_L2, 16, 32, 8, cfg)
    g2.set_trained(ref.cent, ref.codebook)
    g2.add_with_ids(x[:2000], ids[:2000])
    g2.add_with_ids(x[2000:], ids[2000:])
    for l in range(16):
        a, b = gpu.getListCodesAndIds(l), g2.getListCodesAndIds(l)
        assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1])
    # addPQCodes path: rebuild a third index from the raw lists
    g3 = ix.AscendIndexIVFPQ(64, ix.METRIC_L2, 16, 32, 8, cfg)
    g3.set_trained(ref.cent, ref.codebook)
    for l in range(16):
        b, e = ref.list_off[l], ref.list_off[l + 1]
        g3.add_codes(l, ref.codes[b:e], ref.ids[b:e])
    D, I = gpu.search(q, 20)
    D3, I3 = g3.search(q, 20)
    assert np.array_equal(I, I3) and np.array_equal(D, D3)
    # default ids = ntotal + i
    g4 = ix.AscendIndexIVFPQ(64, ix.METRIC_L2, 16, 32, 8, cfg)
    g4.set_trained(ref.cent, ref.codebook)
    g4.add(x[:100])
    g4.add(x[100:300])
    got = np.sort(np.concatenate([g4.getListCodesAndIds(l)[1] for l in range(16)]))
    assert np.array_equal(got, np.arange(300))
    # remove: survivors keep their order
    victims = ids[::3]
    assert gpu.remove_ids(victims) == len(victims)
    assert gpu.ntotal == 5000 - len(victims)
    vs = set(victims.tolist())
    for l in range(16):
        b, e = ref.list_off[l], ref.list_off[l + 1]
        keep = np.array([i not in vs for i in ref.ids[b:e]], dtype=bool)
        codes, lid = gpu.getListCodesAndIds(l)
        assert np.array_equal(lid, ref.ids[b:e][keep]) and np.array_equal(codes, ref.codes[b:e][keep])
    D, I = gpu.search(q, 20)
    assert not (set(I.ravel().tolist()) & vs)


def test_update_replaces_existing_and_reports_missing(ix, oracle):
    gpu, ref, x, q, ids = build_pair(ix, oracle, 35, 4000, 20, 64, 16, 8, ix.METRIC_L2)
    rng = np.random.default_rng(5)
    new_x = (x[:50] + 0.5 * rng.standard_normal((50, 64))).astype(np.float32)
    upd_ids = np.concatenate([ids[:40], np.array([10**9 + i for i in range(10)], dtype=np.int64)])
    missing = gpu.update(new_x, upd_ids)
    assert np.array_equal(missing, upd_ids[40:]) and gpu.ntotal == 4000
    # the oracle index with the same replacement: old entries removed, new ones appended to their lists
    keep = ~np.isin(ids, ids[:40])
    x2 = np.concatenate([x[keep], new_x[:40]])
    ids2 = np.concatenate([ids[keep], ids[:40]])
    ref2 = oracle.CsrIndex.build(64, 8, ix.METRIC_L2, ref.cent, ref.codebook, x2, ids2)
    for l in range(16):
        codes, lid = gpu.getListCodesAndIds(l)
        b, e = ref2.list_off[l], ref2.list_off[l + 1]
        assert np.array_equal(lid, ref2.ids[b:e]) and np.array_equal(codes, ref2.codes[b:e])
    D, I = gpu.search(new_x[:40], 1)
    assert (I[:, 0] == ids[:40]).mean() > 0.9


def test_train_on_gpu_then_parity_with_oracle_on_same_codebooks(ix, oracle):
    x, q = make_data(29, 30000, 100, 64)
    cfg = ix.AscendIndexIVFPQConfig(niter=6)
    gpu = ix.AscendIndexIVFPQ(64, ix.METRIC_L2, 128, 16, 8, cfg)
    assert not gpu.is_trained
    with pytest.raises(ix.IndexSdkError, match="not trained"):
        gpu.add(x[:10])
    gpu.train(x)
    assert gpu.is_trained
    gpu.add(x)
    cent, cb = gpu.get_trained()
    ref = oracle.CsrIndex.build(64, 16, ix.METRIC_L2, cent, cb, x)
    gpu.setNumProbes(16)
    D, I = gpu.search(q, 10)
    Dr, Ir = ref.search(q, 10, 16)
    assert_topk_parity(oracle, ref, q, D, I, Dr, Ir, TOL_FP32)
    # trained quantizer is usable: self queries come back first (reference ST invariant,
    # FR/test/ascend/TestAscendIndexIVFPQ.cpp:150-166)
    D, I = gpu.search(x[:500], 1)
    assert (I[:, 0] == np.arange(500)).mean() > 0.9
    lens = np.array([gpu.getListLength(l) for l in range(128)])
    assert lens.sum() == 30000 and (lens > 0).mean() > 0.9


def _twin(ix, oracle, seed, n, nq, d, comp, sigma, nlist, M, metric, lut_fp16, nprobe, k, zipf=None, niter=4):
    """Scaled-down twin of a benchmark configuration: trained and filled on the GPU, then the lists are
    read back through the C ABI and handed to the oracle (same quantizers, same codes, same ids)."""
    rng = np.random.default_rng(seed)
    centres = rng.standard_normal((comp, d)).astype(np.float32)
    w = None
    if zipf:
        w = 1.0 / np.arange(1, comp + 1) ** zipf
        w /= w.sum()
    unit = metric == ix.METRIC_INNER_PRODUCT
    if unit:
        centres /= np.linalg.norm(centres, axis=1, keepdims=True)

    def draw(m):
        x = centres[rng.choice(comp, m, p=w)] + sigma * rng.standard_normal((m, d)).astype(np.float32)
        if unit:
            x /= np.linalg.norm(x, axis=1, keepdims=True)
        return x.astype(np.float32)

    x, q = draw(n), draw(nq)
    cfg = ix.AscendIndexIVFPQConfig(niter=niter, lut_fp16=lut_fp16, spherical=1 if unit else 0)
    gpu = ix.AscendIndexIVFPQ(d, metric, nlist, M, 8, cfg)
    gpu.train(x[: min(n, 64 * nlist)])
    gpu.add(x)
    cent, cb = gpu.get_trained()
    lens = np.array([gpu.getListLength(l) for l in range(nlist)])
    off = np.zeros(nlist + 1, dtype=np.int64)
    np.cumsum(lens, out=off[1:])
    codes = np.empty((n, M), dtype=np.uint8)
    ids = np.empty(n, dtype=np.int64)
    for l in range(nlist):
        if lens[l]:
            codes[off[l]:off[l + 1]], ids[off[l]:off[l + 1]] = gpu.getListCodesAndIds(l)
    assert np.array_equal(np.sort(ids), np.arange(n))
    # the codes the GPU stored are the reference encoder's codes of those vectors
    probe = rng.choice(n, 2000, replace=False)
    pos = np.empty(n, dtype=np.int64)
    pos[ids] = np.arange(n)
    assert np.array_equal(codes[pos[probe]], oracle.pq_encode(x[probe], cb))
    ref = oracle.CsrIndex(d, M, metric, cent, cb, off, codes, ids)
    gpu.setNumProbes(nprobe)
    D, I = gpu.search(q, k)
    Dr, Ir = ref.search(q, k, nprobe, lut_fp16=bool(lut_fp16))
    pi, pd = gpu.coarse_probe(q)
    oi, od = oracle.coarse_probe(q, cent, nprobe, metric)
    assert np.array_equal(pi, oi) and np.array_equal(pd.view(np.uint32), od.view(np.uint32))
    exempt = assert_topk_parity(oracle, ref, q, D, I, Dr, Ir, TOL_FP16 if lut_fp16 else TOL_FP32)
    assert exempt <= 0.002 * I.size + 5
    assert gpu.last_search_stats()["scanned_codes"] == ref.last_scanned
    return lens


def test_twin_c2_l2_m32(ix, oracle):
    _twin(ix, oracle, 31, 200_000, 400, 128, 256, 0.25, 1024, 32, ix.METRIC_L2, 0, 32, 100)


def test_twin_c3_ip_m96_fp16_lut(ix, oracle):
    _twin(ix, oracle, 32, 60_000, 150, 768, 128, 0.05, 256, 96, ix.METRIC_INNER_PRODUCT, 1, 16, 100, niter=3)


def test_twin_c5_zipf_large_k(ix, oracle):
    lens = _twin(ix, oracle, 33, 300_000, 64, 96, 64, 0.25, 1024, 48, ix.METRIC_L2, 0, 64, 1024, zipf=1.1)
    assert lens.max() > 3 * np.median(lens[lens > 0])      # the lists really are imbalanced


def test_twin_c1_small(ix, oracle):
    _twin(ix, oracle, 34, 100_000, 300, 128, 64, 0.3, 256, 16, ix.METRIC_L2, 0, 16, 10, niter=6)


def test_large_k_shared_pool_one_workgroup_per_query(ix, oracle):
    """k = 1024 with enough queries that each gets a single workgroup: the workgroup-wide candidate
    pool must prune many times per query and still return exactly the oracle's top-k."""
    gpu, ref, x, q, ids = build_pair(ix, oracle, 41, 40000, 2100, 96, 16, 48, ix.METRIC_L2)
    gpu.setNumProbes(8)
    D, I = gpu.search(q, 1024)
    st = gpu.last_search_stats()
    assert st["shared_pool"] == 1 and st["nsplit"] == 1
    Dr, Ir = ref.search(q, 1024, 8)
    assert_topk_parity(oracle, ref, q, D, I, Dr, Ir, TOL_FP32)


@pytest.mark.parametrize("d,M,layout,waves", [(96, 48, 2, 16), (96, 48, 0, 16), (128, 64, 1, 16), (128, 64, 0, 16),
                                              (64, 32, 1, 16), (128, 128, 0, 8)])
def test_large_k_shared_pool_layouts_and_workgroup_sizes(ix, oracle, d, M, layout, waves):
    """The workgroup-wide pool under every code layout, with the workgroup size the LDS plan picks for
    it (sixteen wavefronts unless the LUT leaves no room for their larger pool)."""
    gpu, ref, x, q, ids = build_pair(ix, oracle, 45 + M + layout, 30000, 2100, d, 16, M, ix.METRIC_L2, layout=layout)
    gpu.setNumProbes(8)
    D, I = gpu.search(q, 1024)
    st = gpu.last_search_stats()
    assert st["shared_pool"] == 1 and st["nsplit"] == 1 and st["scan_waves"] == waves
    sub = slice(0, 2100, 7)
    Dr, Ir = ref.search(q[sub], 1024, 8)
    assert_topk_parity(oracle, ref, q[sub], D[sub], I[sub], Dr, Ir, TOL_FP32)


def test_k_beyond_what_the_lds_holds_next_to_the_largest_lut_is_refused(ix, oracle):
    """128 sub-quantizers with an fp32 LUT take 128 of the 160 KB of LDS: pools for k <= 1024 fit beside it
    (previous test), larger k is refused with a message that names the need; an fp16 LUT makes room."""
    gpu, ref, x, q, ids = build_pair(ix, oracle, 77, 3000, 5, 128, 8, 128, ix.METRIC_L2)
    gpu.setNumProbes(4)
    with pytest.raises(ix.IndexSdkError, match="bytes of LDS") as err:
        gpu.search(q, 1025)
    assert err.value.code == 2001
    D, I = gpu.search(q, 1024)                  # the index is still usable
    Dr, Ir = ref.search(q, 1024, 4)
    assert_topk_parity(oracle, ref, q, D, I, Dr, Ir, TOL_FP32)
    half, ref16, _, _, _ = build_pair(ix, oracle, 77, 3000, 5, 128, 8, 128, ix.METRIC_L2, lut_fp16=1)
    half.setNumProbes(4)
    D, I = half.search(q, 2048)
    Dr, Ir = ref16.search(q, 2048, 4, lut_fp16=True)
    assert_topk_parity(oracle, ref16, q, D, I, Dr, Ir, TOL_FP16)


def test_xor48_layout_is_the_default_for_m48_and_lists_read_back_in_row_order(ix, oracle):
    gpu, ref, x, q, ids = build_pair(ix, oracle, 47, 20000, 64, 96, 32, 48, ix.METRIC_L2)
    row, _, _, _, _ = build_pair(ix, oracle, 47, 20000, 64, 96, 32, 48, ix.METRIC_L2, layout=0)
    for l in range(32):
        c_a, i_a = gpu.getListCodesAndIds(l)
        c_b, i_b = row.getListCodesAndIds(l)
        assert np.array_equal(c_a, c_b) and np.array_equal(i_a, i_b)
    gpu.setNumProbes(8)
    row.setNumProbes(8)
    D, I = gpu.search(q, 50)
    D0, I0 = row.search(q, 50)
    Dr, Ir = ref.search(q, 50, 8)
    assert_topk_parity(oracle, ref, q, D, I, Dr, Ir, TOL_FP32)
    assert_topk_parity(oracle, ref, q, D0, I0, Dr, Ir, TOL_FP32)
    # removal and a second add keep the position-dependent byte order consistent
    gone = ids[::3]
    assert gpu.remove_ids(gone) == len(gone) and row.remove_ids(gone) == len(gone)
    extra = np.arange(10 ** 7, 10 ** 7 + 500, dtype=np.int64)
    gpu.add_with_ids(x[:500], extra)
    row.add_with_ids(x[:500], extra)
    for l in range(32):
        c_a, i_a = gpu.getListCodesAndIds(l)
        c_b, i_b = row.getListCodesAndIds(l)
        assert np.array_equal(c_a, c_b) and np.array_equal(i_a, i_b)
    D, I = gpu.search(q, 50)
    D0, I0 = row.search(q, 50)
    assert (I == I0).mean() > 0.99 and np.allclose(D, D0, rtol=TOL_FP32, atol=0)


def test_large_k_shared_pool_all_scores_tie(ix, oracle):
    """A base of few distinct vectors: whole lists share one distance, so the bucket search cannot
    separate candidates and the pool falls back to exact selection by sorting."""
    rng = np.random.default_rng(43)
    d, M, nlist = 96, 48, 8
    protos = rng.standard_normal((6, d)).astype(np.float32)
    x = protos[rng.integers(0, 6, 20000)]
    q = (protos[rng.integers(0, 6, 50)] + 0.1 * rng.standard_normal((50, d))).astype(np.float32)
    cent, _ = oracle.kmeans(x + 0.01 * rng.standard_normal(x.shape).astype(np.float32), nlist, niter=3, seed=1)
    cb = oracle.train_pq((x + 0.3 * rng.standard_normal(x.shape)).astype(np.float32)[:4000], M, niter=3, seed=1)
    ids = np.arange(20000, dtype=np.int64)
    ref = oracle.CsrIndex.build(d, M, ix.METRIC_L2, cent, cb, x, ids)
    gpu = ix.AscendIndexIVFPQ(d, ix.METRIC_L2, nlist, M, 8, ix.AscendIndexIVFPQConfig())
    gpu.set_trained(cent, cb)
    gpu.add_with_ids(x, ids)
    gpu.setNumProbes(nlist)
    D, I = gpu.search(q, 1024)
    assert gpu.last_search_stats()["shared_pool"] == 1
    Dr, Ir = ref.search(q, 1024, nlist)
    assert_topk_parity(oracle, ref, q, D, I, Dr, Ir, TOL_FP32)


@pytest.mark.parametrize("k", [100, 300, 1024])
def test_whole_lists_tie_and_the_answer_does_not_depend_on_the_plan(ix, oracle, k):
    """Four sub-quantizers over clustered data: every vector of a cluster gets the same code, so whole lists of
    thousands of vectors share one distance (the shape of the reference's own latency targets: nlist 1024, M 4,
    k 300).  Ties are decided by position in the index, so the answer is the same whether a query is served by
    one workgroup (a batch of 600) or split over eight (a batch of one), with private pools (k = 100: pools of
    256 keys) or the shared pool (k = 300, k = 1024)."""
    rng = np.random.default_rng(4)
    d, M, nlist, n = 128, 4, 32, 120_000
    centres = rng.standard_normal((nlist, d)).astype(np.float32)
    x = (centres[rng.integers(0, nlist, n)] + 0.05 * rng.standard_normal((n, d))).astype(np.float32)
    q = (centres[rng.integers(0, nlist, 600)] + 0.05 * rng.standard_normal((600, d))).astype(np.float32)
    cb = oracle.train_pq(centres + 0.01, M, niter=1, seed=3) if nlist >= 256 else None
    if cb is None:
        # 256 codewords per sub-quantizer with only 32 clusters: the cluster centres' blocks plus far-away filler
        cb = (10.0 + rng.standard_normal((M, 256, d // M))).astype(np.float32)
        cb[:, :nlist, :] = centres.reshape(nlist, M, d // M).transpose(1, 0, 2)
    ids = np.arange(n, dtype=np.int64)
    gpu = ix.AscendIndexIVFPQ(d, ix.METRIC_L2, nlist, M, 8, ix.AscendIndexIVFPQConfig())
    gpu.set_trained(centres, cb)
    gpu.add_with_ids(x, ids)
    ref = oracle.CsrIndex.build(d, M, ix.METRIC_L2, centres, cb, x, ids)
    codes0, _ = gpu.getListCodesAndIds(0)
    assert len(np.unique(codes0, axis=0)) <= 4, "the lists of this test should hold (almost) one code each"
    gpu.setNumProbes(8)
    D, I = gpu.search(q, k)
    assert gpu.last_search_stats()["shared_pool"] == (1 if k > 128 else 0)
    Dr, Ir = ref.search(q, k, 8)
    assert_topk_parity(oracle, ref, q, D, I, Dr, Ir, TOL_FP32)
    for j in (0, 7, 311):
        D1, I1 = gpu.search(q[j:j + 1], k)
        assert gpu.last_search_stats()["nsplit"] > 1
        assert np.array_equal(I1[0], I[j]) and np.array_equal(D1[0].view(np.uint32), D[j].view(np.uint32))


@pytest.mark.parametrize("k", [2048, 700])
def test_merge_of_slices_that_give_no_bound(ix, oracle, k):
    """Eight probed lists, one per workgroup of a split query: seven of 1500 vectors (fewer than k = 2048, so no
    slice is full) and one of 50 (fewer than the rank the merge samples in every slice), so the slices' own order
    bounds nothing and all 10550 keys -- more than the merge keeps in registers -- go through the radix
    selection in global memory.  With k = 700 the seven slices are full and the bound keeps a few thousand keys
    in registers.  Either way the answer is the oracle's and the one a large batch (no split, no merge) gives."""
    rng = np.random.default_rng(91)
    d, M, nlist = 32, 4, 8
    cent = (4.0 * rng.standard_normal((nlist, d))).astype(np.float32)
    sizes = [1500] * 7 + [50]
    owner = np.repeat(np.arange(nlist), sizes)
    x = (cent[owner] + 0.5 * rng.standard_normal((len(owner), d))).astype(np.float32)
    q = (cent[rng.integers(0, nlist, 500)] + 0.5 * rng.standard_normal((500, d))).astype(np.float32)
    cb = oracle.train_pq(x[::3], M, niter=4, seed=5)
    ids = rng.permutation(10 * len(x))[: len(x)].astype(np.int64)
    ref = oracle.CsrIndex.build(d, M, ix.METRIC_L2, cent, cb, x, ids)
    gpu = ix.AscendIndexIVFPQ(d, ix.METRIC_L2, nlist, M, 8, ix.AscendIndexIVFPQConfig())
    gpu.set_trained(cent, cb)
    gpu.add_with_ids(x, ids)
    assert sorted(gpu.getListLength(l) for l in range(nlist)) == sorted(sizes)
    gpu.setNumProbes(nlist)
    D, I = gpu.search(q, k)
    assert gpu.last_search_stats()["nsplit"] == 1
    Dr, Ir = ref.search(q[:4], k, nlist)
    assert_topk_parity(oracle, ref, q[:4], D[:4], I[:4], Dr, Ir, TOL_FP32)
    for j in (0, 1, 2, 3, 77):
        D1, I1 = gpu.search(q[j:j + 1], k)
        assert gpu.last_search_stats()["nsplit"] == 8
        assert np.array_equal(I1[0], I[j]) and np.array_equal(D1[0].view(np.uint32), D[j].view(np.uint32))


@pytest.mark.parametrize("metric_name,k", [("L2", 50), ("L2", 300), ("IP", 300), ("L2", 2048)])
def test_one_query_split_over_many_workgroups(ix, oracle, metric_name, k):
    """Long lists (25000 codes each): a small batch is split over sixteen workgroups per query, one per probed
    list, and the slices are merged (a bound from their own order, then radix selection) -- a few hundred
    survivors ranked by counting (k = 50, 300), thousands sorted (k = 2048).  The answer is the oracle's, and the one a large batch (one workgroup per
    query, no merge) gives for the same queries, bit for bit."""
    metric = ix.METRIC_L2 if metric_name == "L2" else ix.METRIC_INNER_PRODUCT
    gpu, ref, x, q, ids = build_pair(ix, oracle, 17, 400_000, 1500, 32, 16, 8, metric, niter=3)
    gpu.setNumProbes(16)
    D, I = gpu.search(q, k)
    assert gpu.last_search_stats()["nsplit"] == 1
    D3, I3 = gpu.search(q[:3], k)
    assert gpu.last_search_stats()["nsplit"] == 16
    assert np.array_equal(I3, I[:3]) and np.array_equal(D3.view(np.uint32), D[:3].view(np.uint32))
    D40, I40 = gpu.search(q[100:140], k)
    assert 8 < gpu.last_search_stats()["nsplit"] <= 16
    assert np.array_equal(I40, I[100:140]) and np.array_equal(D40.view(np.uint32), D[100:140].view(np.uint32))
    Dr, Ir = ref.search(q[:3], k, 16)
    assert_topk_parity(oracle, ref, q[:3], D3, I3, Dr, Ir, TOL_FP32)
    # fewer vectors than k in the probed lists: padding comes out of the merge
    gpu.setNumProbes(1)
    small = ix.AscendIndexIVFPQ(32, metric, 16, 8, 8, ix.AscendIndexIVFPQConfig())
    small.set_trained(ref.cent, ref.codebook)
    small.add_with_ids(x[:40], ids[:40])
    small.setNumProbes(16)
    Ds, Is = small.search(q[:2], k)
    assert ((Is >= 0).sum(axis=1) == 40).all() and (Is[:, 40:] == -1).all()


@pytest.mark.parametrize("metric_name", ["L2", "IP"])
def test_search_with_tied_and_nearly_tied_centroids(ix, oracle, metric_name):
    """Half of the centroids are exact or 1e-6-perturbed copies of the other half, so the approximate
    coarse scores cannot decide the rank-nprobe boundary: the probed SET must still be the oracle's
    (equal scanned-code counts, equal results) and the probe lists bit-identical."""
    metric = ix.METRIC_L2 if metric_name == "L2" else ix.METRIC_INNER_PRODUCT
    rng = np.random.default_rng(51)
    d, M, nlist, nprobe = 64, 16, 256, 16
    base_c = rng.standard_normal((nlist // 2, d)).astype(np.float32)
    twin = base_c.copy()
    twin[::2] += (1e-6 * rng.standard_normal((nlist // 4, d))).astype(np.float32)     # odd rows stay exact copies
    cent = np.ascontiguousarray(np.concatenate([base_c, twin])[rng.permutation(nlist)])
    x = (cent[rng.integers(0, nlist, 30000)] + 0.3 * rng.standard_normal((30000, d))).astype(np.float32)
    q = (cent[rng.integers(0, nlist, 300)] + 0.3 * rng.standard_normal((300, d))).astype(np.float32)
    cb = oracle.train_pq(x[:4000], M, niter=3, seed=2)
    ids = np.arange(30000, dtype=np.int64)
    ref = oracle.CsrIndex.build(d, M, metric, cent, cb, x, ids)
    gpu = ix.AscendIndexIVFPQ(d, metric, nlist, M, 8, ix.AscendIndexIVFPQConfig())
    gpu.set_trained(cent, cb)
    gpu.add_with_ids(x, ids)
    gpu.setNumProbes(nprobe)
    pi, pd = gpu.coarse_probe(q)
    oi, od = oracle.coarse_probe(q, cent, nprobe, metric)
    assert np.array_equal(pi, oi) and np.array_equal(pd.view(np.uint32), od.view(np.uint32))
    D, I = gpu.search(q, 20)
    Dr, Ir = ref.search(q, 20, nprobe)
    assert gpu.last_search_stats()["scanned_codes"] == ref.last_scanned
    assert_topk_parity(oracle, ref, q, D, I, Dr, Ir, TOL_FP32)


def test_search_redoes_only_the_queries_whose_coarse_proof_fails(ix, oracle):
    """300 centroids within 1e-6 of each other: for queries near them the approximate coarse scores can
    neither rank them nor prove the candidate list complete, so those queries (and only those) are
    redone by the fp32 plan; results and probe lists must equal the oracle's for all queries."""
    rng = np.random.default_rng(61)
    d, M, nlist, nprobe = 64, 16, 2048, 16          # 2048 lists: enough for the bf16 x 3 plan to be used
    cent = rng.standard_normal((nlist, d)).astype(np.float32)
    cent[:300] = cent[0] + (1e-6 * rng.standard_normal((300, d))).astype(np.float32)
    x = (cent[rng.integers(0, nlist, 40000)] + 0.3 * rng.standard_normal((40000, d))).astype(np.float32)
    near = (cent[0] + 0.3 * rng.standard_normal((40, d))).astype(np.float32)
    far = (cent[rng.integers(300, nlist, 360)] + 0.3 * rng.standard_normal((360, d))).astype(np.float32)
    q = np.ascontiguousarray(np.concatenate([near, far])[rng.permutation(400)])
    cb = oracle.train_pq(x[:4000], M, niter=3, seed=3)
    ids = np.arange(40000, dtype=np.int64)
    ref = oracle.CsrIndex.build(d, M, ix.METRIC_L2, cent, cb, x, ids)
    # (batches this small would select their lists from canonical scores: switched off, the matrix-core plans
    # and their proof are what this test is about)
    gpu = ix.AscendIndexIVFPQ(d, ix.METRIC_L2, nlist, M, 8, ix.AscendIndexIVFPQConfig(coarse_exact_small=0))
    gpu.set_trained(cent, cb)
    gpu.add_with_ids(x, ids)
    gpu.setNumProbes(nprobe)
    D, I = gpu.search(q, 20)
    reruns = gpu.last_search_stats()["coarse_reruns"]
    assert 1 <= reruns <= 100, reruns
    Dr, Ir = ref.search(q, 20, nprobe)
    assert gpu.last_search_stats()["scanned_codes"] == ref.last_scanned
    assert_topk_parity(oracle, ref, q, D, I, Dr, Ir, TOL_FP32)
    pi, pd = gpu.coarse_probe(q)
    oi, od = oracle.coarse_probe(q, cent, nprobe, ix.METRIC_L2)
    assert np.array_equal(pi, oi) and np.array_equal(pd.view(np.uint32), od.view(np.uint32))
    # a small batch: every query is split over eight workgroups, and the second scan (of the redone queries
    # only) goes through the split merge under its own numbering
    q2 = np.ascontiguousarray(np.concatenate([near[:25], far[:15]]))
    D2, I2 = gpu.search(q2, 20)
    st = gpu.last_search_stats()
    assert st["nsplit"] == 8 and 1 <= st["coarse_reruns"] <= 25, st
    Dr2, Ir2 = ref.search(q2, 20, nprobe)
    assert st["scanned_codes"] == ref.last_scanned
    assert_topk_parity(oracle, ref, q2, D2, I2, Dr2, Ir2, TOL_FP32)
    # by default a batch of this size (queries x centroids x dims <= 2^27) selects its lists from canonical
    # scores of every centroid: exact by construction, so the tied centroids cost no rerun, same answers
    exact = ix.AscendIndexIVFPQ(d, ix.METRIC_L2, nlist, M, 8, ix.AscendIndexIVFPQConfig())
    exact.set_trained(cent, cb)
    exact.add_with_ids(x, ids)
    exact.setNumProbes(nprobe)
    for batch, ref_D, ref_I in ((q, D, I), (q2, D2, I2)):
        D3, I3 = exact.search(batch, 20)
        assert exact.last_search_stats()["coarse_reruns"] == 0
        assert np.array_equal(I3, ref_I) and np.array_equal(D3.view(np.uint32), ref_D.view(np.uint32))


def test_reset_keeps_quantizers_and_readd_reproduces_codes(ix, oracle):
    """Reference ST invariant (FR/test/ascend/TestAscendIndexIVFPQ.cpp, case All): add / reset / add gives
    byte-identical lists; reset empties every list and leaves the index trained."""
    gpu, ref, x, q, ids = build_pair(ix, oracle, 81, 9000, 20, 64, 64, 16, ix.METRIC_L2)
    before = [gpu.getListCodesAndIds(l) for l in range(64) if gpu.getListLength(l)]
    D0, I0 = gpu.search(q, 7)
    gpu.reset()
    assert gpu.ntotal == 0 and gpu.is_trained and all(gpu.getListLength(l) == 0 for l in range(64))
    D, I = gpu.search(q, 7)
    assert np.all(I == -1) and np.all(D == FLT_MAX)
    gpu.add_with_ids(x, ids)
    after = [gpu.getListCodesAndIds(l) for l in range(64) if gpu.getListLength(l)]
    assert len(before) == len(after)
    for (c0, i0), (c1, i1) in zip(before, after):
        assert np.array_equal(c0, c1) and np.array_equal(i0, i1)
    D1, I1 = gpu.search(q, 7)
    assert np.array_equal(I0, I1) and np.array_equal(D0.view(np.uint32), D1.view(np.uint32))


def test_maximum_k_and_every_list_probed(ix, oracle):
    """k at the library's limit (2048) with nprobe = nlist: every vector is a candidate for every query."""
    gpu, ref, x, q, ids = build_pair(ix, oracle, 91, 6000, 12, 64, 32, 16, ix.METRIC_L2)
    gpu.setNumProbes(32)
    D, I = gpu.search(q, 2048)
    Dr, Ir = ref.search(q, 2048, 32)
    assert gpu.last_search_stats()["scanned_codes"] == 12 * 6000
    assert_topk_parity(oracle, ref, q, D, I, Dr, Ir, TOL_FP32)
    with pytest.raises(ix.IndexSdkError):
        gpu.search(q, 2049)


@pytest.mark.parametrize("d,M", [(64, 16), (96, 48), (60, 6)])
def test_pq_training_step_is_the_lloyd_update_in_sample_order(ix, oracle, d, M):
    """Codebooks after n + 1 iterations = one Lloyd update of the codebooks after n iterations: reference
    encoder for the assignment, float64 sums in sample order for the means (the sub-quantizer update
    runs on the device for sub-vector lengths up to 16 and on the host beyond; both give these bits)."""
    rng = np.random.default_rng(d)
    x = rng.standard_normal((6000, d)).astype(np.float32)
    books = []
    for niter in (2, 3):
        cfg = ix.AscendIndexIVFPQConfig(niter=1, pq_niter=niter, train_samples_per_list=1 << 20)
        gpu = ix.AscendIndexIVFPQ(d, ix.METRIC_L2, 8, M, 8, cfg)
        gpu.train(x)
        books.append(gpu.get_trained()[1])
    # get_trained() after pq_niter iterations returns the codebook the last update produced
    cb_a, cb_b = books
    codes = oracle.pq_encode(x, cb_a)
    dsub = d // M
    checked = 0
    for m in range(M):
        xm = x[:, m * dsub:(m + 1) * dsub].astype(np.float64)
        counts = np.bincount(codes[:, m], minlength=256)
        if (counts == 0).any():
            continue        # an empty codeword is re-seeded by splitting the largest: not a plain mean
        for k in range(0, 256, 7):
            rows = xm[codes[:, m] == k]
            mean = (np.cumsum(rows, axis=0)[-1] / len(rows)).astype(np.float32)
            assert np.array_equal(mean.view(np.uint32), cb_b[m, k].view(np.uint32)), (m, k)
            checked += 1
    assert checked > 100


def test_training_from_device_memory_equals_training_from_host_memory_and_pq_spherical(ix, oracle):
    """A training set in device memory is sampled on the device and never visits the host; the quantizers are the
    ones the host call produces from the same rows, bit for bit (same sample, same seeds, same arithmetic).
    pq_spherical normalises the sub-quantizer codewords after every update (the reference's host training,
    AscendIndexIVFPQImpl.cpp:1064-1067)."""
    import ctypes
    import torch
    from indexsdk_amd import _capi
    lib = _capi.load()
    rng = np.random.default_rng(12)
    d, M, nlist = 64, 8, 32
    x = (rng.standard_normal((20000, d)) + 3.0 * rng.standard_normal((1, d))).astype(np.float32)
    kw = dict(niter=3, train_samples_per_list=200)       # 6400 of the 20000 rows are sampled
    a = ix.AscendIndexIVFPQ(d, ix.METRIC_L2, nlist, M, 8, ix.AscendIndexIVFPQConfig(**kw))
    a.train(x)
    b = ix.AscendIndexIVFPQ(d, ix.METRIC_L2, nlist, M, 8, ix.AscendIndexIVFPQConfig(**kw))
    xd = torch.from_numpy(x).cuda()
    torch.cuda.synchronize()
    _capi.check(lib.ivfpq_train_device(b._h, len(x), ctypes.c_void_p(xd.data_ptr())))
    (ca, ba), (cb, bb) = a.get_trained(), b.get_trained()
    assert np.array_equal(ca.view(np.uint32), cb.view(np.uint32))
    assert np.array_equal(ba.view(np.uint32), bb.view(np.uint32))
    assert not np.allclose(np.linalg.norm(ba, axis=2), 1.0, atol=1e-3)
    s = ix.AscendIndexIVFPQ(d, ix.METRIC_L2, nlist, M, 8, ix.AscendIndexIVFPQConfig(pq_spherical=1, **kw))
    s.train(x)
    cs, bs = s.get_trained()
    assert np.array_equal(cs.view(np.uint32), ca.view(np.uint32))          # the coarse quantizer is not affected
    assert np.allclose(np.linalg.norm(bs, axis=2), 1.0, atol=1e-5)


def test_few_heavy_workgroups_run_heaviest_first(ix, oracle):
    """Long lists, few queries: the scan orders its queries by decreasing work (a scheduling matter only:
    results are those of the oracle, whatever the order)."""
    gpu, ref, x, q, ids = build_pair(ix, oracle, 81, 200000, 1400, 32, 16, 8, ix.METRIC_L2, niter=3)
    gpu.setNumProbes(8)
    for nq, split in ((1400, False), (300, True)):     # one workgroup per query, and three
        D, I = gpu.search(q[:nq], 20)
        st = gpu.last_search_stats()
        assert st["ordered"] == 1 and (st["nsplit"] > 1) == split
        Dr, Ir = ref.search(q[:nq], 20, 8)
        assert_topk_parity(oracle, ref, q[:nq], D, I, Dr, Ir, TOL_FP32)
        assert st["scanned_codes"] == ref.last_scanned
    gpu.setNumProbes(1)
    gpu.search(q[:70], 20)
    assert gpu.last_search_stats()["ordered"] == 0


def test_large_batches_run_in_locality_order_with_the_same_results(ix, oracle):
    """Large batches: the scan's workgroups run in an order that puts queries probing the same lists side by
    side, one contiguous chunk of that order per XCD (a scheduling matter only).  Results are bit-identical
    to those in input order, for a query count that is no multiple of eight, and equal the oracle's."""
    gpu, ref, x, q, ids = build_pair(ix, oracle, 83, 60000, 2051, 64, 128, 16, ix.METRIC_L2, niter=3)
    cent, cb = gpu.get_trained()
    results = {}
    for mode, nq, want in ((0, 2051, 0), (-1, 2051, 2), (1, 2051, 2), (1, 501, 2), (0, 501, 0), (-1, 501, 0)):
        g = ix.AscendIndexIVFPQ(64, ix.METRIC_L2, 128, 16, 8, ix.AscendIndexIVFPQConfig(scan_locality=mode))
        g.set_trained(cent, cb)
        g.add_with_ids(x, ids)
        g.setNumProbes(12)
        D, I = g.search(q[:nq], 50)
        st = g.last_search_stats()
        assert st["ordered"] == want and st["nsplit"] == 1
        assert st["scanned_codes"] == np.diff(ref.list_off)[oracle.coarse_probe(q[:nq], cent, 12, ix.METRIC_L2)[0]].sum()
        if nq in results:
            assert np.array_equal(I, results[nq][1])
            assert np.array_equal(D.view(np.uint32), results[nq][0].view(np.uint32))
        else:
            results[nq] = (D, I)
            Dr, Ir = ref.search(q[:nq], 50, 12)
            assert_topk_parity(oracle, ref, q[:nq], D, I, Dr, Ir, TOL_FP32)


def test_sixteen_wave_pool_with_an_lds_plan_that_fills_whole_allocation_granules(ix, oracle):
    """M = 48 (64 KB LUT), d = 96, k = 1024 and 64 lists per workgroup make the scan's LDS plan end within
    a few bytes of a multiple of 1280: the control words of the sixteen-wave pool must lie inside it."""
    gpu, ref, x, q, ids = build_pair(ix, oracle, 91, 30000, 2100, 96, 64, 48, ix.METRIC_L2)
    gpu.setNumProbes(64)
    D, I = gpu.search(q, 1024)
    st = gpu.last_search_stats()
    assert st["shared_pool"] == 1 and st["nsplit"] == 1 and st["scan_waves"] == 16
    sub = slice(0, 2100, 21)
    Dr, Ir = ref.search(q[sub], 1024, 64)
    assert_topk_parity(oracle, ref, q[sub], D[sub], I[sub], Dr, Ir, TOL_FP32)


def test_concurrent_callers_of_one_index_are_serialised(ix, oracle):
    """Searches from several threads on the same index (ctypes releases the GIL): every call holds the
    handle's lock, so each thread gets the result a lone caller gets
    (FR/ascend/impl/AscendIndexImpl.h:62, 230: the reference's optional per-index lock)."""
    import threading
    gpu, ref, x, q, ids = build_pair(ix, oracle, 93, 20000, 400, 64, 32, 16, ix.METRIC_L2)
    gpu.setNumProbes(8)
    want = [gpu.search(q[i::4], 10 + i) for i in range(4)]
    got = [None] * 4

    def work(i):
        for _ in range(5):
            got[i] = gpu.search(q[i::4], 10 + i)

    threads = [threading.Thread(target=work, args=(i,)) for i in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    for i in range(4):
        assert np.array_equal(got[i][1], want[i][1]) and np.array_equal(got[i][0].view(np.uint32), want[i][0].view(np.uint32))


def test_recall_harness_against_exact_neighbours(ix, oracle):
    """evaluate() / ground_truth() of indexsdk_amd.datasets, the counterpart of the reference's SIFT1M
    recall harness (FR/test/python/datasets.py:71-84, TestAscendIndexIVFPQ.py:33-72): the GPU brute force
    agrees with the oracle's, recall grows with r and with nprobe, and probing every list with fine
    codes finds almost every true neighbour."""
    from indexsdk_amd.datasets import evaluate, ground_truth
    gpu, ref, x, q, ids = build_pair(ix, oracle, 90, 20000, 300, 64, 64, 32, ix.METRIC_L2)
    gt = ground_truth(x, q, 1, "L2", ids)
    Do, Io = oracle.flat_f32(x, q, 1, ix.METRIC_L2)
    assert np.array_equal(gt[:, 0], ids[Io[:, 0]])
    gpu.setNumProbes(1)
    _, r1 = evaluate(gpu, q, gt, 100)
    gpu.setNumProbes(64)
    ms, r64 = evaluate(gpu, q, gt, 100)
    assert list(r64) == [1, 10, 100] and ms > 0
    assert r64[1] <= r64[10] <= r64[100] and r1[1] <= r1[10] <= r1[100]
    assert r64[100] >= r1[100] and r64[100] >= 0.99 and r64[1] >= 0.3
    # the same figures from the oracle's result lists: parity of ids makes the recall identical
    Dr, Ir = ref.search(q, 100, 64)
    want = {r: float((Ir[:, :r] == gt[:, :1]).any(axis=1).mean()) for r in (1, 10, 100)}
    assert all(abs(r64[r] - want[r]) <= 1.0 / len(q) for r in want)


def test_largest_nprobe(ix, oracle):
    """nprobe = 2048 of 2500 lists (the limit: 2048 + 16 + 256 candidates per query go through the probe
    selection): probe ids and distances bit-exact, search parity; one more is refused, and a request
    beyond the number of lists is clamped to it first."""
    nlist, d, M = 2500, 32, 8
    rng = np.random.default_rng(12)
    centres = rng.standard_normal((40, d)).astype(np.float32)
    cent = (centres[rng.integers(0, 40, nlist)] + 0.5 * rng.standard_normal((nlist, d))).astype(np.float32)
    x = (centres[rng.integers(0, 40, 30000)] + 0.5 * rng.standard_normal((30000, d))).astype(np.float32)
    q = (centres[rng.integers(0, 40, 20)] + 0.5 * rng.standard_normal((20, d))).astype(np.float32)
    cb = oracle.train_pq(x[:4000], M, niter=2, seed=2)
    gpu = ix.AscendIndexIVFPQ(d, ix.METRIC_L2, nlist, M, 8, ix.AscendIndexIVFPQConfig())
    gpu.set_trained(cent, cb)
    gpu.add(x)
    with pytest.raises(ix.IndexSdkError, match="nprobe must be <= 2048"):
        gpu.setNumProbes(2049)
    gpu.setNumProbes(2048)
    gi, gd = gpu.coarse_probe(q)
    oi, od = oracle.coarse_probe(q, cent, 2048, ix.METRIC_L2)
    assert np.array_equal(gi, oi) and np.array_equal(gd.view(np.uint32), od.view(np.uint32))
    ref = oracle.CsrIndex.build(d, M, ix.METRIC_L2, cent, cb, x)
    D, I = gpu.search(q, 100)
    Dr, Ir = ref.search(q, 100, 2048)
    assert_topk_parity(oracle, ref, q, D, I, Dr, Ir, TOL_FP32)
    small = ix.AscendIndexIVFPQ(d, ix.METRIC_L2, 64, M, 8, ix.AscendIndexIVFPQConfig())
    small.setNumProbes(100000)
    assert small.getNumProbes() == 64


@pytest.mark.parametrize("nlist,nq,scratch", [(2600, 3000, 4 << 20), (5000, 3000, 32 << 20), (12900, 3000, 32 << 20),
                                              (12900, 700, 64 << 20), (4096, 10000, 64 << 20)])
def test_coarse_probe_with_a_small_score_scratch(ix, oracle, nlist, nq, scratch):
    """A score scratch (the reference's resourceSize) far below the default makes the coarse stage walk the
    centroids in chunks.  The matrix-core kernel for split operands only serves chunks of 2048 rows or more:
    the plan narrows the query block instead of the chunk, and where a remainder would still be too short it
    leaves the whole call to the fp32 kernels.  Either way probes and distances are the oracle's."""
    d, M, nprobe = 32, 8, 24
    rng = np.random.default_rng(nlist + nq)
    centres = rng.standard_normal((30, d)).astype(np.float32)
    cent = (centres[rng.integers(0, 30, nlist)] + 0.4 * rng.standard_normal((nlist, d))).astype(np.float32)
    q = (centres[rng.integers(0, 30, nq)] + 0.4 * rng.standard_normal((nq, d))).astype(np.float32)
    cb = rng.standard_normal((M, 256, d // M)).astype(np.float32)
    gpu = ix.AscendIndexIVFPQ(d, ix.METRIC_L2, nlist, M, 8, ix.AscendIndexIVFPQConfig(scratch_bytes=scratch))
    gpu.set_trained(cent, cb)
    gpu.setNumProbes(nprobe)
    gi, gd = gpu.coarse_probe(q)
    oi, od = oracle.coarse_probe(q, cent, nprobe, ix.METRIC_L2)
    assert np.array_equal(gi, oi) and np.array_equal(gd.view(np.uint32), od.view(np.uint32))
    assert np.array_equal(gpu.assign(q), oracle.assign(q, cent))


def test_search_in_query_pages_equals_one_batch(ix, oracle):
    """A scratch budget (the reference's resourceSize) of 1 MiB holds the workspaces of 768 of these queries:
    2500 queries are served in four pages, with the answers of the unpaged search bit for bit and the
    statistics summed over the pages (AscendIndexImpl::searchPaged, FR/ascend/impl/AscendIndexImpl.cpp:296-346)."""
    gpu, ref, x, q, ids = build_pair(ix, oracle, 83, 30000, 2500, 64, 96, 16, ix.METRIC_L2)
    cent, cb = gpu.get_trained()
    small = ix.AscendIndexIVFPQ(64, ix.METRIC_L2, 96, 16, 8, ix.AscendIndexIVFPQConfig(scratch_bytes=1 << 20))
    small.set_trained(cent, cb)
    small.add_with_ids(x, ids)
    for g in (gpu, small):
        g.setNumProbes(8)
    D, I = gpu.search(q, 20)
    one = gpu.last_search_stats()
    Dp, Ip = small.search(q, 20)
    paged = small.last_search_stats()
    assert one["pages"] == 1 and paged["pages"] == 4, (one["pages"], paged["pages"])
    assert np.array_equal(Ip, I) and np.array_equal(Dp.view(np.uint32), D.view(np.uint32))
    assert paged["scanned_codes"] == one["scanned_codes"]
    Dr, Ir = ref.search(q, 20, 8)
    assert paged["scanned_codes"] == ref.last_scanned
    assert_topk_parity(oracle, ref, q, Dp, Ip, Dr, Ir, TOL_FP32)


@pytest.mark.parametrize("spherical,metric_name,nlist,n", [(0, "L2", 96, 5000), (1, "L2", 96, 5000), (-1, "IP", 96, 5000),
                                                           (0, "L2", 12, 40000)])
def test_coarse_training_step_is_the_lloyd_update_in_sample_order(ix, oracle, spherical, metric_name, nlist, n):
    """Centroids after n + 1 iterations = one Lloyd update of the centroids after n: nearest-centroid
    assignment under L2 (the add path's rule), float64 sums in sample order for the means, a cluster without
    members re-seeded by splitting the most populated one (its centroid times 1 -+ 1/1024, the sign
    alternating over the components, members shared out evenly), rows normalised when spherical (which
    inner product switches on by default).  The data leave some of the clusters empty; the last case has clusters
    of several thousand members (the member lists are sorted on the device, whatever their length)."""
    metric = ix.METRIC_L2 if metric_name == "L2" else ix.METRIC_INNER_PRODUCT
    d = 32
    rng = np.random.default_rng(17 + spherical)
    centres = rng.standard_normal((6, d)).astype(np.float32) * 4
    x = (centres[rng.integers(0, 6, n)] + 0.05 * rng.standard_normal((n, d))).astype(np.float32)
    x[100:] = centres[rng.integers(0, 6, n - 100)]        # 4900 rows are exact copies of six points: of the
    #                                                       centroids that coincide on one, all but the first stay empty
    if metric == ix.METRIC_INNER_PRODUCT:
        x /= np.linalg.norm(x, axis=1, keepdims=True)
    cents = []
    for niter in (2, 3):
        cfg = ix.AscendIndexIVFPQConfig(niter=niter, pq_niter=0, spherical=spherical, train_samples_per_list=1 << 20)
        gpu = ix.AscendIndexIVFPQ(d, metric, nlist, 8, 8, cfg)
        gpu.train(x)
        cents.append(gpu.get_trained()[0])
    before, after = cents
    asg = oracle.assign(x, before)
    cnt = np.bincount(asg, minlength=nlist).astype(np.int64)
    want = before.copy()
    for c in range(nlist):
        if cnt[c]:
            rows = x[asg == c].astype(np.float64)
            want[c] = (np.cumsum(rows, axis=0)[-1] / cnt[c]).astype(np.float32)
    empties = int((cnt == 0).sum())
    eps = np.where(np.arange(d) % 2 == 1, np.float32(1 / 1024), np.float32(-1 / 1024)).astype(np.float32)
    for c in range(nlist):
        if cnt[c] == 0:
            big = int(np.argmax(cnt))
            v = want[big].copy()
            want[c] = v * (np.float32(1) + eps)
            want[big] = v * (np.float32(1) - eps)
            cnt[c] = cnt[big] // 2
            cnt[big] -= cnt[c]
    if spherical == 1 or (spherical < 0 and metric == ix.METRIC_INNER_PRODUCT):
        norm = np.sqrt(np.cumsum(want.astype(np.float64) ** 2, axis=1)[:, -1])      # summed left to right
        want = (want.astype(np.float64) / norm[:, None]).astype(np.float32)
    assert empties >= 1, "the data should leave clusters empty"
    assert np.array_equal(want.view(np.uint32), after.view(np.uint32))


def test_host_batch_beyond_the_staging_buffer_equals_its_pieces(ix, oracle):
    """Host searches of up to 256 MB of queries + results go through the index's page-locked staging buffer (the
    kernels write the results into it, the copy-out is shared by threads); larger ones are copied by the runtime.
    Both routes, and the pieces of a batch searched on their own, give the same bits."""
    d, nlist, M, n, nq, k = 32, 64, 8, 20000, 450_000, 40
    assert nq * (d * 4 + k * 12) > 256 << 20
    rng = np.random.default_rng(77)
    x = rng.standard_normal((n, d)).astype(np.float32)
    q = rng.standard_normal((nq, d)).astype(np.float32)
    cent, _ = oracle.kmeans(x[:4000], nlist, niter=3, seed=5)
    cb = oracle.train_pq(x[:4000], M, niter=3, seed=5)
    gpu = ix.AscendIndexIVFPQ(d, ix.METRIC_L2, nlist, M, 8)
    gpu.set_trained(cent, cb)
    gpu.add(x)
    gpu.setNumProbes(8)
    D, I = gpu.search(q, k)
    for a, m in ((0, 3000), (200_000, 150_000), (nq - 2500, 2500)):     # a small piece, a multi-threaded copy-out, the tail
        Dp, Ip = gpu.search(q[a:a + m], k)
        assert np.array_equal(Ip, I[a:a + m]) and np.array_equal(Dp.view(np.uint32), D[a:a + m].view(np.uint32))
    ref = oracle.CsrIndex.build(d, M, ix.METRIC_L2, cent, cb, x, np.arange(n, dtype=np.int64))
    Dr, Ir = ref.search(q[:500], k, 8)
    assert_topk_parity(oracle, ref, q[:500], D[:500], I[:500], Dr, Ir, TOL_FP32)
