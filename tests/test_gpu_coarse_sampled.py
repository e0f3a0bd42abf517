"""GPU parity tests of the coarse stage's sampled-bound plan (large query x centroid products): the score
kernel's admission bound comes from group minima over a seed stretch of the centroids, runs of four scores
at or below it are appended as records, and every query's result is proven afterwards; queries without
proof are redone exactly.  Whatever the plan, probe ids and distances are the oracle's bit for bit."""
import numpy as np
import pytest

from tests.parity import assert_topk_parity

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ix():
    import indexsdk_amd
    return indexsdk_amd


def _mixture(rng, comp, n, d, sigma, centres=None):
    if centres is None:
        centres = rng.standard_normal((comp, d)).astype(np.float32)
    return (centres[rng.integers(0, len(centres), n)] + sigma * rng.standard_normal((n, d))).astype(np.float32), centres


@pytest.mark.parametrize("metric_name,nlist,nprobe,nq,scratch,d,resident", [
    ("L2", 8192, 32, 2200, 0, 64, 1),          # the smallest product the plan takes (seed 2048 of 8192 centroids)
    ("IP", 12000, 64, 2048, 0, 64, 1),         # a last tile of 224 centroids
    ("L2", 16384, 64, 1500, 0, 64, 1),
    ("L2", 8192, 32, 2304, 8 << 20, 64, 1),    # a scratch that holds the records of 512 queries: five query blocks
    ("L2", 32768, 200, 512, 0, 64, 1),         # 241 candidates per query, seed of 4096 centroids, > 1024 scores per fold
    # the other dimensions the resident-query score kernel has instances for, query counts that end inside a tile
    ("L2", 16384, 64, 1111, 0, 128, 1),
    ("IP", 9000, 32, 2500, 0, 96, 1),
    ("L2", 8192, 16, 4000, 0, 96, 1),
    # the ring kernel (what dimensions without such an instance use), on the shapes above
    ("L2", 8192, 32, 2200, 0, 64, 0),
    ("IP", 12000, 64, 2048, 0, 64, 0),
    ("L2", 16384, 64, 1111, 0, 128, 0),
    ("L2", 8192, 32, 2200, 0, 160, 1),         # no resident instance for 160 dimensions: the ring kernel serves them
])
def test_sampled_bound_plan_is_bit_exact(ix, oracle, metric_name, nlist, nprobe, nq, scratch, d, resident):
    metric = ix.METRIC_L2 if metric_name == "L2" else ix.METRIC_INNER_PRODUCT
    M = 8
    rng = np.random.default_rng(nlist + nprobe)
    cent, centres = _mixture(rng, 48, nlist, d, 0.4)
    q, _ = _mixture(rng, 48, nq, d, 0.4, centres)
    x, _ = _mixture(rng, 48, 30000, d, 0.4, centres)
    if metric == ix.METRIC_INNER_PRODUCT:
        for a in (cent, q, x):
            a /= np.linalg.norm(a, axis=1, keepdims=True)
    cb = rng.standard_normal((M, 256, d // M)).astype(np.float32)
    kw = {"scratch_bytes": scratch} if scratch else {}
    gpu = ix.AscendIndexIVFPQ(d, metric, nlist, M, 8, ix.AscendIndexIVFPQConfig(coarse_resident=resident, **kw))
    gpu.set_trained(cent, cb)
    gpu.setNumProbes(nprobe)
    gi, gd = gpu.coarse_probe(q)
    oi, od = oracle.coarse_probe(q, cent, nprobe, metric)
    assert np.array_equal(gi, oi)
    assert np.array_equal(gd.view(np.uint32), od.view(np.uint32))
    assert np.array_equal(gpu.assign(q), oracle.assign(q, cent))          # the same plan with one list per row
    ids = np.arange(30000, dtype=np.int64)
    gpu.add_with_ids(x, ids)
    ref = oracle.CsrIndex.build(d, M, metric, cent, cb, x, ids)
    D, I = gpu.search(q, 20)
    stats = gpu.last_search_stats()
    assert stats["coarse_plan"] == 1, "this product should take the sampled-bound plan"
    Dr, Ir = ref.search(q, 20, nprobe)
    assert stats["scanned_codes"] == ref.last_scanned                      # the same SET of lists for every query
    assert_topk_parity(oracle, ref, q, D, I, Dr, Ir, 1e-4)
    # the plan that writes the score matrix gives the same answer
    off = ix.AscendIndexIVFPQ(d, metric, nlist, M, 8, ix.AscendIndexIVFPQConfig(coarse_sampled_bound=0, **kw))
    off.set_trained(cent, cb)
    off.setNumProbes(nprobe)
    off.add_with_ids(x, ids)
    D0, I0 = off.search(q, 20)
    assert off.last_search_stats()["coarse_plan"] == 0
    assert np.array_equal(I0, I) and np.array_equal(D0.view(np.uint32), D.view(np.uint32))


def _group_column(g, resident):
    """First column of score-kernel group g, the 32 columns one group minimum of the seed launch covers: 32 consecutive
    centroids (one wavefront's block) in the resident-query kernel, the 32 columns of a 256-column tile that one lane
    owns in the ring kernel."""
    if resident:
        return 32 * g
    return (g // 8) * 256 + ((g % 8) // 2) * 64 + 4 * (g % 2)


@pytest.mark.parametrize("resident", [1, 0])
@pytest.mark.parametrize("case,scratch", [("farthest_first", 0), ("farthest_first", 8 << 20), ("decoys", 0)])
def test_sampled_bound_with_centroids_in_an_adverse_order(ix, oracle, case, scratch, resident):
    """All queries come from one cluster, and the seed stretch (the first 2048 centroids) says nothing about
    the rest.  farthest_first: the centroids are sorted by decreasing distance to that cluster, so the bound
    admits more than a row's records hold.  decoys: 30 centroids next to the cluster sit in 30 different
    groups of the seed, so the bound (the 29th smallest group minimum) lies below the score at rank nprobe
    and the proof fails.  Every such query is redone exactly, the answers stay the oracle's, and the index
    stops using the plan.  (With the small scratch the queries go through the plan in blocks: the redone
    rows are named across blocks.)"""
    d, M, nlist, nprobe, nq = 64, 8, 8192, 32, 2112
    rng = np.random.default_rng(77)
    cent = rng.standard_normal((nlist, d)).astype(np.float32)
    centre = cent[0].copy()
    if case == "farthest_first":
        dist = ((cent - centre) ** 2).sum(axis=1)
        cent = np.ascontiguousarray(cent[np.argsort(dist)[::-1]])
    else:
        for g in range(30):
            cent[_group_column(g, resident)] = centre + (0.05 * rng.standard_normal(d)).astype(np.float32)
    q = (centre + 0.2 * rng.standard_normal((nq, d))).astype(np.float32)
    x = (cent[rng.integers(0, nlist, 20000)] + 0.2 * rng.standard_normal((20000, d))).astype(np.float32)
    cb = rng.standard_normal((M, 256, d // M)).astype(np.float32)
    ids = np.arange(20000, dtype=np.int64)
    kw = {"scratch_bytes": scratch} if scratch else {}
    gpu = ix.AscendIndexIVFPQ(d, ix.METRIC_L2, nlist, M, 8, ix.AscendIndexIVFPQConfig(coarse_resident=resident, **kw))
    gpu.set_trained(cent, cb)
    gpu.setNumProbes(nprobe)
    # the first search runs on the empty index, so that nothing but these queries has met the plan yet (adding
    # vectors assigns them with the same plan, and may already have switched it off)
    D, I = gpu.search(q, 10)
    stats = gpu.last_search_stats()
    assert stats["coarse_plan"] == 1 and stats["coarse_reruns"] >= nq // 2, stats
    assert (I == -1).all()
    gi, gd = gpu.coarse_probe(q)
    oi, od = oracle.coarse_probe(q, cent, nprobe, ix.METRIC_L2)
    assert np.array_equal(gi, oi) and np.array_equal(gd.view(np.uint32), od.view(np.uint32))
    gpu.add_with_ids(x, ids)
    ref = oracle.CsrIndex.build(d, M, ix.METRIC_L2, cent, cb, x, ids)
    for l in range(0, nlist, 97):
        assert gpu.getListLength(l) == ref.list_off[l + 1] - ref.list_off[l]
    D, I = gpu.search(q, 10)
    stats = gpu.last_search_stats()
    assert stats["coarse_plan"] == 0 and stats["coarse_reruns"] == 0, stats
    Dr, Ir = ref.search(q, 10, nprobe)
    assert stats["scanned_codes"] == ref.last_scanned
    assert_topk_parity(oracle, ref, q, D, I, Dr, Ir, 1e-4)
