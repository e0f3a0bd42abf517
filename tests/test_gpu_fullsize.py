"""The headline configuration at its full size (10M x 128, nlist 16384, M 32, 10000 queries, nprobe 64,
k 100) through properties that do not need a full-size reference run, plus oracle parity on a sample of
the queries against the index copied back to the host."""
import numpy as np
import pytest

from tests.parity import assert_topk_parity

pytestmark = pytest.mark.gpu

N, D, NLIST, M, NQ, NPROBE, K = 10_000_000, 128, 16384, 32, 10_000, 64, 100


@pytest.fixture(scope="module")
def big():
    import indexsdk_amd as ix
    rng = np.random.default_rng(1236)
    centres = rng.standard_normal((1024, D), dtype=np.float32)

    def draw(n):
        x = rng.standard_normal((n, D), dtype=np.float32)
        x *= np.float32(0.25)
        x += centres[rng.integers(0, 1024, n)]
        return x

    cfg = ix.AscendIndexIVFPQConfig(niter=4, train_samples_per_list=1 << 20)
    index = ix.AscendIndexIVFPQ(D, ix.METRIC_L2, NLIST, M, 8, cfg)
    index.train(draw(500_000))
    keep = {}
    for c in range(10):
        x = draw(N // 10)
        if c == 3:
            keep["rows"] = x[:2000].copy()                  # database vectors used as queries later
            keep["first_id"] = c * (N // 10)
        index.add(x)
    del x
    q = draw(NQ)
    index.setNumProbes(NPROBE)
    return ix, index, q, keep


def test_full_size_result_properties(big):
    ix, index, q, keep = big
    assert index.ntotal == N
    lens = np.array([index.getListLength(l) for l in range(NLIST)], dtype=np.int64)
    assert lens.sum() == N
    Dm, Im = index.search(q, K)
    st = index.last_search_stats()
    assert (Im >= 0).all() and (Im < N).all()
    assert (np.diff(Dm, axis=1) >= 0).all()                                   # best first
    assert (np.diff(np.sort(Im, axis=1), axis=1) > 0).all()                   # no id twice
    # idempotence, and k = 10 is a prefix of k = 100
    D2, I2 = index.search(q, K)
    assert np.array_equal(I2, Im) and np.array_equal(D2.view(np.uint32), Dm.view(np.uint32))
    D10, I10 = index.search(q, 10)
    assert np.array_equal(I10, Im[:, :10]) and np.array_equal(D10.view(np.uint32), Dm[:, :10].view(np.uint32))
    # the scanned-code count is the sum of the probed lists' lengths
    probes, _ = index.coarse_probe(q)
    assert st["scanned_codes"] == lens[probes].sum()
    # fewer probes can only make the k-th distance worse
    index.setNumProbes(16)
    D16, _ = index.search(q, K)
    index.setNumProbes(NPROBE)
    assert (D16[:, K - 1] >= Dm[:, K - 1]).all()


def test_full_size_self_queries_come_back_first(big):
    """A database vector's own code minimises every term of its ADC sum, and its own list is its first
    probe: it is the top result unless another vector of a probed list has the same code
    (FR/test/ascend/TestAscendIndexIVFPQ.cpp:150-166)."""
    ix, index, q, keep = big
    rows, first = keep["rows"], keep["first_id"]
    Ds, Is = index.search(rows, 5)
    own = np.arange(first, first + len(rows))
    hit = Is[:, 0] == own
    assert hit.mean() > 0.995
    # where another id came first it ties with the vector's own entry
    for i in np.flatnonzero(~hit):
        pos = np.flatnonzero(Is[i] == own[i])
        assert len(pos) == 1 and Ds[i, pos[0]] == Ds[i, 0]


def test_full_size_sample_against_the_oracle(big, oracle):
    ix, index, q, keep = big
    cent, cb = index.get_trained()
    lens = np.array([index.getListLength(l) for l in range(NLIST)], dtype=np.int64)
    off = np.zeros(NLIST + 1, dtype=np.int64)
    np.cumsum(lens, out=off[1:])
    codes = np.empty((N, M), dtype=np.uint8)
    ids = np.empty(N, dtype=np.int64)
    for l in range(NLIST):
        if lens[l]:
            codes[off[l]:off[l + 1]], ids[off[l]:off[l + 1]] = index.getListCodesAndIds(l)
    assert np.array_equal(np.sort(ids), np.arange(N))
    ref = oracle.CsrIndex(D, M, ix.METRIC_L2, cent, cb, off, codes, ids)
    sample = q[::50]
    Dg, Ig = index.search(sample, K)
    Dr, Ir = ref.search(sample, K, NPROBE)
    exempt = assert_topk_parity(oracle, ref, sample, Dg, Ig, Dr, Ir, 1e-4)
    assert exempt <= 0.002 * Ig.size + 5
    pi, pd = index.coarse_probe(sample)
    oi, od = oracle.coarse_probe(sample, cent, NPROBE, ix.METRIC_L2)
    assert np.array_equal(pi, oi) and np.array_equal(pd.view(np.uint32), od.view(np.uint32))


def test_full_size_incremental_writes(big):
    """On the 10M index: small adds extend lists in place (the arena is not replaced every time), a removal
    of 1000 ids is a device-side compaction that takes milliseconds, removed ids never come back, and vectors
    added afterwards are found by their own queries.  (Runs last of the tests that share the index: it
    changes it.)"""
    import time
    ix, index, q, keep = big
    rng = np.random.default_rng(99)
    sizes = {index.arena_state()[0]}
    t0 = time.perf_counter()
    new_rows = []
    for c in range(20):
        x = (keep["rows"][rng.integers(0, 2000, 10_000)] + 0.25 * rng.standard_normal((10_000, D))).astype(np.float32)
        ids = np.arange(N + c * 10_000, N + (c + 1) * 10_000, dtype=np.int64)
        index.add_with_ids(x, ids)
        sizes.add(index.arena_state()[0])
        new_rows.append(x[:50])
    t_add = time.perf_counter() - t0
    assert index.ntotal == N + 200_000
    assert len(sizes) <= 2, f"20 small adds replaced the arena {len(sizes) - 1} times"
    assert t_add < 5.0, f"20 adds of 10000 vectors took {t_add:.2f} s"
    victims = rng.choice(N, 1000, replace=False).astype(np.int64)
    t0 = time.perf_counter()
    assert index.remove_ids(victims) == 1000
    t_rm = time.perf_counter() - t0
    assert t_rm < 0.5, f"remove_ids(1000) on 10M vectors took {t_rm * 1e3:.0f} ms"
    assert index.ntotal == N + 199_000 and index.remove_ids(victims) == 0
    Dm, Im = index.search(q, K)
    assert not np.isin(Im, victims).any()
    assert (np.diff(Dm, axis=1) >= 0).all() and (Im >= 0).all()
    rows = np.concatenate(new_rows)
    own = np.concatenate([np.arange(N + c * 10_000, N + c * 10_000 + 50) for c in range(20)])
    Ds, Is = index.search(rows, 5)
    hit = Is[:, 0] == own
    assert hit.mean() > 0.98
    for i in np.flatnonzero(~hit):
        pos = np.flatnonzero(Is[i] == own[i])
        assert len(pos) == 1 and Ds[i, pos[0]] == Ds[i, 0]


def test_full_size_flat_int8_exact(oracle):
    """Flat int8 at its full size (10M x 512, 2048 queries, k 100): every returned distance is the exact
    integer distance of the returned id, rows are ordered by (distance, id), planted copies of base
    vectors come back at distance 0, and a sample of the queries equals brute force over the whole base."""
    import indexsdk_amd as ix
    n, d, nq, k = 10_000_000, 512, 2048, 100
    rng = np.random.default_rng(1238)
    index = ix.AscendIndexInt8Flat(d)
    chunks = []
    for c in range(10):
        b = rng.integers(-127, 128, size=(n // 10, d), dtype=np.int8)
        index.add(b)
        chunks.append(b)
    base = np.concatenate(chunks)
    del chunks
    q = rng.integers(-127, 128, size=(nq, d), dtype=np.int8)
    planted = rng.integers(0, n, 64)
    q[:64] = base[planted]
    Dg, Ig = index.search_int32(q, k)
    assert index.ntotal == n and (Ig >= 0).all() and (Ig < n).all()
    assert (Dg[:64, 0] == 0).all() and (Ig[:64, 0] == planted).all()
    # ordered by (distance, id); no id twice
    dd, di = np.diff(Dg, axis=1), np.diff(Ig, axis=1)
    assert ((dd > 0) | ((dd == 0) & (di > 0))).all()
    # returned distances are the exact integer distances of the returned ids (a sample of rows)
    for i in range(0, nq, 97):
        diff = base[Ig[i]].astype(np.int32) - q[i].astype(np.int32)
        assert np.array_equal((diff * diff).sum(axis=1), Dg[i])
    # brute force over the whole base for a few queries
    sample = np.arange(0, nq, 128)
    Dr, Ir = oracle.flat_i8(base, q[sample], k)
    assert np.array_equal(Ig[sample], Ir) and np.array_equal(Dg[sample], Dr)
