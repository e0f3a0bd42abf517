"""Concurrent searches on one IVFPQ index (the reference's MX_INDEX_MULTITHREAD mode: shared lock for search,
exclusive lock for everything that changes the index; FR/ascend/impl/AscendIndexImpl.h:62, 230 and
FR/ascend/impl/AscendIndexImpl.cpp:204, 508-564).

Threads call through the C ABI (ctypes releases the interpreter lock for the call).  Bar: every search that ran
beside others returns bit for bit what the same search returns alone; against the oracle at 1e-4 like every
other IVFPQ parity test."""
import threading

import numpy as np
import pytest

from tests.parity import assert_topk_parity
from tests.test_gpu_ivfpq import build_pair, make_data, TOL_FP32

pytestmark = pytest.mark.gpu

BATCHES = (1, 7, 32, 200)


def run_threads(nthreads, body):
    errors = []
    start = threading.Barrier(nthreads)

    def wrapped(t):
        try:
            start.wait()
            body(t)
        except BaseException as e:   # noqa: BLE001 - reported by the test below
            errors.append((t, repr(e)))

    threads = [threading.Thread(target=wrapped, args=(t,)) for t in range(nthreads)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    assert not errors, errors


def serial_results(gpu, queries, k):
    return [gpu.search(q, k) for q in queries]


def concurrent_equal_serial(gpu, queries, k, nthreads, rounds):
    want = serial_results(gpu, queries, k)

    def body(t):
        for r in range(rounds):
            j = (t + r) % len(queries)
            D, I = gpu.search(queries[j], k)
            assert np.array_equal(I, want[j][1]), f"thread {t} round {r} batch {j}: labels differ"
            assert np.array_equal(D, want[j][0]), f"thread {t} round {r} batch {j}: distances differ"

    run_threads(nthreads, body)
    return want


def test_searches_side_by_side_equal_searches_alone(ix, oracle):
    gpu, ref, x, q, ids = build_pair(ix, oracle, 91, 60000, sum(BATCHES), 64, 256, 16, ix.METRIC_L2)
    gpu.setNumProbes(16)
    k = 10
    cuts = np.cumsum((0,) + BATCHES)
    queries = [np.ascontiguousarray(q[a:b]) for a, b in zip(cuts[:-1], cuts[1:])]
    assert gpu.search_lanes() == 1
    # six threads on four lanes: two of them wait for a lane now and then
    want = concurrent_equal_serial(gpu, queries, k, nthreads=6, rounds=40)
    assert 2 <= gpu.search_lanes() <= 4
    Dref, Iref = ref.search(queries[3], k, 16)
    assert_topk_parity(oracle, ref, queries[3], want[3][0], want[3][1], Dref, Iref, TOL_FP32)

    # the index changes (the arena is replaced, lists move, ids go away): every lane has to see the new state
    x2, _ = make_data(92, 50000, 1, 64)
    ids2 = np.arange(10_000_000, 10_000_000 + len(x2), dtype=np.int64)
    gpu.add_with_ids(x2, ids2)
    gone = ids[::7]
    assert gpu.remove_ids(gone) == len(gone)
    ref2 = oracle.CsrIndex.build(64, 16, ix.METRIC_L2, ref.cent, ref.codebook,
                                 np.concatenate([np.delete(x, np.arange(0, len(x), 7), axis=0), x2]),
                                 np.concatenate([np.delete(ids, np.arange(0, len(ids), 7)), ids2]))
    want = concurrent_equal_serial(gpu, queries, k, nthreads=4, rounds=25)
    Dref, Iref = ref2.search(queries[3], k, 16)
    assert_topk_parity(oracle, ref2, queries[3], want[3][0], want[3][1], Dref, Iref, TOL_FP32)
    # large batches (the coarse stage's sampled-bound plan, the scan in locality order) beside small ones
    _, big = make_data(95, 1, 3000, 64)
    concurrent_equal_serial(gpu, [big, queries[3], np.ascontiguousarray(big[:2048]), queries[0]], k, nthreads=3, rounds=6)
    gpu.setNumProbes(4)
    want = concurrent_equal_serial(gpu, queries, k, nthreads=4, rounds=10)
    Dref, Iref = ref2.search(queries[2], k, 4)
    assert_topk_parity(oracle, ref2, queries[2], want[2][0], want[2][1], Dref, Iref, TOL_FP32)


def test_searches_beside_adds_and_removes_stay_valid(ix, oracle):
    """Writers take the lock exclusively between searches: every search sees one consistent state of the index."""
    gpu, ref, x, q, ids = build_pair(ix, oracle, 93, 30000, 64, 64, 128, 8, ix.METRIC_L2)
    gpu.setNumProbes(128)   # every list: the nearest stored vector is found whatever the state
    extra, _ = make_data(94, 6000, 1, 64)
    stop = threading.Event()
    added = []

    def body(t):
        if t == 0:
            for r in range(12):
                new_ids = np.arange(5_000_000 + 500 * r, 5_000_500 + 500 * r, dtype=np.int64)
                gpu.add_with_ids(extra[500 * r: 500 * (r + 1)], new_ids)
                added.append(new_ids)
                if r % 3 == 2:
                    assert gpu.remove_ids(added.pop(0)) == 500
            stop.set()
            return
        rounds = 0
        while not stop.is_set() or rounds < 5:
            D, I = gpu.search(q[8 * t: 8 * t + 8], 5)
            assert (I >= 0).all() and (np.diff(D, axis=1) >= 0).all()
            known = np.isin(I, ids) | ((I >= 5_000_000) & (I < 5_006_000))
            assert known.all(), f"thread {t}: a label that was never added"
            rounds += 1

    run_threads(4, body)
    assert gpu.ntotal == 30000 + 12 * 500 - 4 * 500
    # and afterwards the lanes agree with a search alone
    concurrent_equal_serial(gpu, [np.ascontiguousarray(q[:16]), np.ascontiguousarray(q[16:17])], 5, 4, 10)


@pytest.mark.parametrize("kind", ["int8", "fp32"])
def test_flat_searches_side_by_side_equal_searches_alone(ix, oracle, kind):
    """The Flat handles lock the same way: searches share the lock and run on lanes of their own, changes are exclusive."""
    rng = np.random.default_rng(5)
    d, n = 64, 30000
    if kind == "int8":
        base = rng.integers(-127, 128, size=(n, d), dtype=np.int8)
        q = rng.integers(-127, 128, size=(300, d), dtype=np.int8)
        index = ix.AscendIndexInt8Flat(d, ix.METRIC_L2)
        search = index.search_int32
        ref = lambda qq, kk, b, i: oracle.flat_i8(b, qq, kk, ids=i)
    else:
        base = rng.standard_normal((n, d)).astype(np.float32)
        q = rng.standard_normal((300, d)).astype(np.float32)
        index = ix.AscendIndexFlat(d, ix.METRIC_L2)
        search = index.search
        ref = lambda qq, kk, b, i: oracle.flat_f32(b, qq, kk, ids=i)
    ids = np.arange(n, dtype=np.int64) * 3 + 1
    index.add_with_ids(base[:20000], ids[:20000])
    queries = [np.ascontiguousarray(q[a:b]) for a, b in ((0, 1), (1, 9), (9, 50), (50, 300))]
    k = 10

    def check(b, i):
        want = [search(qq, k) for qq in queries]

        def body(t):
            for r in range(20):
                j = (t + r) % len(queries)
                D, I = search(queries[j], k)
                assert np.array_equal(I, want[j][1]) and np.array_equal(D.view(np.uint32), want[j][0].view(np.uint32)), (t, r, j)

        run_threads(5, body)
        Dr, Ir = ref(queries[2], k, b, i)
        assert np.array_equal(want[2][1], Ir) and np.array_equal(want[2][0].view(np.uint32), np.asarray(Dr).view(np.uint32))

    check(base[:20000], ids[:20000])
    index.add_with_ids(base[20000:], ids[20000:])       # the base is reallocated: every lane borrows again
    check(base, ids)
    assert index.remove_ids(ids[:100]) == 100
    D, I = search(queries[3], k)
    assert not np.isin(I, ids[:100]).any()
    want = [search(qq, k) for qq in queries]
    run_threads(4, lambda t: [np.testing.assert_array_equal(search(queries[(t + r) % 4], k)[1], want[(t + r) % 4][1]) for r in range(10)])


@pytest.fixture(scope="module")
def ix():
    import indexsdk_amd
    return indexsdk_amd
