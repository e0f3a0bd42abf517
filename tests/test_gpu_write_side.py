"""The write side at a million vectors: random sequences of add, add_codes, remove_ids, update, reserveMemory
and reclaimMemory against a plain host model of the inverted lists (reference encoder, input order inside a
list, survivors keep their order), with a position-dependent code layout, plus what makes the add path
amortised: lists extend in place, move one at a time when they outgrow their slack, and the arena is only
replaced now and then."""
import numpy as np
import pytest

from tests.parity import assert_topk_parity

pytestmark = pytest.mark.gpu


class ListModel:
    """Host model of the inverted lists: per list an id array and a code array, in list order."""

    def __init__(self, nlist, M):
        self.ids = [np.empty(0, np.int64) for _ in range(nlist)]
        self.codes = [np.empty((0, M), np.uint8) for _ in range(nlist)]
        self.nlist, self.M = nlist, M

    def add(self, asg, codes, ids):
        order = np.argsort(asg, kind="stable")          # input order inside a list
        asg_s = asg[order]
        starts = np.searchsorted(asg_s, np.arange(self.nlist + 1))
        for l in np.unique(asg_s):
            sel = order[starts[l]:starts[l + 1]]
            self.ids[l] = np.concatenate([self.ids[l], ids[sel]])
            self.codes[l] = np.concatenate([self.codes[l], codes[sel]])

    def remove(self, victims):
        gone = 0
        v = np.unique(victims)
        for l in range(self.nlist):
            if len(self.ids[l]) == 0:
                continue
            keep = ~np.isin(self.ids[l], v)
            gone += int((~keep).sum())
            if not keep.all():
                self.ids[l], self.codes[l] = self.ids[l][keep], self.codes[l][keep]
        return gone

    @property
    def ntotal(self):
        return sum(len(i) for i in self.ids)

    def present(self):
        return np.concatenate(self.ids)


def _check(gpu, model, lists):
    assert gpu.ntotal == model.ntotal
    for l in lists:
        codes, lid = gpu.getListCodesAndIds(int(l))
        assert np.array_equal(lid, model.ids[l]), f"list {l}: ids differ"
        assert np.array_equal(codes, model.codes[l]), f"list {l}: codes differ"


def test_random_write_sequences_at_a_million_vectors(oracle):
    import indexsdk_amd as ix
    d, M, nlist, n0 = 64, 32, 1024, 1_000_000          # 32 sub-quantizers: the rot32 code layout
    rng = np.random.default_rng(4242)
    centres = rng.standard_normal((64, d)).astype(np.float32)

    def draw(n):
        return (centres[rng.integers(0, 64, n)] + 0.35 * rng.standard_normal((n, d))).astype(np.float32)

    train = draw(40_000)
    cent, _ = oracle.kmeans(train, nlist, niter=3, seed=5)
    cb = oracle.train_pq(train[:8000], M, niter=2, seed=5)
    gpu = ix.AscendIndexIVFPQ(d, ix.METRIC_L2, nlist, M, 8, ix.AscendIndexIVFPQConfig(code_layout=1))
    gpu.set_trained(cent, cb)
    assert gpu.code_layout() == 1
    model = ListModel(nlist, M)
    next_id = [0]

    def fresh(n):
        out = np.arange(next_id[0], next_id[0] + n, dtype=np.int64) * 5 + 2
        next_id[0] += n
        return out

    def add(n):
        x, ids = draw(n), fresh(n)
        gpu.add_with_ids(x, ids)
        model.add(oracle.assign(x, cent), oracle.pq_encode(x, cb), ids)

    add(n0)
    _check(gpu, model, rng.integers(0, nlist, 24))
    allocated0 = gpu.arena_state()[0]
    replaced = 0
    for step in range(36):
        op = ["add", "add", "add_small", "add_codes", "remove", "update", "reserve", "reclaim"][int(rng.integers(0, 8))]
        before = gpu.arena_state()[0]
        if op == "add":
            add(int(rng.integers(1, 30_000)))
        elif op == "add_small":
            add(int(rng.integers(1, 200)))
        elif op == "add_codes":
            l, n = int(rng.integers(0, nlist)), int(rng.integers(1, 3000))
            codes, ids = rng.integers(0, 256, size=(n, M), dtype=np.uint8), fresh(n)
            gpu.add_codes(l, codes, ids)
            model.ids[l] = np.concatenate([model.ids[l], ids])
            model.codes[l] = np.concatenate([model.codes[l], codes])
        elif op == "remove":
            present = model.present()
            victims = np.concatenate([rng.choice(present, int(rng.integers(1, 6000)), replace=False),
                                      np.array([-7, 1], dtype=np.int64)])      # two ids that do not exist
            assert gpu.remove_ids(victims) == model.remove(victims)
        elif op == "update":
            present = model.present()
            ids = np.concatenate([rng.choice(present, int(rng.integers(1, 2500)), replace=False),
                                  np.array([3], dtype=np.int64)])
            x = draw(len(ids))
            assert gpu.update(x, ids).tolist() == [3]
            model.remove(ids[:-1])
            model.add(oracle.assign(x[:-1], cent), oracle.pq_encode(x[:-1], cb), ids[:-1])
        elif op == "reserve":
            gpu.reserveMemory(int(rng.integers(1000, 200_000)))
        else:
            released = gpu.reclaimMemory()
            slots, used, holes = gpu.arena_state()
            assert released >= 0 and holes == 0 and used <= slots
        replaced += gpu.arena_state()[0] != before and op not in ("reserve", "reclaim")
        _check(gpu, model, rng.integers(0, nlist, 16))
    _check(gpu, model, range(nlist))
    slots, used, holes = gpu.arena_state()
    assert used <= slots and holes <= used
    assert replaced <= 6, f"adds replaced the arena {replaced} times (first allocation: {allocated0} slots)"
    # and the index still answers like the oracle on the same lists
    off = np.zeros(nlist + 1, dtype=np.int64)
    np.cumsum([len(i) for i in model.ids], out=off[1:])
    ref = oracle.CsrIndex(d, M, ix.METRIC_L2, cent, cb, off, np.concatenate(model.codes), np.concatenate(model.ids))
    q = draw(300)
    gpu.setNumProbes(24)
    D, I = gpu.search(q, 50)
    Dr, Ir = ref.search(q, 50, 24)
    assert gpu.last_search_stats()["scanned_codes"] == ref.last_scanned
    assert_topk_parity(oracle, ref, q, D, I, Dr, Ir, 1e-4)


def test_many_small_adds_extend_lists_in_place(oracle):
    """400 adds of 250 vectors: a list extends in place while it has slack and moves alone when it has not;
    the arena is replaced a handful of times (geometric growth), not once per call."""
    import indexsdk_amd as ix
    d, M, nlist = 32, 8, 256
    rng = np.random.default_rng(11)
    x = rng.standard_normal((100_000, d)).astype(np.float32)
    cent, _ = oracle.kmeans(x[:20000], nlist, niter=3, seed=2)
    cb = oracle.train_pq(x[:5000], M, niter=2, seed=2)
    gpu = ix.AscendIndexIVFPQ(d, ix.METRIC_L2, nlist, M, 8, ix.AscendIndexIVFPQConfig())
    gpu.set_trained(cent, cb)
    model = ListModel(nlist, M)
    asg, codes = oracle.assign(x, cent), oracle.pq_encode(x, cb)
    sizes = set()
    for c in range(400):
        sl = slice(c * 250, (c + 1) * 250)
        ids = np.arange(sl.start, sl.stop, dtype=np.int64)
        gpu.add_with_ids(x[sl], ids)
        model.add(asg[sl], codes[sl], ids)
        sizes.add(gpu.arena_state()[0])
    _check(gpu, model, range(nlist))
    assert len(sizes) <= 16, f"the arena was replaced {len(sizes)} times in 400 adds"
    slots, used, holes = gpu.arena_state()
    assert used <= slots and holes * 2 <= used + 64 * nlist
    released = gpu.reclaimMemory()
    assert released > 0
    _check(gpu, model, range(0, nlist, 7))
    assert gpu.arena_state()[2] == 0


@pytest.mark.parametrize("layout", [0, 1])
def test_remove_by_id_range_equals_removing_those_ids(oracle, layout):
    """remove_ids(IDSelectorRange) (FR/ascend/impl/AscendIndexIVFImpl.cpp:432-440): the vectors whose id lies in
    [imin, imax) leave, every list keeps the order of its survivors, with a position-dependent code layout too;
    an empty or inverted range removes nothing."""
    import indexsdk_amd as ix
    d, M, nlist, n = 64, 32, 64, 60000
    rng = np.random.default_rng(77)
    x = rng.standard_normal((n, d)).astype(np.float32)
    cent, _ = oracle.kmeans(x[:8000], nlist, niter=3, seed=3)
    cb = oracle.train_pq(x[:4000], M, niter=2, seed=3)
    gpu = ix.AscendIndexIVFPQ(d, ix.METRIC_L2, nlist, M, 8, ix.AscendIndexIVFPQConfig(code_layout=layout))
    gpu.set_trained(cent, cb)
    ids = rng.permutation(4 * n)[:n].astype(np.int64)
    gpu.add_with_ids(x, ids)
    model = ListModel(nlist, M)
    model.add(oracle.assign(x, cent), oracle.pq_encode(x, cb), ids)
    assert gpu.remove_range(500, 500) == 0 and gpu.remove_range(900, 100) == 0
    lo, hi = 30000, 90000
    victims = ids[(ids >= lo) & (ids < hi)]
    assert len(victims) > 10000
    assert gpu.remove_range(lo, hi) == model.remove(victims) == len(victims)
    _check(gpu, model, range(nlist))
    assert gpu.remove_range(lo, hi) == 0
    assert gpu.remove_range(-10, 10 * n) == model.ntotal and gpu.ntotal == 0
