"""A deterministic sweep over small random configurations of the IVFPQ search (dimensions, sub-quantizers,
list counts, probes, k, metric, LUT precision, batch size): each is checked against the CPU oracle.
Its purpose is breadth over the scan kernel's variants and LDS plans rather than depth in any of them."""
import numpy as np
import pytest

from tests.parity import assert_topk_parity
from tests.test_gpu_ivfpq import build_pair

pytestmark = pytest.mark.gpu


def _configs():
    rng = np.random.default_rng(20240)
    out = []
    ms = [1, 2, 4, 8, 12, 16, 24, 32, 48, 64, 96]
    for i in range(160):
        M = int(ms[i % len(ms)])
        dsub = int(rng.choice([1, 2, 4, 8]))
        d = M * dsub
        nlist = int(rng.choice([1, 7, 16, 40, 128]))
        nprobe = int(min(nlist, rng.choice([1, 3, 8, 32, 128])))
        k = int(rng.choice([1, 5, 10, 64, 100, 257, 600, 1024, 2048]))
        nq = int(rng.choice([1, 3, 17, 64, 130, 400, 2100]))
        metric_l2 = bool(rng.integers(0, 2))
        fp16 = bool(rng.integers(0, 2))
        layout = int(rng.choice([-1, -1, 0]))
        out.append((i, d, M, nlist, nprobe, k, nq, metric_l2, fp16, layout))
    return out


@pytest.mark.parametrize("seed,d,M,nlist,nprobe,k,nq,metric_l2,fp16,layout", _configs())
def test_search_sweep(oracle, seed, d, M, nlist, nprobe, k, nq, metric_l2, fp16, layout):
    import indexsdk_amd as ix
    metric = ix.METRIC_L2 if metric_l2 else ix.METRIC_INNER_PRODUCT
    n = 6000 if nq < 1000 else 3000
    gpu, ref, x, q, ids = build_pair(ix, oracle, 500 + seed, n, nq, d, nlist, M, metric, layout=layout, lut_fp16=int(fp16), niter=2)
    gpu.setNumProbes(nprobe)
    D, I = gpu.search(q, k)
    sub = slice(0, nq, max(1, nq // 150))
    Dr, Ir = ref.search(q[sub], k, nprobe, lut_fp16=fp16)
    assert_topk_parity(oracle, ref, q[sub], D[sub], I[sub], Dr, Ir, 1e-2 if fp16 else 1e-4)
    if sub == slice(0, nq, 1):
        assert gpu.last_search_stats()["scanned_codes"] == ref.last_scanned


def _flat_configs():
    rng = np.random.default_rng(777)
    out = []
    for i in range(40):
        d = int(rng.choice([32, 64, 96, 128, 256]))
        n = int(rng.choice([700, 2048, 2500, 4096, 9000, 20000, 30001]))
        nq = int(rng.choice([1, 5, 127, 128, 129, 256, 300]))
        k = int(rng.choice([1, 10, 100, 128, 300, 1000]))
        kind = int(rng.integers(0, 3))                 # 0: fp32 L2, 1: fp32 IP, 2: int8
        scratch = int(rng.choice([0, 0, 2 << 20, 8 << 20]))
        out.append((i, kind, d, n, nq, k, scratch))
    return out


@pytest.mark.parametrize("seed,kind,d,n,nq,k,scratch", _flat_configs())
def test_flat_sweep(oracle, seed, kind, d, n, nq, k, scratch):
    """Flat fp32 (L2, inner product) and int8 over base sizes on both sides of the kernels' shape limits
    (2048 rows for the matrix-core kernel, 4096 columns for the register row selection), query counts
    around the 128/256-row tile edges and both selection plans (whole base in the scratch, or streamed)."""
    import indexsdk_amd as ix
    rng = np.random.default_rng(9000 + seed)
    if kind == 2:
        base = rng.integers(-127, 128, size=(n, d), dtype=np.int8)
        q = rng.integers(-127, 128, size=(nq, d), dtype=np.int8)
        base[n // 3] = base[1]
        index = ix.AscendIndexInt8Flat(d, ix.METRIC_L2, scratch_bytes=scratch)
        index.add(base)
        D, I = index.search_int32(q, k)
        Dr, Ir = oracle.flat_i8(base, q, k)
        assert np.array_equal(I, Ir) and np.array_equal(D, Dr)
        return
    metric = ix.METRIC_L2 if kind == 0 else ix.METRIC_INNER_PRODUCT
    centres = rng.standard_normal((16, d)).astype(np.float32)
    base = (centres[rng.integers(0, 16, n)] + 0.3 * rng.standard_normal((n, d))).astype(np.float32)
    q = (centres[rng.integers(0, 16, nq)] + 0.3 * rng.standard_normal((nq, d))).astype(np.float32)
    index = ix.AscendIndexFlat(d, metric, scratch_bytes=scratch)
    index.add(base)
    D, I = index.search(q, k)
    Dr, Ir = oracle.flat_f32(base, q, k, metric)
    assert np.array_equal(I, Ir)
    assert np.array_equal(D.view(np.uint32), Dr.view(np.uint32))


def _coarse_configs():
    rng = np.random.default_rng(4242)
    out = []
    for i in range(36):
        d = int(rng.choice([32, 64, 100, 128]))
        nlist = int(rng.choice([300, 2048, 3000, 4096, 5000, 9000, 20000, 40000]))
        nprobe = int(min(nlist, rng.choice([1, 8, 64, 200, 320])))
        nq = int(rng.choice([1, 100, 257, 600]))
        metric_l2 = bool(rng.integers(0, 2))
        near_ties = bool(rng.integers(0, 4) == 0)
        out.append((i, d, nlist, nprobe, nq, metric_l2, near_ties))
    return out


@pytest.mark.parametrize("seed,d,nlist,nprobe,nq,metric_l2,near_ties", _coarse_configs())
def test_coarse_probe_sweep(oracle, seed, d, nlist, nprobe, nq, metric_l2, near_ties):
    """Probe ids and distances bit for bit over list counts on both sides of the matrix-core kernel's and
    the register selection's shape limits, with a few configurations of nearly coincident centroids (whose
    candidate lists cannot be proven complete and are redone exactly)."""
    import indexsdk_amd as ix
    metric = ix.METRIC_L2 if metric_l2 else ix.METRIC_INNER_PRODUCT
    rng = np.random.default_rng(7000 + seed)
    M = 4
    centres = rng.standard_normal((24, d)).astype(np.float32)
    spread = 1e-4 if near_ties else 0.4
    cent = (centres[rng.integers(0, 24, nlist)] + spread * rng.standard_normal((nlist, d))).astype(np.float32)
    q = (centres[rng.integers(0, 24, nq)] + 0.4 * rng.standard_normal((nq, d))).astype(np.float32)
    if not metric_l2:
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
    assert np.array_equal(gpu.assign(q), oracle.assign(q, cent))


@pytest.mark.parametrize("d,M,fp16", [(64, 16, 0), (64, 32, 0), (96, 48, 0), (192, 96, 1), (128, 64, 0)])
def test_write_side_random_sequences_against_a_host_model(oracle, d, M, fp16):
    """Random sequences of add, remove, update, add_codes and a file round trip, mirrored in a plain host
    model of the inverted lists (reference encoder, input order inside a list, survivors keep their
    order): after every step lists read back equal the model, under every code layout (row, rot32,
    xor48) whose byte order depends on the position inside the list."""
    import os
    import tempfile
    import indexsdk_amd as ix
    rng = np.random.default_rng(d * 7 + M)
    nlist = 12
    centres = rng.standard_normal((20, d)).astype(np.float32)

    def draw(n):
        return (centres[rng.integers(0, 20, n)] + 0.3 * rng.standard_normal((n, d))).astype(np.float32)

    x0 = draw(4000)
    cent, _ = oracle.kmeans(x0, nlist, niter=3, seed=3)
    cb = oracle.train_pq(x0, M, niter=2, seed=3)
    gpu = ix.AscendIndexIVFPQ(d, ix.METRIC_L2, nlist, M, 8, ix.AscendIndexIVFPQConfig(lut_fp16=fp16))
    gpu.set_trained(cent, cb)
    lists = [([], []) for _ in range(nlist)]          # per list: ids, codes (rows)
    next_id = [1000]

    def fresh_ids(n):
        out = np.arange(next_id[0], next_id[0] + n, dtype=np.int64) * 3 + 1
        next_id[0] += n
        return out

    def model_add(x, ids):
        asg = oracle.assign(x, cent)
        codes = oracle.pq_encode(x, cb)
        for i in range(len(ids)):
            lists[asg[i]][0].append(int(ids[i]))
            lists[asg[i]][1].append(codes[i])

    def model_remove(victims):
        vs = set(int(v) for v in victims)
        n = 0
        for l in range(nlist):
            keep = [j for j, v in enumerate(lists[l][0]) if v not in vs]
            n += len(lists[l][0]) - len(keep)
            lists[l] = ([lists[l][0][j] for j in keep], [lists[l][1][j] for j in keep])
        return n

    def check(which):
        assert gpu.ntotal == sum(len(l[0]) for l in lists)
        for l in which:
            codes, lid = gpu.getListCodesAndIds(l)
            assert lid.tolist() == lists[l][0], f"list {l}: ids differ"
            want = np.array(lists[l][1], dtype=np.uint8).reshape(-1, M)
            assert np.array_equal(codes, want), f"list {l}: codes differ"

    for step in range(14):
        op = ["add", "add", "remove", "update", "add_codes", "file"][int(rng.integers(0, 6))] if step else "add"
        present = np.array([v for l in lists for v in l[0]], dtype=np.int64)
        if op == "add":
            n = int(rng.integers(1, 1500))
            x, ids = draw(n), fresh_ids(n)
            gpu.add_with_ids(x, ids)
            model_add(x, ids)
        elif op == "remove" and len(present):
            victims = np.concatenate([rng.choice(present, min(len(present), int(rng.integers(1, 400))), replace=False),
                                      np.array([7, 8], dtype=np.int64)])          # two ids that do not exist
            assert gpu.remove_ids(victims) == model_remove(victims)
        elif op == "update" and len(present):
            ids = np.concatenate([rng.choice(present, min(len(present), int(rng.integers(1, 150))), replace=False),
                                  np.array([5], dtype=np.int64)])
            x = draw(len(ids))
            missing = gpu.update(x, ids)
            assert missing.tolist() == [5]
            model_remove(ids[:-1])
            model_add(x[:-1], ids[:-1])
        elif op == "add_codes":
            l, n = int(rng.integers(0, nlist)), int(rng.integers(1, 90))
            codes = rng.integers(0, 256, size=(n, M), dtype=np.uint8)
            ids = fresh_ids(n)
            gpu.add_codes(l, codes, ids)
            lists[l][0].extend(int(v) for v in ids)
            lists[l][1].extend(list(codes))
        elif op == "file":
            with tempfile.TemporaryDirectory() as tmp:
                path = os.path.join(tmp, "index.faiss")
                gpu.write_faiss(path)
                gpu = ix.AscendIndexIVFPQ.read_faiss(path, ix.AscendIndexIVFPQConfig(lut_fp16=fp16))
        check(rng.choice(nlist, 4, replace=False))
    check(range(nlist))
    # the lists as they stand, searched: parity with the oracle on the model's content
    off = np.zeros(nlist + 1, dtype=np.int64)
    np.cumsum([len(l[0]) for l in lists], out=off[1:])
    codes = np.concatenate([np.array(l[1], dtype=np.uint8).reshape(-1, M) for l in lists])
    ids = np.concatenate([np.array(l[0], dtype=np.int64) for l in lists])
    ref = oracle.CsrIndex(d, M, ix.METRIC_L2, cent, cb, off, codes, ids)
    q = draw(60)
    gpu.setNumProbes(5)
    D, I = gpu.search(q, 30)
    Dr, Ir = ref.search(q, 30, 5, lut_fp16=bool(fp16))
    assert_topk_parity(oracle, ref, q, D, I, Dr, Ir, 1e-2 if fp16 else 1e-4)


def test_search_with_more_queries_than_one_coarse_block(oracle):
    """40000 queries: the coarse stage walks them in blocks of 16384 rows (the score scratch never holds
    more), the scan takes them in one launch."""
    import indexsdk_amd as ix
    d, M, nlist, nq, nprobe, k = 32, 8, 4100, 40000, 6, 10
    rng = np.random.default_rng(31)
    centres = rng.standard_normal((50, d)).astype(np.float32)
    cent = (centres[rng.integers(0, 50, nlist)] + 0.5 * rng.standard_normal((nlist, d))).astype(np.float32)
    x = (centres[rng.integers(0, 50, 60000)] + 0.5 * rng.standard_normal((60000, d))).astype(np.float32)
    q = (centres[rng.integers(0, 50, nq)] + 0.5 * rng.standard_normal((nq, d))).astype(np.float32)
    cb = oracle.train_pq(x[:5000], M, niter=2, seed=1)
    gpu = ix.AscendIndexIVFPQ(d, ix.METRIC_L2, nlist, M, 8, ix.AscendIndexIVFPQConfig())
    gpu.set_trained(cent, cb)
    gpu.add(x)
    gpu.setNumProbes(nprobe)
    D, I = gpu.search(q, k)
    gi, gd = gpu.coarse_probe(q)
    oi, od = oracle.coarse_probe(q, cent, nprobe, ix.METRIC_L2)
    assert np.array_equal(gi, oi) and np.array_equal(gd.view(np.uint32), od.view(np.uint32))
    ref = oracle.CsrIndex.build(d, M, ix.METRIC_L2, cent, cb, x, np.arange(60000, dtype=np.int64))
    Dr, Ir = ref.search(q, k, nprobe)
    assert_topk_parity(oracle, ref, q, D, I, Dr, Ir, 1e-4)
    assert gpu.last_search_stats()["scanned_codes"] == ref.last_scanned
