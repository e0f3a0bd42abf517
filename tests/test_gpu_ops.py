"""GPU parity tests of the stage operators (C ABI, device pointers) against the CPU oracle, bit for bit:
the reference's DistanceFlatL2MinsAtFP32, TopkFlatFp32 and AscendcIvfpqSubspaceDistance, and stages 2-4
on caller-supplied probe lists."""
import ctypes

import numpy as np
import pytest

pytestmark = pytest.mark.gpu
FLT_MAX = np.finfo(np.float32).max


class _Hip:
    """Device buffers through the HIP runtime itself (the one the library is linked against), so that the
    test depends on nothing but the library under test."""

    def __init__(self):
        self.rt = ctypes.CDLL("libamdhip64.so")
        self.rt.hipMalloc.argtypes = [ctypes.POINTER(ctypes.c_void_p), ctypes.c_size_t]
        self.rt.hipMemcpy.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int]
        self.rt.hipFree.argtypes = [ctypes.c_void_p]
        self.live = []

    def _ok(self, rc):
        assert rc == 0, f"HIP runtime call failed with {rc}"

    def empty(self, shape, dtype):
        a = np.empty(shape, dtype=dtype)
        p = ctypes.c_void_p()
        self._ok(self.rt.hipMalloc(ctypes.byref(p), max(a.nbytes, 16)))
        self.live.append(p)
        return _Buf(self, p, a.shape, a.dtype)

    def put(self, a):
        a = np.ascontiguousarray(a)
        b = self.empty(a.shape, a.dtype)
        self._ok(self.rt.hipMemcpy(b.ptr, a.ctypes.data, a.nbytes, 1))
        return b

    def close(self):
        self._ok(self.rt.hipDeviceSynchronize())
        for p in self.live:
            self.rt.hipFree(p)
        self.live = []


class _Buf:
    def __init__(self, hip, ptr, shape, dtype):
        self.hip, self.ptr, self.shape, self.dtype = hip, ptr, shape, dtype

    def get(self):
        self.hip._ok(self.hip.rt.hipDeviceSynchronize())
        out = np.empty(self.shape, dtype=self.dtype)
        self.hip._ok(self.hip.rt.hipMemcpy(out.ctypes.data, self.ptr, out.nbytes, 2))
        return out


@pytest.fixture()
def env():
    import indexsdk_amd as ix
    from indexsdk_amd import _capi
    hip = _Hip()
    yield hip, ix, _capi, _capi.load()
    hip.close()


def _p(b):
    return b.ptr


@pytest.mark.parametrize("batch,n,d", [(37, 1013, 96), (5, 64, 128), (3, 7, 30), (20, 4096, 64)])
def test_distance_flat_l2_mins(env, oracle, batch, n, d):
    hip, ix, _capi, lib = env
    rng = np.random.default_rng(batch + n)
    q = rng.standard_normal((batch, d)).astype(np.float32)
    c = rng.standard_normal((n, d)).astype(np.float32)
    c[n // 2] = c[0]                                   # a tie inside or across bursts
    sqr = oracle.sqnorms(c)
    bursts = (n + 63) // 64
    dq, dc, ds = hip.put(q), hip.put(c), hip.put(sqr)
    dist = hip.put(np.full((batch, n), -1.0, dtype=np.float32))
    mins = hip.put(np.zeros((batch, bursts * 2), dtype=np.float32))
    _capi.check(lib.ixa_op_distance_flat_l2_mins_fp32(_p(dq), batch, _p(dc), n, d, _p(ds), _p(dist), _p(mins), None))
    want = oracle.coarse_dist(q, c, oracle.METRIC_L2)
    got = dist.get()
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    m = mins.get().reshape(batch, bursts, 2)
    for b in range(bursts):
        seg = want[:, b * 64:(b + 1) * 64]
        assert np.array_equal(m[:, b, 0].view(np.uint32), seg.min(axis=1).view(np.uint32))
        assert np.array_equal(m[:, b, 1].view(np.uint32), seg.argmin(axis=1).astype(np.uint32))   # first minimum
    # min output is optional
    _capi.check(lib.ixa_op_distance_flat_l2_mins_fp32(_p(dq), batch, _p(dc), n, d, _p(ds), _p(dist), None, None))
    assert np.array_equal(dist.get().view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("batch,n,ld,k", [(33, 1013, 1013, 70), (4, 50, 64, 128), (9, 20000, 20000, 100),
                                          (6, 5000, 5120, 300), (2, 1, 4, 3), (5, 30000, 30000, 2048), (3, 3000, 3000, 1100)])
def test_topk_flat_fp32(env, batch, n, ld, k):
    hip, ix, _capi, lib = env
    rng = np.random.default_rng(n + k)
    d = np.round(rng.standard_normal((batch, ld)) * 50).astype(np.float32) / 8     # many exact ties
    dd = hip.put(d)
    out_d = hip.empty((batch, k), np.float32)
    out_l = hip.empty((batch, k), np.int64)
    _capi.check(lib.ixa_op_topk_flat_fp32(_p(dd), batch, n, ld, k, 1, _p(out_d), _p(out_l), None))
    order = np.argsort(d[:, :n], axis=1, kind="stable")[:, :k]
    want_l = np.full((batch, k), -1, dtype=np.int64)
    want_d = np.full((batch, k), FLT_MAX, dtype=np.float32)
    kk = min(n, k)
    want_l[:, :kk] = order
    want_d[:, :kk] = np.take_along_axis(d[:, :n], order, 1)
    assert np.array_equal(out_l.get(), want_l)
    assert np.array_equal(out_d.get().view(np.uint32), want_d.view(np.uint32))
    assert lib.ixa_op_topk_flat_fp32(_p(dd), batch, n, ld, k, 0, _p(out_d), _p(out_l), None) != 0   # asc only


@pytest.mark.parametrize("metric_name", ["L2", "IP"])
@pytest.mark.parametrize("batch,d,M", [(25, 128, 32), (3, 96, 48), (8, 768, 96), (2, 60, 12)])
def test_ivfpq_subspace_distance(env, oracle, metric_name, batch, d, M):
    hip, ix, _capi, lib = env
    metric = ix.METRIC_L2 if metric_name == "L2" else ix.METRIC_INNER_PRODUCT
    rng = np.random.default_rng(d + M)
    q = rng.standard_normal((batch, d)).astype(np.float32)
    cb = rng.standard_normal((M, 256, d // M)).astype(np.float32)
    q[0, : d // M] = cb[0, 17]                         # a query sub-vector equal to a codeword
    dq, dcb = hip.put(q), hip.put(cb)
    lut = hip.empty((batch, M, 256), np.float32)
    _capi.check(lib.ixa_op_ivfpq_subspace_distance(_p(dq), batch, d, _p(dcb), M, metric, _p(lut), None))
    want = oracle.lut(q, cb, metric)
    assert np.array_equal(lut.get().view(np.uint32), want.view(np.uint32))


def test_operators_chained_equal_the_fused_search(env, oracle):
    """Coarse distances -> top-nprobe -> stages 2-4 on those probes, one operator at a time, returns what
    the fused search returns (the probe SET is the same, and equal scores are ordered by slot)."""
    hip, ix, _capi, lib = env
    from tests.test_gpu_ivfpq import build_pair
    from tests.parity import assert_topk_parity
    nlist, nprobe, k = 96, 12, 40
    gpu, ref, x, q, ids = build_pair(ix, oracle, 71, 20000, 130, 64, nlist, 16, ix.METRIC_L2)
    gpu.setNumProbes(nprobe)
    D, I = gpu.search(q, k)
    cent, cb = gpu.get_trained()
    nq, d = q.shape
    dq, dc = hip.put(q), hip.put(cent)
    ds = hip.put(oracle.sqnorms(cent))
    dist = hip.empty((nq, nlist), np.float32)
    _capi.check(lib.ixa_op_distance_flat_l2_mins_fp32(_p(dq), nq, _p(dc), nlist, d, _p(ds), _p(dist), None, None))
    pd = hip.empty((nq, nprobe), np.float32)
    pl = hip.empty((nq, nprobe), np.int64)
    _capi.check(lib.ixa_op_topk_flat_fp32(_p(dist), nq, nlist, nlist, nprobe, 1, _p(pd), _p(pl), None))
    gi, gd = gpu.coarse_probe(q)
    assert np.array_equal(pl.get(), gi) and np.array_equal(pd.get().view(np.uint32), gd.view(np.uint32))
    probes_h = pl.get().astype(np.int32)
    probes = hip.put(probes_h)
    D2 = hip.empty((nq, k), np.float32)
    I2 = hip.empty((nq, k), np.int64)
    _capi.check(lib.ivfpq_search_probes_device(gpu._h, nq, _p(dq), _p(probes), nprobe, k, _p(D2), _p(I2)))
    assert np.array_equal(I2.get(), I) and np.array_equal(D2.get().view(np.uint32), D.view(np.uint32))
    Dr, Ir = ref.search(q, k, nprobe)
    assert_topk_parity(oracle, ref, q, D2.get(), I2.get(), Dr, Ir, 1e-4)
    # a probe list with holes: -1 entries, and values that name no list, are skipped
    holes = probes_h.copy()
    holes[:, ::2] = -1
    holes[:, ::4] = nlist
    holes[0, 0] = 2 ** 31 - 1
    holes[1, 0] = -(2 ** 31)
    _capi.check(lib.ivfpq_search_probes_device(gpu._h, nq, _p(dq), _p(hip.put(holes)), nprobe, k, _p(D2), _p(I2)))
    keep = np.ascontiguousarray(probes_h[:, 1::2])
    D3 = hip.empty((nq, k), np.float32)
    I3 = hip.empty((nq, k), np.int64)
    _capi.check(lib.ivfpq_search_probes_device(gpu._h, nq, _p(dq), _p(hip.put(keep)), keep.shape[1], k, _p(D3), _p(I3)))
    assert np.array_equal(I2.get(), I3.get())
    assert np.array_equal(D2.get().view(np.uint32), D3.get().view(np.uint32))
    # one list named twice is scanned twice: every result of the single scan comes back doubled, the two
    # copies next to each other (the two scans run in different workgroups here and meet in the split merge)
    one = np.ascontiguousarray(probes_h[:, :1])
    two = np.ascontiguousarray(np.repeat(one, 2, axis=1))
    kk = 16
    D1, I1 = hip.empty((nq, kk), np.float32), hip.empty((nq, kk), np.int64)
    Dd, Id = hip.empty((nq, 2 * kk), np.float32), hip.empty((nq, 2 * kk), np.int64)
    _capi.check(lib.ivfpq_search_probes_device(gpu._h, nq, _p(dq), _p(hip.put(one)), 1, kk, _p(D1), _p(I1)))
    _capi.check(lib.ivfpq_search_probes_device(gpu._h, nq, _p(dq), _p(hip.put(two)), 2, 2 * kk, _p(Dd), _p(Id)))
    assert gpu.last_search_stats()["nsplit"] == 2
    assert np.array_equal(Id.get(), np.repeat(I1.get(), 2, axis=1))
    assert np.array_equal(Dd.get().view(np.uint32), np.repeat(D1.get(), 2, axis=1).view(np.uint32))


def test_read_probe_reports_a_duration_and_rejects_bad_sizes(env):
    hip, ix, _capi, lib = env
    import ctypes
    buf = hip.empty((1 << 22,), np.float32)          # 16 MiB
    ms = ctypes.c_double(-1.0)
    _capi.check(lib.ixa_read_probe(_p(buf), (1 << 22) * 4, 3, ctypes.byref(ms)))
    assert 0.0 < ms.value < 50.0
    assert lib.ixa_read_probe(_p(buf), 24, 3, ctypes.byref(ms)) != 0            # not a multiple of 16
    assert lib.ixa_read_probe(_p(buf), 1 << 20, 0, ctypes.byref(ms)) != 0       # no passes
    assert lib.ixa_read_probe(None, 1 << 20, 1, ctypes.byref(ms)) != 0


@pytest.mark.parametrize("metric_name,M,k", [("L2", 16, 100), ("L2", 6, 320), ("IP", 8, 50)])
def test_scan_topk_operator_with_the_reference_operands_and_the_tile_merge(env, oracle, metric_name, M, k):
    """AscendcIvfpqSearchDistanceL2 with its own operands -- the LUT of the subspace operator, code and label base
    pointers with per-(query, block) offsets and sizes -- equals the oracle's search over the same lists (row
    order arithmetic: distances bit for bit); split over two tiles and merged by TopkIvfpqL3 it gives the same."""
    from tests.parity import assert_topk_parity
    hip, ix, _capi, lib = env
    metric = ix.METRIC_L2 if metric_name == "L2" else ix.METRIC_INNER_PRODUCT
    rng = np.random.default_rng(M + k)
    d, nlist, n, nq, nprobe = 48, 24, 30000, 41, 10
    x = rng.standard_normal((n, d)).astype(np.float32)
    q = rng.standard_normal((nq, d)).astype(np.float32)
    cent, _ = oracle.kmeans(x[:2000], nlist, niter=2, seed=1)
    cb = oracle.train_pq(x[:3000], M, niter=2, seed=1)
    ids = rng.permutation(10 * n)[:n].astype(np.int64)
    ref = oracle.CsrIndex.build(d, M, metric, cent, cb, x, ids)
    probes, _ = oracle.coarse_probe(q, cent, nprobe, metric)
    probes = probes.astype(np.int64)
    probes[3, 4] = probes[3, 5]                        # one list twice: scanned twice, as the reference would
    lens = (ref.list_off[1:] - ref.list_off[:-1]).astype(np.int64)
    code_off = (ref.list_off[:-1].astype(np.int64) * M)[probes]            # bytes from the code base
    label_off = ref.list_off[:-1].astype(np.int64)[probes]                 # elements from the label base
    sizes = lens[probes]
    sizes[5, 2] = 0                                     # a block the caller marks empty is skipped
    d_lut = hip.empty((nq, M, 256), np.float32)
    _capi.check(lib.ixa_op_ivfpq_subspace_distance(_p(hip.put(q)), nq, d, _p(hip.put(cb)), M, metric, _p(d_lut), None))
    d_codes, d_ids = hip.put(ref.codes), hip.put(ref.ids)
    out_v, out_l = hip.empty((nq, k), np.float32), hip.empty((nq, k), np.int64)
    _capi.check(lib.ixa_op_ivfpq_search_distance_topk(_p(d_lut), nq, M, _p(d_codes), _p(hip.put(code_off)),
                                                      _p(hip.put(sizes)), nprobe, k, _p(d_ids), _p(hip.put(label_off)),
                                                      metric, _p(out_v), _p(out_l), None))
    V, L = out_v.get(), out_l.get()
    # the oracle on the same (query, list) visits: per query, the union of its blocks
    for j in range(nq):
        cand_d, cand_i = [], []
        for b in range(nprobe):
            l, sz = probes[j, b], sizes[j, b]
            if sz == 0:
                continue
            s, e = ref.list_off[l], ref.list_off[l] + sz
            lut = oracle.lut(q[j:j + 1], cb, metric)[0]                    # [M][256]
            acc = np.zeros(e - s, dtype=np.float32)
            for m in range(M):
                acc = (acc + lut[m][ref.codes[s:e, m]]).astype(np.float32)
            cand_d.append(acc)
            cand_i.append(ref.ids[s:e])
        cd, ci = np.concatenate(cand_d), np.concatenate(cand_i)
        order = np.lexsort((np.arange(len(cd)), cd if metric == ix.METRIC_L2 else -cd))[:k]
        kk = len(order)
        assert np.array_equal(V[j, :kk].view(np.uint32), cd[order].view(np.uint32)), j
        same = L[j, :kk] == ci[order]
        assert same.all() or np.array_equal(np.sort(cd[order][~same]), np.sort(V[j, :kk][~same])), j   # ties only
        assert (L[j, kk:] == -1).all()
    # two tiles of five blocks each, merged
    tv, tl = hip.empty((2, nq, k), np.float32), hip.empty((2, nq, k), np.int64)
    for t in range(2):
        sl = slice(5 * t, 5 * t + 5)
        ov, ol = hip.empty((nq, k), np.float32), hip.empty((nq, k), np.int64)
        _capi.check(lib.ixa_op_ivfpq_search_distance_topk(
            _p(d_lut), nq, M, _p(d_codes), _p(hip.put(np.ascontiguousarray(code_off[:, sl]))),
            _p(hip.put(np.ascontiguousarray(sizes[:, sl]))), 5, k, _p(d_ids),
            _p(hip.put(np.ascontiguousarray(label_off[:, sl]))), metric, _p(ov), _p(ol), None))
        hip._ok(hip.rt.hipMemcpy(ctypes.c_void_p(tv.ptr.value + t * nq * k * 4), ov.ptr, nq * k * 4, 3))
        hip._ok(hip.rt.hipMemcpy(ctypes.c_void_p(tl.ptr.value + t * nq * k * 8), ol.ptr, nq * k * 8, 3))
    mv, ml = hip.empty((nq, k), np.float32), hip.empty((nq, k), np.int64)
    _capi.check(lib.ixa_op_topk_ivfpq_l3(_p(tl), _p(tv), 2, nq, k, k, 1 if metric == ix.METRIC_L2 else 0, _p(mv), _p(ml),
                                         None))
    MV, ML = mv.get(), ml.get()
    assert np.array_equal(MV.view(np.uint32), V.view(np.uint32))
    diff = ML != L
    assert not diff.any() or np.array_equal(np.sort(MV[diff]), np.sort(V[diff]))
    # refusals
    assert lib.ixa_op_ivfpq_search_distance_topk(_p(d_lut), nq, M, _p(d_codes), _p(hip.put(code_off)), _p(hip.put(sizes)),
                                                 nprobe, 385, _p(d_ids), _p(hip.put(label_off)), metric, _p(out_v),
                                                 _p(out_l), None) != 0
    assert lib.ixa_op_topk_ivfpq_l3(_p(tl), _p(tv), 2, nq, k, k + 1, 1, _p(mv), _p(ml), None) != 0
