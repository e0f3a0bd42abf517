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
