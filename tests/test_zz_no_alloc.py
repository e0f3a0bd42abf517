"""The entry point that allocates nothing, ivfpq_search_probes_device_noalloc, against
ivfpq_search_probes_device (C ABI, device pointers): the same ids and the same distance bit patterns, on
calls in a row that share the static device scratch -- a large batch (one workgroup per query, queries in
locality order), then a smaller one (queries split over workgroups, partial lists merged), then a size the
scratch cannot hold."""
import numpy as np
import pytest

from tests.test_gpu_ops import _Hip, _p

pytestmark = pytest.mark.gpu


@pytest.fixture()
def env():
    import indexsdk_amd as ix
    from indexsdk_amd import _capi
    hip = _Hip()
    yield hip, ix, _capi, _capi.load()
    hip.close()


def _both(hip, _capi, lib, gpu, dq, probes_h, n, k):
    nprobe = probes_h.shape[1]
    probes = hip.put(np.ascontiguousarray(probes_h[:n]))
    D0, I0 = hip.empty((n, k), np.float32), hip.empty((n, k), np.int64)
    D1, I1 = hip.empty((n, k), np.float32), hip.empty((n, k), np.int64)
    _capi.check(lib.ivfpq_search_probes_device(gpu._h, n, _p(dq), _p(probes), nprobe, k, _p(D0), _p(I0)))
    _capi.check(lib.ivfpq_search_probes_device_noalloc(gpu._h, n, _p(dq), _p(probes), nprobe, k, _p(D1), _p(I1)))
    return D0.get(), I0.get(), D1.get(), I1.get()


def test_no_alloc_entry_point_equals_the_allocating_one(env, oracle):
    hip, ix, _capi, lib = env
    from tests.test_gpu_ivfpq import build_pair
    nlist, nprobe = 128, 16
    gpu, ref, x, q, ids = build_pair(ix, oracle, 91, 40000, 3000, 64, nlist, 16, ix.METRIC_L2)
    gpu.setNumProbes(nprobe)
    probes_h, _ = gpu.coarse_probe(q)
    probes_h = probes_h.astype(np.int32)
    probes_h[2500, 3] = -1                   # holes and values that name no list are skipped by both
    probes_h[2501, 0] = nlist + 7
    dq = hip.put(q)
    # first call: 3000 queries, one workgroup each, locality order (order and histogram in the scratch)
    D0, I0, D1, I1 = _both(hip, _capi, lib, gpu, dq, probes_h, 3000, 50)
    assert np.array_equal(I0, I1) and np.array_equal(D0.view(np.uint32), D1.view(np.uint32))
    assert (I1[:, 0] >= 0).all()
    # second call, smaller: 20 queries split over 8 workgroups each (partial lists in the scratch)
    D0, I0, D1, I1 = _both(hip, _capi, lib, gpu, dq, probes_h, 20, 100)
    assert np.array_equal(I0, I1) and np.array_equal(D0.view(np.uint32), D1.view(np.uint32))
    assert gpu.last_search_stats()["nsplit"] == 8
    # and against the oracle: these rows hold the index's own probe lists, so its search is the reference
    from tests.parity import assert_topk_parity
    Dr, Ir = ref.search(q[:20], 100, nprobe)
    assert_topk_parity(oracle, ref, q[:20], D1, I1, Dr, Ir, 1e-4)
    # third call, again larger than the second
    D0, I0, D1, I1 = _both(hip, _capi, lib, gpu, dq, probes_h, 700, 10)
    assert np.array_equal(I0, I1) and np.array_equal(D0.view(np.uint32), D1.view(np.uint32))


def test_no_alloc_entry_point_refuses_what_the_scratch_cannot_hold(env, oracle):
    hip, ix, _capi, lib = env
    from tests.test_gpu_ivfpq import build_pair
    gpu, ref, x, q, ids = build_pair(ix, oracle, 92, 5000, 8, 32, 64, 8, ix.METRIC_L2)
    n, nprobe, k = 40000, 64, 10               # 4 * 40000 * 64 bytes of probe lists alone exceed 8 MiB
    probes = hip.put(np.zeros((n, nprobe), np.int32))
    dq = hip.put(np.zeros((n, 32), np.float32))
    D, I = hip.empty((n, k), np.float32), hip.empty((n, k), np.int64)
    rc = lib.ivfpq_search_probes_device_noalloc(gpu._h, n, _p(dq), _p(probes), nprobe, k, _p(D), _p(I))
    msg = lib.ixa_last_error().decode()
    assert rc == 2001 and "static scratch" in msg and str(8 << 20) in msg
    # the allocating entry point serves the same call
    _capi.check(lib.ivfpq_search_probes_device(gpu._h, n, _p(dq), _p(probes), nprobe, k, _p(D), _p(I)))
