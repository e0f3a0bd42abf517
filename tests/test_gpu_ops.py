"""GPU parity tests of the stage operators (C ABI, device pointers) against the CPU oracle, bit for bit:
the reference's DistanceFlatL2MinsAtFP32, TopkFlatFp32 and AscendcIvfpqSubspaceDistance, and stages 2-4
on caller-supplied probe lists."""
import ctypes

import numpy as np
import pytest

pytestmark = pytest.mark.gpu
FLT_MAX = np.finfo(np.float32).max


@pytest.fixture(scope="module")
def env():
    import torch
    import indexsdk_amd as ix
    from indexsdk_amd import _capi
    return torch, ix, _capi, _capi.load()


def _dev(torch, a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _p(t):
    return ctypes.c_void_p(t.data_ptr())


@pytest.mark.parametrize("batch,n,d", [(37, 1013, 96), (5, 64, 128), (3, 7, 30), (20, 4096, 64)])
def test_distance_flat_l2_mins(env, oracle, batch, n, d):
    torch, ix, _capi, lib = env
    rng = np.random.default_rng(batch + n)
    q = rng.standard_normal((batch, d)).astype(np.float32)
    c = rng.standard_normal((n, d)).astype(np.float32)
    c[n // 2] = c[0]                                   # a tie inside or across bursts
    sqr = oracle.sqnorms(c)
    bursts = (n + 63) // 64
    dq, dc, ds = _dev(torch, q), _dev(torch, c), _dev(torch, sqr)
    dist = torch.full((batch, n), -1.0, device="cuda")
    mins = torch.zeros((batch, bursts * 2), device="cuda")
    _capi.check(lib.ixa_op_distance_flat_l2_mins_fp32(_p(dq), batch, _p(dc), n, d, _p(ds), _p(dist), _p(mins), None))
    torch.cuda.synchronize()
    want = oracle.coarse_dist(q, c, oracle.METRIC_L2)
    got = dist.cpu().numpy()
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    m = mins.cpu().numpy().reshape(batch, bursts, 2)
    for b in range(bursts):
        seg = want[:, b * 64:(b + 1) * 64]
        assert np.array_equal(m[:, b, 0].view(np.uint32), seg.min(axis=1).view(np.uint32))
        assert np.array_equal(m[:, b, 1].view(np.uint32), seg.argmin(axis=1).astype(np.uint32))   # first minimum
    # min output is optional
    _capi.check(lib.ixa_op_distance_flat_l2_mins_fp32(_p(dq), batch, _p(dc), n, d, _p(ds), _p(dist), None, None))
    torch.cuda.synchronize()
    assert np.array_equal(dist.cpu().numpy().view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("batch,n,ld,k", [(33, 1013, 1013, 70), (4, 50, 64, 128), (9, 20000, 20000, 100),
                                          (6, 5000, 5120, 300), (2, 1, 4, 3)])
def test_topk_flat_fp32(env, batch, n, ld, k):
    torch, ix, _capi, lib = env
    rng = np.random.default_rng(n + k)
    d = np.round(rng.standard_normal((batch, ld)) * 50).astype(np.float32) / 8     # many exact ties
    dd = _dev(torch, d)
    out_d = torch.zeros((batch, k), device="cuda")
    out_l = torch.zeros((batch, k), device="cuda", dtype=torch.int64)
    _capi.check(lib.ixa_op_topk_flat_fp32(_p(dd), batch, n, ld, k, 1, _p(out_d), _p(out_l), None))
    torch.cuda.synchronize()
    order = np.argsort(d[:, :n], axis=1, kind="stable")[:, :k]
    want_l = np.full((batch, k), -1, dtype=np.int64)
    want_d = np.full((batch, k), FLT_MAX, dtype=np.float32)
    kk = min(n, k)
    want_l[:, :kk] = order
    want_d[:, :kk] = np.take_along_axis(d[:, :n], order, 1)
    assert np.array_equal(out_l.cpu().numpy(), want_l)
    assert np.array_equal(out_d.cpu().numpy().view(np.uint32), want_d.view(np.uint32))
    assert lib.ixa_op_topk_flat_fp32(_p(dd), batch, n, ld, k, 0, _p(out_d), _p(out_l), None) != 0   # asc only


@pytest.mark.parametrize("metric_name", ["L2", "IP"])
@pytest.mark.parametrize("batch,d,M", [(25, 128, 32), (3, 96, 48), (8, 768, 96), (2, 60, 12)])
def test_ivfpq_subspace_distance(env, oracle, metric_name, batch, d, M):
    torch, ix, _capi, lib = env
    metric = ix.METRIC_L2 if metric_name == "L2" else ix.METRIC_INNER_PRODUCT
    rng = np.random.default_rng(d + M)
    q = rng.standard_normal((batch, d)).astype(np.float32)
    cb = rng.standard_normal((M, 256, d // M)).astype(np.float32)
    q[0, : d // M] = cb[0, 17]                         # a query sub-vector equal to a codeword
    dq, dcb = _dev(torch, q), _dev(torch, cb)
    lut = torch.zeros((batch, M, 256), device="cuda")
    _capi.check(lib.ixa_op_ivfpq_subspace_distance(_p(dq), batch, d, _p(dcb), M, metric, _p(lut), None))
    torch.cuda.synchronize()
    want = oracle.lut(q, cb, metric)
    assert np.array_equal(lut.cpu().numpy().view(np.uint32), want.view(np.uint32))


def test_operators_chained_equal_the_fused_search(env, oracle):
    """Coarse distances -> top-nprobe -> stages 2-4 on those probes, one operator at a time, returns what
    the fused search returns (the probe SET is the same, and equal scores are ordered by slot)."""
    torch, ix, _capi, lib = env
    from tests.test_gpu_ivfpq import build_pair
    from tests.parity import assert_topk_parity
    nlist, nprobe, k = 96, 12, 40
    gpu, ref, x, q, ids = build_pair(ix, oracle, 71, 20000, 130, 64, nlist, 16, ix.METRIC_L2)
    gpu.setNumProbes(nprobe)
    D, I = gpu.search(q, k)
    cent, cb = gpu.get_trained()
    nq, d = q.shape
    dq, dc = _dev(torch, q), _dev(torch, cent)
    ds = _dev(torch, oracle.sqnorms(cent))
    dist = torch.empty((nq, nlist), device="cuda")
    _capi.check(lib.ixa_op_distance_flat_l2_mins_fp32(_p(dq), nq, _p(dc), nlist, d, _p(ds), _p(dist), None, None))
    pd = torch.empty((nq, nprobe), device="cuda")
    pl = torch.empty((nq, nprobe), device="cuda", dtype=torch.int64)
    _capi.check(lib.ixa_op_topk_flat_fp32(_p(dist), nq, nlist, nlist, nprobe, 1, _p(pd), _p(pl), None))
    torch.cuda.synchronize()
    gi, gd = gpu.coarse_probe(q)
    assert np.array_equal(pl.cpu().numpy(), gi) and np.array_equal(pd.cpu().numpy().view(np.uint32), gd.view(np.uint32))
    probes = pl.to(torch.int32).contiguous()
    D2 = torch.empty((nq, k), device="cuda")
    I2 = torch.empty((nq, k), device="cuda", dtype=torch.int64)
    _capi.check(lib.ivfpq_search_probes_device(gpu._h, nq, _p(dq), _p(probes), nprobe, k, _p(D2), _p(I2)))
    assert np.array_equal(I2.cpu().numpy(), I) and np.array_equal(D2.cpu().numpy().view(np.uint32), D.view(np.uint32))
    Dr, Ir = ref.search(q, k, nprobe)
    assert_topk_parity(oracle, ref, q, D2.cpu().numpy(), I2.cpu().numpy(), Dr, Ir, 1e-4)
    # a probe list with holes: -1 entries are skipped
    probes[:, ::2] = -1
    _capi.check(lib.ivfpq_search_probes_device(gpu._h, nq, _p(dq), _p(probes), nprobe, k, _p(D2), _p(I2)))
    keep = pl.cpu().numpy()[:, 1::2]
    gpu.setNumProbes(keep.shape[1])
    D3 = torch.empty((nq, k), device="cuda")
    I3 = torch.empty((nq, k), device="cuda", dtype=torch.int64)
    _capi.check(lib.ivfpq_search_probes_device(gpu._h, nq, _p(dq), _p(_dev(torch, keep.astype(np.int32))), keep.shape[1], k,
                                               _p(D3), _p(I3)))
    assert np.array_equal(I2.cpu().numpy(), I3.cpu().numpy())
    assert np.array_equal(D2.cpu().numpy().view(np.uint32), D3.cpu().numpy().view(np.uint32))
