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
