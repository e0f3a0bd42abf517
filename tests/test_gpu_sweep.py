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
