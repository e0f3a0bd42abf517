"""The reference's own acceptance grid for IVFPQ search as a parity test.

Its design document asks for nlist in {1024, 2048, 4096, 8192}, M in {2, 4, 8, 16}, d = 128, L2, batches of 1 to 64 and
top-k up to 320, with results within 1e-5 of the CPU implementation
(docs/rfc/26.1.0/IVFPQ...A2-A3...RFC.md:94-110; the parameter whitelists are FR/ascend/impl/AscendIndexIVFPQImpl.cpp:130-140,
510-525).  Every (nlist, M) pair of that grid is built here under `strict_reference_params` -- the library accepts
exactly the reference's envelope -- on quantizers shared with the oracle, and searched at batch 1 / 8 / 64 and
k 10 / 320: distances equal the oracle's bit for bit (these shapes use the `row` code layout, whose sums run in the
oracle's order), ids equal except between candidates whose distances tie.
"""
import numpy as np
import pytest

from tests.parity import assert_topk_parity

pytestmark = pytest.mark.gpu

D, N, NPROBE = 128, 60000, 64


def _data(seed):
    rng = np.random.default_rng(seed)
    centres = rng.standard_normal((200, D)).astype(np.float32)
    which = rng.integers(0, 200, N + 64)
    x = (centres[which] + 0.6 * rng.standard_normal((N + 64, D))).astype(np.float32)
    return x[:N], x[N:]


@pytest.mark.parametrize("nlist", [1024, 2048, 4096, 8192])
@pytest.mark.parametrize("M", [2, 4, 8, 16])
def test_reference_acceptance_grid(oracle, nlist, M):
    import indexsdk_amd as ix
    x, q = _data(nlist + M)
    rng = np.random.default_rng(nlist * 31 + M)
    # quantizers both sides share: centroids and codewords drawn from the data (how they were trained is not what
    # this test is about; the oracle's k-means at 8192 lists would take longer than everything else here)
    cent = x[rng.choice(N, nlist, replace=False)].copy()
    dsub = D // M
    cb = np.stack([x[rng.choice(N, 256, replace=False), m * dsub:(m + 1) * dsub] for m in range(M)]).copy()
    ref = oracle.CsrIndex.build(D, M, oracle.METRIC_L2, cent, cb, x)
    cfg = ix.AscendIndexIVFPQConfig(strict_reference_params=1)
    gpu = ix.AscendIndexIVFPQ(D, ix.METRIC_L2, nlist, M, 8, cfg)
    gpu.set_trained(cent, cb)
    gpu.add(x)
    assert gpu.code_layout() == 0
    gpu.setNumProbes(NPROBE)
    for batch in (1, 8, 64):
        for k in (10, 320):
            Dg, Ig = gpu.search(q[:batch], k)
            Dr, Ir = ref.search(q[:batch], k, NPROBE)
            assert np.array_equal(Dg.view(np.uint32), Dr.view(np.uint32)), f"batch {batch}, k {k}: distances differ"
            assert_topk_parity(oracle, ref, q[:batch], Dg, Ig, Dr, Ir, 1e-5)
            assert gpu.last_search_stats()["scanned_codes"] == ref.last_scanned
