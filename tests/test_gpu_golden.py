"""HIP path (through the C ABI) against the committed golden fixture."""
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ivfpq_small.npz")


@pytest.mark.parametrize("tag", ["l2", "ip"])
@pytest.mark.parametrize("lut16", [0, 1])
def test_ivfpq_matches_fixture(tag, lut16):
    import indexsdk_amd as ix
    g = np.load(GOLDEN, allow_pickle=False)
    metric = ix.METRIC_L2 if tag == "l2" else ix.METRIC_INNER_PRODUCT
    x, q = g["base"].astype(np.float32), g["queries"].astype(np.float32)
    d, M, nlist, k, nprobe = (int(g[n]) for n in ("d", "M", "nlist", "k", "nprobe"))
    index = ix.AscendIndexIVFPQ(d, metric, nlist, M, 8, ix.AscendIndexIVFPQConfig(lut_fp16=lut16))
    index.set_trained(g["centroids"], g["codebook"])
    index.add_with_ids(x, g["ids"])
    index.setNumProbes(nprobe)
    assert np.array_equal(index.assign(x), g["assign"])
    assert np.array_equal(index.encode(x), g["codes"])
    pi, pd = index.coarse_probe(q)
    assert np.array_equal(pi, g[f"probe_ids_{tag}"])
    assert np.array_equal(pd.view(np.uint32), g[f"probe_dist_{tag}"].view(np.uint32))
    D, I = index.search(q, k)
    suffix = "_lut16" if lut16 else ""
    Dg, Ig = g[f"D_{tag}{suffix}"], g[f"I_{tag}{suffix}"]
    # M = 8 uses the row code layout, whose accumulation order is the oracle's: bit-identical
    assert np.array_equal(D.view(np.uint32), Dg.view(np.uint32))
    assert np.array_equal(I, Ig)


LAYOUTS = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ivfpq_layouts.npz")


@pytest.mark.parametrize("tag,layout", [("m32", 1), ("m48", 2), ("m96", 1), ("m32", 0), ("m48", 0), ("m96", 0)])
def test_ivfpq_layouts_match_fixture(oracle, tag, layout):
    """32 sub-quantizers (rot32), 48 (xor48) and 96 with a half-precision LUT (rot32, paired blocks and
    64-byte rows) against the committed answers: codes and list assignment bit for bit; results through the
    tolerance of a re-associated sum, bit for bit under the row layout."""
    import indexsdk_amd as ix
    from tests.parity import assert_topk_parity
    g = np.load(LAYOUTS, allow_pickle=False)
    d, M, nlist, k, nprobe, metric, lut16 = (int(v) for v in g[f"{tag}_meta"])
    x, q = g[f"{tag}_base"].astype(np.float32), g[f"{tag}_queries"].astype(np.float32)
    cent, cb = g[f"{tag}_centroids"], g[f"{tag}_codebook"].astype(np.float32)
    index = ix.AscendIndexIVFPQ(d, metric, nlist, M, 8, ix.AscendIndexIVFPQConfig(lut_fp16=lut16, code_layout=layout))
    index.set_trained(cent, cb)
    index.add_with_ids(x, g[f"{tag}_ids"])
    index.setNumProbes(nprobe)
    assert np.array_equal(index.assign(x), g[f"{tag}_assign"])
    assert np.array_equal(index.encode(x), g[f"{tag}_codes"])
    D, I = index.search(q, k)
    Dg, Ig = g[f"{tag}_D"], g[f"{tag}_I"]
    if layout == 0:
        assert np.array_equal(D.view(np.uint32), Dg.view(np.uint32)) and np.array_equal(I, Ig)
    else:
        ref = oracle.CsrIndex.build(d, M, metric, cent, cb, x, g[f"{tag}_ids"])
        assert_topk_parity(oracle, ref, q, D, I, Dg, Ig, 1e-2 if lut16 else 1e-4)
