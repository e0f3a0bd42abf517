"""The CPU oracle must reproduce the committed golden fixture bit for bit (CPU only)."""
import os

import numpy as np
import pytest

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ivfpq_small.npz")


@pytest.fixture(scope="module")
def g():
    return np.load(GOLDEN, allow_pickle=False)


def test_fixture_is_loadable_without_pickle(g):
    assert int(g["d"]) == 32 and g["base"].dtype == np.float16 and g["codes"].dtype == np.uint8


@pytest.mark.parametrize("tag", ["l2", "ip"])
def test_oracle_reproduces_fixture(oracle, g, tag):
    metric = oracle.METRIC_L2 if tag == "l2" else oracle.METRIC_INNER_PRODUCT
    x, q = g["base"].astype(np.float32), g["queries"].astype(np.float32)
    d, M, k, nprobe = int(g["d"]), int(g["M"]), int(g["k"]), int(g["nprobe"])
    assert np.array_equal(oracle.assign(x, g["centroids"]), g["assign"])
    assert np.array_equal(oracle.pq_encode(x, g["codebook"]), g["codes"])
    pi, pd = oracle.coarse_probe(q, g["centroids"], nprobe, metric)
    assert np.array_equal(pi, g[f"probe_ids_{tag}"]) and np.array_equal(pd, g[f"probe_dist_{tag}"])
    assert np.array_equal(oracle.lut(q[:2], g["codebook"], metric), g[f"lut_{tag}"])
    idx = oracle.CsrIndex.build(d, M, metric, g["centroids"], g["codebook"], x, g["ids"])
    D, I = idx.search(q, k, nprobe)
    assert np.array_equal(D, g[f"D_{tag}"]) and np.array_equal(I, g[f"I_{tag}"])
    D, I = idx.search(q, k, nprobe, lut_fp16=True)
    assert np.array_equal(D, g[f"D_{tag}_lut16"]) and np.array_equal(I, g[f"I_{tag}_lut16"])


def test_oracle_reproduces_flat_fixture(oracle, g):
    D, I = oracle.flat_i8(g["flat_i8_base"], g["flat_i8_queries"], 12)
    assert np.array_equal(D, g["flat_i8_D"]) and np.array_equal(I, g["flat_i8_I"])
    x, q = g["base"].astype(np.float32), g["queries"].astype(np.float32)
    D, I = oracle.flat_f32(x[:400], q[:6], 12, oracle.METRIC_L2)
    assert np.array_equal(D, g["flat_f32_D"]) and np.array_equal(I, g["flat_f32_I"])


LAYOUTS = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ivfpq_layouts.npz")


@pytest.mark.parametrize("tag", ["m32", "m48", "m96"])
def test_oracle_reproduces_layouts_fixture(oracle, tag):
    """32, 48 and 96 sub-quantizers (the shapes whose GPU kernels re-order code bytes and LUT)."""
    g = np.load(LAYOUTS, allow_pickle=False)
    d, M, nlist, k, nprobe, metric, lut16 = (int(v) for v in g[f"{tag}_meta"])
    x, q = g[f"{tag}_base"].astype(np.float32), g[f"{tag}_queries"].astype(np.float32)
    cent, cb = g[f"{tag}_centroids"], g[f"{tag}_codebook"].astype(np.float32)
    assert cent.shape == (nlist, d) and cb.shape == (M, 256, d // M)
    assert np.array_equal(oracle.assign(x, cent), g[f"{tag}_assign"])
    assert np.array_equal(oracle.pq_encode(x, cb), g[f"{tag}_codes"])
    idx = oracle.CsrIndex.build(d, M, metric, cent, cb, x, g[f"{tag}_ids"])
    D, I = idx.search(q, k, nprobe, lut_fp16=bool(lut16))
    assert np.array_equal(D, g[f"{tag}_D"]) and np.array_equal(I, g[f"{tag}_I"])
