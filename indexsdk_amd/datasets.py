"""Seeded synthetic data for the benchmark configurations (numpy, host side).

The reference ships no data; its python harness reads SIFT1M from disk
(FR/test/python/datasets.py:71-84).  Here every configuration is a seeded mixture so that tests,
golden fixtures and the benchmark draw base, train and query vectors from the same distribution.
``scale`` shrinks the base/query counts for CI-sized twins; the distribution is unchanged.

``evaluate`` is the reference harness's recall measurement with the same contract, and ``ground_truth``
produces the exact-neighbour array it is measured against.
"""
import time

import numpy as np


def _mixture(rng, centres, sigma, n, weights=None):
    comp = rng.choice(centres.shape[0], size=n, p=weights)
    x = centres[comp] + sigma * rng.standard_normal((n, centres.shape[1]), dtype=np.float32)
    return x.astype(np.float32)


def gaussian_mixture(seed, n_base, n_query, d, n_comp, sigma, zipf=None):
    """Base and query vectors from one Gaussian mixture: centres ~ N(0, I), within-cluster sigma."""
    rng = np.random.default_rng(seed)
    centres = rng.standard_normal((n_comp, d), dtype=np.float32)
    weights = None
    if zipf is not None:
        weights = 1.0 / np.arange(1, n_comp + 1, dtype=np.float64) ** zipf
        weights /= weights.sum()
    return _mixture(rng, centres, sigma, n_base, weights), _mixture(rng, centres, sigma, n_query, weights)


def vmf_like_mixture(seed, n_base, n_query, d, n_comp, sigma):
    """Unit vectors: normalised Gaussian centres + N(0, sigma^2) noise, renormalised."""
    rng = np.random.default_rng(seed)
    centres = rng.standard_normal((n_comp, d), dtype=np.float32)
    centres /= np.linalg.norm(centres, axis=1, keepdims=True)

    def draw(n):
        x = _mixture(rng, centres, sigma, n)
        x /= np.linalg.norm(x, axis=1, keepdims=True)
        return x.astype(np.float32)

    return draw(n_base), draw(n_query)


def int8_uniform(seed, n_base, n_query, d):
    rng = np.random.default_rng(seed)
    return (rng.integers(-127, 128, size=(n_base, d), dtype=np.int8),
            rng.integers(-127, 128, size=(n_query, d), dtype=np.int8))


# name -> parameters of the five benchmark configurations (full size)
CONFIGS = {
    "C1": dict(kind="gauss", n=100_000, nq=1000, d=128, comp=64, sigma=0.3, nlist=256, M=16, nprobe=16, k=10,
               metric="L2", lut="fp32", seed=1235),
    "C2": dict(kind="gauss", n=10_000_000, nq=10_000, d=128, comp=1024, sigma=0.25, nlist=16384, M=32, nprobe=64,
               k=100, metric="L2", lut="fp32", seed=1236, ntrain=500_000),
    "C3": dict(kind="vmf", n=20_000_000, nq=4096, d=768, comp=4096, sigma=0.05, nlist=32768, M=96, nprobe=128,
               k=100, metric="IP", lut="fp16", seed=1237),
    "C4": dict(kind="int8", n=10_000_000, nq=2048, d=512, k=100, metric="L2", seed=1238),
    "C5": dict(kind="gauss", n=100_000_000, nq=1024, d=96, comp=256, sigma=0.25, zipf=1.1, nlist=65536, M=48,
               nprobe=256, k=1024, metric="L2", lut="fp32", seed=1239),
}


def make(name, scale=1.0, nq=None):
    """Return (base, queries) for configuration ``name`` with the base count scaled by ``scale``."""
    c = CONFIGS[name]
    n = max(1, int(c["n"] * scale))
    nq = int(nq if nq is not None else max(1, int(c["nq"] * min(1.0, scale * 10))))
    if c["kind"] == "gauss":
        return gaussian_mixture(c["seed"], n, nq, c["d"], c["comp"], c["sigma"], c.get("zipf"))
    if c["kind"] == "vmf":
        return vmf_like_mixture(c["seed"], n, nq, c["d"], c["comp"], c["sigma"])
    return int8_uniform(c["seed"], n, nq, c["d"])


def ground_truth(xb, xq, k=1, metric="L2", ids=None):
    """Exact k nearest neighbours of every query by brute force on the GPU (AscendIndexFlat, fp32):
    the ``gt`` array of ``evaluate``; ``gt[:, 0]`` is the true nearest neighbour.  The reference reads
    this array from SIFT1M's ground-truth file (FR/test/python/datasets.py:43-45)."""
    from . import ascendfaiss
    flat = ascendfaiss.AscendIndexFlat(xb.shape[1], ascendfaiss.METRIC_L2 if metric == "L2"
                                       else ascendfaiss.METRIC_INNER_PRODUCT)
    flat.add_with_ids(xb, ids)
    return flat.search(xq, k)[1]


def evaluate(index, xq, gt, k):
    """(milliseconds per query, {r: recall@r}) for r = 1, 10, 100, ... <= k, where recall@r is the
    fraction of queries whose true nearest neighbour ``gt[:, 0]`` is among the first r results of
    ``index.search(xq, k)`` -- the measure of the reference's harness (FR/test/python/datasets.py:71-84)."""
    nq = xq.shape[0]
    t0 = time.time()
    _, labels = index.search(xq, k)
    t1 = time.time()
    truth = np.asarray(gt)[:, :1]
    recalls = {}
    r = 1
    while r <= k:
        recalls[r] = float((labels[:, :r] == truth).any(axis=1).sum()) / nq
        r *= 10
    return (t1 - t0) * 1000.0 / nq, recalls
