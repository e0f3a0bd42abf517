#!/usr/bin/env python3
"""Generates tests/golden/ivfpq_small.npz: inputs and expected outputs of the IVFPQ path.

The reference holds no stored vectors for this path (its IVFPQ tests assert invariants only), and
its own sources cannot be built or imported here (they need faiss, CANN/AscendCL and the AscendC
toolchain).  The fixture is therefore produced by the CPU oracle (oracle/ivfpq_oracle.c), whose
functions are pinned one by one in tests/test_oracle_pins.py.  Its purpose is to freeze those
answers: a later change of the oracle or of the HIP path that alters any bit shows up against the
committed file.

Run from the repository root:  python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle import oracle as orc  # noqa: E402


def main():
    rng = np.random.default_rng(20240)
    d, M, nlist, n, nq, k, nprobe = 32, 8, 16, 1500, 24, 10, 4
    centres = rng.standard_normal((10, d)).astype(np.float32)
    x = (centres[rng.integers(0, 10, n)] + 0.3 * rng.standard_normal((n, d))).astype(np.float32)
    q = (centres[rng.integers(0, 10, nq)] + 0.3 * rng.standard_normal((nq, d))).astype(np.float32)
    # quantizers are rounded to 2^-10 so that the fixture stores them compactly and exactly
    cent = np.round(orc.kmeans(x, nlist, niter=5, seed=3)[0] * 1024) / 1024
    cb = np.round(orc.train_pq(x, M, niter=4, seed=3) * 1024) / 1024
    cent, cb = cent.astype(np.float32), cb.astype(np.float32)
    ids = rng.permutation(100000)[:n].astype(np.int64)
    out = dict(d=d, M=M, nlist=nlist, k=k, nprobe=nprobe, base=x.astype(np.float16), queries=q.astype(np.float16),
               centroids=cent, codebook=cb, ids=ids)
    # inputs are stored as float16 to keep the file small; the float32 widening of those halves IS the input
    x, q = out["base"].astype(np.float32), out["queries"].astype(np.float32)
    for metric, tag in ((orc.METRIC_L2, "l2"), (orc.METRIC_INNER_PRODUCT, "ip")):
        idx = orc.CsrIndex.build(d, M, metric, cent, cb, x, ids)
        out[f"assign"] = orc.assign(x, cent).astype(np.int32)
        out[f"codes"] = orc.pq_encode(x, cb)
        pi, pd = orc.coarse_probe(q, cent, nprobe, metric)
        out[f"probe_ids_{tag}"], out[f"probe_dist_{tag}"] = pi.astype(np.int32), pd
        out[f"lut_{tag}"] = orc.lut(q[:2], cb, metric)
        D, I = idx.search(q, k, nprobe)
        out[f"D_{tag}"], out[f"I_{tag}"] = D, I
        D16, I16 = idx.search(q, k, nprobe, lut_fp16=True)
        out[f"D_{tag}_lut16"], out[f"I_{tag}_lut16"] = D16, I16
    # flat int8 (exact int32) and flat fp32
    b8 = rng.integers(-127, 128, size=(300, 64), dtype=np.int8)
    q8 = rng.integers(-127, 128, size=(6, 64), dtype=np.int8)
    D8, I8 = orc.flat_i8(b8, q8, 12)
    out.update(flat_i8_base=b8, flat_i8_queries=q8, flat_i8_D=D8, flat_i8_I=I8)
    Df, If = orc.flat_f32(x[:400], q[:6], 12, orc.METRIC_L2)
    out.update(flat_f32_D=Df, flat_f32_I=If)
    path = os.path.join(ROOT, "tests", "golden", "ivfpq_small.npz")
    np.savez_compressed(path, **out)
    print(path, os.path.getsize(path), "bytes")


def layouts():
    """tests/golden/ivfpq_layouts.npz: the three shapes whose scan kernels re-order the code bytes and the
    LUT (32 sub-quantizers: rot32; 48: xor48; 96 with a half-precision LUT: rot32 with paired blocks and
    64-byte rows), as small as they can be.  Results do not depend on a layout; the fixture holds what the
    oracle returns, and the GPU test compares through the tolerance of a re-associated sum."""
    out = {}
    for tag, d, M, metric, lut16, seed in (("m32", 32, 32, orc.METRIC_L2, False, 1),
                                           ("m48", 48, 48, orc.METRIC_L2, False, 2),
                                           ("m96", 96, 96, orc.METRIC_INNER_PRODUCT, True, 3)):
        rng = np.random.default_rng(777 + seed)
        nlist, n, nq, k, nprobe = 8, 400, 12, 20, 3
        centres = rng.standard_normal((6, d)).astype(np.float32)
        x = (centres[rng.integers(0, 6, n)] + 0.3 * rng.standard_normal((n, d))).astype(np.float16)
        q = (centres[rng.integers(0, 6, nq)] + 0.3 * rng.standard_normal((nq, d))).astype(np.float16)
        xf, qf = x.astype(np.float32), q.astype(np.float32)
        if metric == orc.METRIC_INNER_PRODUCT:
            # unit vectors, as far as halves allow: the stored halves are the input
            x = (xf / np.linalg.norm(xf, axis=1, keepdims=True)).astype(np.float16)
            q = (qf / np.linalg.norm(qf, axis=1, keepdims=True)).astype(np.float16)
            xf, qf = x.astype(np.float32), q.astype(np.float32)
        cent = (np.round(orc.kmeans(xf, nlist, niter=4, seed=seed)[0] * 1024) / 1024).astype(np.float32)
        cb = (np.round(orc.train_pq(xf, M, niter=3, seed=seed) * 1024) / 1024).astype(np.float16)
        ids = rng.permutation(50000)[:n].astype(np.int64)
        idx = orc.CsrIndex.build(d, M, metric, cent, cb.astype(np.float32), xf, ids)
        D, I = idx.search(qf, k, nprobe, lut_fp16=lut16)
        out.update({f"{tag}_base": x, f"{tag}_queries": q, f"{tag}_centroids": cent, f"{tag}_codebook": cb,
                    f"{tag}_ids": ids, f"{tag}_codes": orc.pq_encode(xf, cb.astype(np.float32)),
                    f"{tag}_assign": orc.assign(xf, cent).astype(np.int32), f"{tag}_D": D, f"{tag}_I": I,
                    f"{tag}_meta": np.array([d, M, nlist, k, nprobe, metric, int(lut16)], dtype=np.int64)})
    path = os.path.join(ROOT, "tests", "golden", "ivfpq_layouts.npz")
    np.savez_compressed(path, **out)
    print(path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
    layouts()
