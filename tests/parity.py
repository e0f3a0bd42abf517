"""Parity rules shared by the GPU tests (tie-aware comparison of top-k results)."""
import numpy as np

FLT_MAX = float(np.finfo(np.float32).max)


def rel_close(a, b, tol):
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    return np.abs(a - b) <= tol * np.maximum(np.maximum(np.abs(a), np.abs(b)), 1e-30)


def candidate_distances(orc, idx, q_row, ids, lut_fp16=False):
    """Oracle ADC distance of arbitrary database ids for one query (for the tie exemption)."""
    lut = orc.lut(q_row[None, :], idx.codebook, idx.metric, lut_fp16=lut_fp16)[0]
    pos = {int(v): i for i, v in enumerate(idx.ids)}
    out = []
    for i in ids:
        out.append(orc.adc_list(lut, idx.codes[pos[int(i)]][None, :])[0])
    return np.array(out, dtype=np.float32)


def assert_topk_parity(orc, idx, q, D_gpu, I_gpu, D_ref, I_ref, tol, lut_fp16=None):
    """Position-wise id equality; a mismatch is accepted only between candidates whose oracle
    distances tie within ``tol`` (relative), including across the k-th boundary.  Distances at
    equal rank must agree within ``tol``.  Returns the number of exempted positions."""
    assert D_gpu.shape == D_ref.shape and I_gpu.shape == I_ref.shape
    if lut_fp16 is None:
        lut_fp16 = tol > 1e-3          # the fp16-LUT tests are the ones that use the wide tolerance
    # padding must be identical
    assert np.array_equal(I_gpu == -1, I_ref == -1), "padding differs"
    pad = I_ref == -1
    assert np.array_equal(D_gpu[pad], D_ref[pad]), "sentinel distances differ"
    ok = rel_close(D_gpu, D_ref, tol) | pad
    assert ok.all(), f"distance mismatch beyond {tol}: {np.argwhere(~ok)[:5]}"
    exempt = 0
    for qi in np.argwhere((I_gpu != I_ref).any(axis=1))[:, 0]:
        bad = np.flatnonzero(I_gpu[qi] != I_ref[qi])
        # each id the GPU reports there must be a real candidate whose oracle distance ties with
        # the oracle's entry at that rank
        d_or = candidate_distances(orc, idx, q[qi], I_gpu[qi, bad], lut_fp16)
        assert rel_close(d_or, D_ref[qi, bad], tol).all(), f"query {qi}: non-tied id mismatch at ranks {bad}"
        assert len(set(I_gpu[qi][I_gpu[qi] >= 0].tolist())) == (I_gpu[qi] >= 0).sum(), "duplicate ids"
        exempt += len(bad)
    return exempt
