"""Parity rules shared by the GPU tests (tie-aware comparison of top-k results)."""
import numpy as np

FLT_MAX = float(np.finfo(np.float32).max)


def rel_close(a, b, tol):
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    return np.abs(a - b) <= tol * np.maximum(np.maximum(np.abs(a), np.abs(b)), 1e-30)


def positions_of(idx, ids):
    """Rows of ``idx.codes`` that hold the given database ids.  The lookup (ids sorted once, then a binary
    search) is kept on the index object, so that an index of 10^8 vectors costs one sort, not one per query."""
    if getattr(idx, "_ids_sorter", None) is None or len(idx._ids_sorter) != len(idx.ids):
        idx._ids_sorter = np.argsort(idx.ids, kind="stable")
        idx._ids_sorted = idx.ids[idx._ids_sorter]
    ids = np.asarray(ids, dtype=np.int64)
    at = np.searchsorted(idx._ids_sorted, ids)
    assert (at < len(idx._ids_sorted)).all() and (idx._ids_sorted[at] == ids).all(), "an id that is not in the index"
    return idx._ids_sorter[at]


def candidate_distances(orc, idx, q_row, ids, lut_fp16=False):
    """Oracle ADC distance of arbitrary database ids for one query (for the tie exemption)."""
    lut = orc.lut(q_row[None, :], idx.codebook, idx.metric, lut_fp16=lut_fp16)[0]
    out = [orc.adc_list(lut, idx.codes[p][None, :])[0] for p in positions_of(idx, ids)]
    return np.array(out, dtype=np.float32)


def term_scale(orc, idx, q_row, ids, lut_fp16=False):
    """Sum of the |LUT entries| that make up the ADC distance of each id: the magnitude that the
    rounding of an fp32 sum is relative to.  For L2 every entry is (essentially) non-negative and this
    is the distance itself; for inner product the entries have both signs and the sum can cancel to
    almost nothing, where a different association order moves it by ulps of the entries, not of the sum."""
    lut = orc.lut(q_row[None, :], idx.codebook, idx.metric, lut_fp16=lut_fp16)[0].astype(np.float64)
    m = np.arange(lut.shape[0])
    return np.array([np.abs(lut[m, idx.codes[p]]).sum() for p in positions_of(idx, ids)])


def close_at_scale(orc, idx, q, I, a, b, tol, lut_fp16):
    """rel_close, and where that fails |a - b| <= tol x term_scale of the id at that position."""
    ok = rel_close(a, b, tol)
    for qi, r in np.argwhere(~ok):
        if I[qi, r] >= 0:
            scale = term_scale(orc, idx, q[qi], [I[qi, r]], lut_fp16)[0]
            ok[qi, r] = abs(float(a[qi, r]) - float(b[qi, r])) <= tol * scale
    return ok


def assert_topk_parity(orc, idx, q, D_gpu, I_gpu, D_ref, I_ref, tol, lut_fp16=None):
    """Position-wise id equality; a mismatch is accepted only between candidates whose oracle
    distances tie within ``tol`` (relative), including across the k-th boundary.  Distances at
    equal rank must agree within ``tol``, relative to the distance or, for sums that cancel (inner
    product), to the sum of the magnitudes of its terms.  Returns the number of exempted positions."""
    assert D_gpu.shape == D_ref.shape and I_gpu.shape == I_ref.shape
    if lut_fp16 is None:
        lut_fp16 = tol > 1e-3          # the fp16-LUT tests are the ones that use the wide tolerance
    # padding must be identical
    assert np.array_equal(I_gpu == -1, I_ref == -1), "padding differs"
    pad = I_ref == -1
    assert np.array_equal(D_gpu[pad], D_ref[pad]), "sentinel distances differ"
    ok = close_at_scale(orc, idx, q, I_ref, D_gpu, D_ref, tol, lut_fp16) | pad
    assert ok.all(), f"distance mismatch beyond {tol}: {np.argwhere(~ok)[:5]}"
    exempt = 0
    for qi in np.argwhere((I_gpu != I_ref).any(axis=1))[:, 0]:
        bad = np.flatnonzero(I_gpu[qi] != I_ref[qi])
        # each id the GPU reports there must be a real candidate whose oracle distance ties with
        # the oracle's entry at that rank
        d_or = candidate_distances(orc, idx, q[qi], I_gpu[qi, bad], lut_fp16)
        tied = rel_close(d_or, D_ref[qi, bad], tol)
        if not tied.all():
            scale = term_scale(orc, idx, q[qi], I_gpu[qi, bad], lut_fp16)
            tied |= np.abs(d_or.astype(np.float64) - D_ref[qi, bad]) <= tol * scale
        assert tied.all(), f"query {qi}: non-tied id mismatch at ranks {bad}"
        assert len(set(I_gpu[qi][I_gpu[qi] >= 0].tolist())) == (I_gpu[qi] >= 0).sum(), "duplicate ids"
        exempt += len(bad)
    return exempt
