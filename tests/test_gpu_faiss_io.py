"""faiss interchange files (fourcc IwPQ): write -> bytes equal to an independent restatement of
faiss::write_index's layout; read -> the same index (lists, ids, search results); rejects by_residual.

faiss itself is not installed here and the reference holds no stored index file, so the layout is
pinned only against the published faiss 1.10 writer restated below (parity with a real faiss build:
unpinned)."""
import struct

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def fourcc(s):
    return struct.pack("<I", s[0] | s[1] << 8 | s[2] << 16 | s[3] << 24)


def header(d, ntotal, metric):
    return struct.pack("<iqqqBi", d, ntotal, 1 << 20, 1 << 20, 1, metric)


def faiss_bytes(d, metric, nlist, M, nprobe, cent, cb, lists, by_residual=0):
    """lists: per list (codes [n, M] uint8, ids [n] int64).  faiss/impl/index_write.cpp, IndexIVFPQ branch."""
    ntotal = sum(len(i) for _, i in lists)
    out = [fourcc(b"IwPQ"), header(d, ntotal, metric), struct.pack("<QQ", nlist, nprobe)]
    out += [fourcc(b"IxF2" if metric == 1 else b"IxFI"), header(d, nlist, metric), struct.pack("<Q", nlist * d),
            cent.astype("<f4").tobytes()]
    out += [struct.pack("<BQ", 0, 0)]                                   # direct map: none, empty
    out += [struct.pack("<BQ", by_residual, M)]                         # by_residual, code_size
    out += [struct.pack("<QQQQ", d, M, 8, cb.size), cb.astype("<f4").tobytes()]
    out += [fourcc(b"ilar"), struct.pack("<QQ", nlist, M)]
    sizes = [len(i) for _, i in lists]
    if sum(s > 0 for s in sizes) > nlist // 2:
        out += [fourcc(b"full"), struct.pack("<Q", nlist), np.array(sizes, dtype="<u8").tobytes()]
    else:
        pairs = [v for l, s in enumerate(sizes) if s for v in (l, s)]
        out += [fourcc(b"sprs"), struct.pack("<Q", len(pairs)), np.array(pairs, dtype="<u8").tobytes()]
    for codes, ids in lists:
        if len(ids):
            out += [codes.tobytes(), ids.astype("<i8").tobytes()]
    return b"".join(out)


def small_index(ix, oracle, metric, n, nlist, seed, used_lists=None):
    rng = np.random.default_rng(seed)
    d, M = 32, 8
    x = rng.standard_normal((n, d)).astype(np.float32)
    cent, _ = oracle.kmeans(x, nlist, niter=3, seed=seed)
    if used_lists is not None:       # push most centroids far away so that their lists stay empty
        cent[used_lists:] += 100.0
    cb = oracle.train_pq(x, M, niter=3, seed=seed)
    index = ix.AscendIndexIVFPQ(d, metric, nlist, M, 8)
    index.set_trained(cent, cb)
    index.add_with_ids(x, rng.permutation(10 * n)[:n].astype(np.int64))
    index.setNumProbes(5)
    return index, x, cent, cb


def lists_of(index):
    return [index.getListCodesAndIds(l) if index.getListLength(l) else
            (np.empty((0, index.msubs), np.uint8), np.empty(0, np.int64)) for l in range(index.nlist)]


@pytest.mark.parametrize("metric_name,used", [("L2", None), ("IP", None), ("L2", 3)])
def test_write_matches_faiss_layout_and_round_trips(tmp_path, oracle, metric_name, used):
    import indexsdk_amd as ix
    metric = ix.METRIC_L2 if metric_name == "L2" else ix.METRIC_INNER_PRODUCT
    index, x, cent, cb = small_index(ix, oracle, metric, 3000, 16, 7, used)
    path = tmp_path / "a.faissindex"
    index.write_faiss(path)
    lists = lists_of(index)
    if used is not None:
        assert sum(len(i) > 0 for _, i in lists) <= 8           # the sparse size table is exercised
    expect = faiss_bytes(32, metric, 16, 8, 5, cent, cb, lists)
    assert path.read_bytes() == expect

    back = ix.AscendIndexIVFPQ.read_faiss(path)
    assert (back.d, back.metric_type, back.nlist, back.msubs) == (32, metric, 16, 8)
    assert back.ntotal == index.ntotal and back.getNumProbes() == 5 and back.is_trained
    for (c0, i0), (c1, i1) in zip(lists, lists_of(back)):
        assert np.array_equal(c0, c1) and np.array_equal(i0, i1)
    q = x[:200] + 0.01
    D0, I0 = index.search(q, 10)
    D1, I1 = back.search(q, 10)
    assert np.array_equal(I0, I1) and np.array_equal(D0.view(np.uint32), D1.view(np.uint32))
    # and a second generation file is byte-identical
    path2 = tmp_path / "b.faissindex"
    back.write_faiss(path2)
    assert path2.read_bytes() == expect


def test_read_rejects_by_residual_and_garbage(tmp_path, oracle):
    import indexsdk_amd as ix
    index, x, cent, cb = small_index(ix, oracle, ix.METRIC_L2, 2000, 16, 9)
    data = faiss_bytes(32, 1, 16, 8, 5, cent, cb, lists_of(index), by_residual=1)
    p = tmp_path / "res.faissindex"
    p.write_bytes(data)
    with pytest.raises(ix.IndexSdkError, match="by_residual"):
        ix.AscendIndexIVFPQ.read_faiss(p)
    p.write_bytes(b"IxF2" + data[4:])
    with pytest.raises(ix.IndexSdkError, match="IwPQ"):
        ix.AscendIndexIVFPQ.read_faiss(p)
    good = faiss_bytes(32, 1, 16, 8, 5, cent, cb, lists_of(index))
    p.write_bytes(good[:len(good) // 2])
    with pytest.raises(ix.IndexSdkError, match="truncated"):
        ix.AscendIndexIVFPQ.read_faiss(p)
    with pytest.raises(ix.IndexSdkError, match="cannot open"):
        ix.AscendIndexIVFPQ.read_faiss(tmp_path / "missing")
