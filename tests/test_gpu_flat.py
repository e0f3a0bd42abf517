"""GPU parity tests of the Flat paths (through the C ABI) against the CPU oracle.

int8: exact int32 distances and ids, bit for bit.  fp32: the final candidates are re-evaluated in
the canonical scalar arithmetic, so distances and ids equal the oracle's bit for bit as well.
"""
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ivfpq_small.npz")


@pytest.fixture(scope="module")
def ix():
    import indexsdk_amd
    return indexsdk_amd


@pytest.mark.parametrize("d,n,nq,k", [(64, 5000, 33, 10), (512, 20000, 130, 100), (96, 3000, 7, 128), (40, 1000, 5, 3),
                                      # query rows in every 128-row block of several 256-row tiles, with and
                                      # without the staged epilogue operands (nq % 4)
                                      (128, 9000, 516, 20), (256, 6000, 301, 7)])
def test_flat_i8_exact(ix, oracle, d, n, nq, k):
    rng = np.random.default_rng(d + n)
    base = rng.integers(-127, 128, size=(n, d), dtype=np.int8)
    base[17] = base[5]                 # exact duplicates: ties resolve to the vector added first
    q = rng.integers(-127, 128, size=(nq, d), dtype=np.int8)
    q[0] = base[5]
    ids = (np.arange(n, dtype=np.int64) * 7 + 3)
    # a small scratch forces several base chunks, exercising the streaming top-k
    index = ix.AscendIndexInt8Flat(d, ix.METRIC_L2, scratch_bytes=4 << 20)
    index.add_with_ids(base[: n // 2], ids[: n // 2])
    index.add_with_ids(base[n // 2:], ids[n // 2:])
    assert index.ntotal == n
    assert np.array_equal(index.getBase(3, 10), base[3:13])
    D, I = index.search_int32(q, k)
    Dr, Ir = oracle.flat_i8(base, q, k, ids=ids)
    assert np.array_equal(D, Dr)
    assert np.array_equal(I, Ir)
    assert D[0, 0] == 0 and I[0, 0] == ids[5] and I[0, 1] == ids[17]
    Df, If = index.search(q, k)
    assert np.array_equal(If, Ir) and np.array_equal(Df, Dr.astype(np.float32))


def test_flat_i8_extremes_and_padding(ix, oracle):
    base = np.full((3, 512), -127, dtype=np.int8)
    base[1] = 127
    q = np.full((2, 512), 127, dtype=np.int8)
    index = ix.AscendIndexInt8Flat(512)
    index.add(base)
    D, I = index.search_int32(q, 5)
    Dr, Ir = oracle.flat_i8(base, q, 5)
    assert np.array_equal(D, Dr) and np.array_equal(I, Ir)
    assert D[0].tolist() == [0, 512 * 254 * 254, 512 * 254 * 254, 2**31 - 1, 2**31 - 1]
    assert I[0].tolist() == [1, 0, 2, -1, -1]
    index.reset()
    assert index.ntotal == 0
    D, I = index.search_int32(q, 2)
    assert np.all(I == -1)


def test_flat_i8_golden(ix):
    g = np.load(GOLDEN, allow_pickle=False)
    index = ix.AscendIndexInt8Flat(64)
    index.add(g["flat_i8_base"])
    D, I = index.search_int32(g["flat_i8_queries"], 12)
    assert np.array_equal(D, g["flat_i8_D"]) and np.array_equal(I, g["flat_i8_I"])


@pytest.mark.parametrize("d", [64, 128, 256, 384, 512, 768, 1024])
def test_flat_i8_every_dimension_of_the_resident_kernel(ix, oracle, d):
    """The dimensions of the reference's Int8Flat (AscendIndexInt8FlatImpl.cpp:55), each a kernel instance of its own:
    a base long enough for the seeded stretch (stored scores) and several bound-filtered launches, queries in more
    than one query tile with a ragged last block, a base that ends inside a tile of 256 and inside a block of 32."""
    n, nq, k = 41000 + 77, 300, 20
    rng = np.random.default_rng(d)
    base = rng.integers(-127, 128, size=(n, d), dtype=np.int8)
    q = rng.integers(-127, 128, size=(nq, d), dtype=np.int8)
    q[:5] = base[[0, 255, 256, n - 1, 31999]]          # tile edges come back at distance 0
    base[n - 3] = base[100]                             # a tie across launches: the vector added first wins
    index = ix.AscendIndexInt8Flat(d, ix.METRIC_L2, scratch_bytes=4 << 20)
    index.add(base[:1000])
    index.add(base[1000:1037])                          # adds that start and end inside blocks of 32
    index.add(base[1037:])
    D, I = index.search_int32(q, k)
    Dr, Ir = oracle.flat_i8(base, q, k)
    assert np.array_equal(D, Dr) and np.array_equal(I, Ir)
    assert index.last_search_stats()["score_launches"] >= 3
    assert D[:5, 0].tolist() == [0] * 5 and I[:5, 0].tolist() == [0, 255, 256, n - 1, 31999]


def test_flat_i8_storage_in_matrix_core_order_round_trips(ix, oracle):
    """What goes into the tiled base comes back row-major, across blocks of 32 and tiles of 256, for a dimension
    that is padded (100 -> 128 bytes per row) and one that is not; removal moves vectors inside that layout."""
    rng = np.random.default_rng(3)
    for d in (100, 64):
        n = 3000 + 19
        base = rng.integers(-127, 128, size=(n, d), dtype=np.int8)
        index = ix.AscendIndexInt8Flat(d)
        for s, e in ((0, 1), (1, 33), (33, 300), (300, n)):
            index.add(base[s:e])
        assert np.array_equal(index.getBase(0, n), base)
        assert np.array_equal(index.getBase(31, 2), base[31:33])
        assert np.array_equal(index.getBase(250, 600), base[250:850])
        gone = np.array([0, 31, 32, 255, 256, 1000, n - 1, n - 40], dtype=np.int64)
        assert index.remove_ids(gone) == len(gone)
        order = oracle.flat_remove_order(n, np.sort(gone))
        assert np.array_equal(index.getBase(0, n - len(gone)), base[order])
        q = rng.integers(-127, 128, size=(9, d), dtype=np.int8)
        D, I = index.search_int32(q, 7)
        Dr, Ir = oracle.flat_i8(base[order], q, 7, ids=order.astype(np.int64))
        assert np.array_equal(D, Dr) and np.array_equal(I, Ir)


@pytest.mark.parametrize("metric_name", ["L2", "IP"])
@pytest.mark.parametrize("d,n,nq,k", [(128, 20000, 100, 10), (96, 7000, 40, 100), (30, 900, 9, 5), (64, 9000, 300, 10)])
def test_flat_f32_bit_exact(ix, oracle, metric_name, d, n, nq, k):
    metric = ix.METRIC_L2 if metric_name == "L2" else ix.METRIC_INNER_PRODUCT
    rng = np.random.default_rng(n + d)
    centres = rng.standard_normal((20, d)).astype(np.float32)
    base = (centres[rng.integers(0, 20, n)] + 0.3 * rng.standard_normal((n, d))).astype(np.float32)
    q = (centres[rng.integers(0, 20, nq)] + 0.3 * rng.standard_normal((nq, d))).astype(np.float32)
    index = ix.AscendIndexFlat(d, metric, scratch_bytes=2 << 20)
    index.add(base[: n // 3])
    index.add(base[n // 3:])
    D, I = index.search(q, k)
    Dr, Ir = oracle.flat_f32(base, q, k, metric)
    assert np.array_equal(I, Ir)
    assert np.array_equal(D.view(np.uint32), Dr.view(np.uint32))
    assert np.array_equal(index.getBase(10, 5), base[10:15])


def test_flat_f32_padding_and_golden(ix, oracle):
    g = np.load(GOLDEN, allow_pickle=False)
    x, q = g["base"].astype(np.float32), g["queries"].astype(np.float32)
    index = ix.AscendIndexFlatL2(32)
    index.add(x[:400])
    D, I = index.search(q[:6], 12)
    assert np.array_equal(D.view(np.uint32), g["flat_f32_D"].view(np.uint32)) and np.array_equal(I, g["flat_f32_I"])
    small = ix.AscendIndexFlatL2(32)
    small.add(x[:5])
    D, I = small.search(q[:3], 9)
    Dr, Ir = oracle.flat_f32(x[:5], q[:3], 9)
    assert np.array_equal(I, Ir) and np.array_equal(D, Dr)
    assert np.all(I[:, 5:] == -1) and np.all(D[:, 5:] == np.finfo(np.float32).max)


def test_flat_i8_many_fused_chunks_and_overflow_fallback(ix, oracle):
    # 150k rows: one seeded stretch through the score scratch, then several filtered chunks
    rng = np.random.default_rng(77)
    d, n, nq, k = 64, 150_000, 70, 50
    base = rng.integers(-127, 128, size=(n, d), dtype=np.int8)
    q = rng.integers(-127, 128, size=(nq, d), dtype=np.int8)
    index = ix.AscendIndexInt8Flat(d, ix.METRIC_L2, scratch_bytes=8 << 20)
    index.add(base)
    D, I = index.search_int32(q, k)
    Dr, Ir = oracle.flat_i8(base, q, k)
    assert np.array_equal(D, Dr) and np.array_equal(I, Ir)
    # adversarial order: every later row is closer to the query than all earlier ones, so the
    # filtered chunks admit everything and overflow their candidate buffers -> exact fallback path
    n2 = 60_000
    ramp = np.zeros((n2, d), dtype=np.int8)
    steps = np.linspace(127, 0, n2).astype(np.int64)
    ramp[:, 0] = steps.astype(np.int8)
    ramp[:, 1] = (np.arange(n2) % 100).astype(np.int8)      # breaks ties between equal first coordinates
    q2 = np.zeros((3, d), dtype=np.int8)
    index2 = ix.AscendIndexInt8Flat(d, ix.METRIC_L2)
    index2.add(ramp)
    D, I = index2.search_int32(q2, 20)
    Dr, Ir = oracle.flat_i8(ramp, q2, 20)
    assert np.array_equal(D, Dr) and np.array_equal(I, Ir)


def test_flat_f32_many_fused_chunks(ix, oracle):
    rng = np.random.default_rng(78)
    d, n, nq, k = 32, 120_000, 40, 20
    base = rng.standard_normal((n, d)).astype(np.float32)
    q = rng.standard_normal((nq, d)).astype(np.float32)
    for metric in (ix.METRIC_L2, ix.METRIC_INNER_PRODUCT):
        index = ix.AscendIndexFlat(d, metric, scratch_bytes=8 << 20)
        index.add(base)
        D, I = index.search(q, k)
        Dr, Ir = oracle.flat_f32(base, q, k, metric)
        assert np.array_equal(I, Ir) and np.array_equal(D.view(np.uint32), Dr.view(np.uint32))


@pytest.mark.parametrize("metric_name", ["L2", "IP"])
def test_flat_f32_near_duplicates_are_redone_exactly(ix, oracle, metric_name):
    """3000 base vectors within 1e-6 of each other: for queries near them the matrix-core scores can
    neither rank them nor prove a candidate list complete; those queries are redone from canonical
    scores of the whole base and every result still equals the oracle's bit for bit."""
    metric = ix.METRIC_L2 if metric_name == "L2" else ix.METRIC_INNER_PRODUCT
    rng = np.random.default_rng(71)
    d, n, nq, k = 64, 12000, 60, 20
    base = rng.standard_normal((n, d)).astype(np.float32)
    base[:3000] = base[0] + (1e-6 * rng.standard_normal((3000, d))).astype(np.float32)
    q = rng.standard_normal((nq, d)).astype(np.float32)
    q[:10] = base[0] + (0.05 * rng.standard_normal((10, d))).astype(np.float32)
    if metric == ix.METRIC_INNER_PRODUCT:
        q[:10] = 3.0 * base[0] + (0.05 * rng.standard_normal((10, d))).astype(np.float32)
    index = ix.AscendIndexFlat(d, metric)
    index.add(base)
    D, I = index.search(q, k)
    reruns = index.last_search_stats()["exact_reruns"]
    assert 10 <= reruns < nq, reruns
    Dr, Ir = oracle.flat_f32(base, q, k, metric)
    assert np.array_equal(I, Ir)
    assert np.array_equal(D.view(np.uint32), Dr.view(np.uint32))


# Score rows of 4096 .. 98304 columns with k <= 384 are selected from registers (bound from group
# minima); the cases below hold a ragged last segment, every group count, running keys from an
# earlier chunk, and rows of many equal scores, which overflow the candidate list and are redone by
# the streaming selection.
@pytest.mark.parametrize("n,k,scratch", [(20003, 100, 0), (20003, 300, 0), (33000, 150, 0), (40000, 60, 6 << 20)])
def test_flat_f32_rows_selected_from_registers(ix, oracle, n, k, scratch):
    d, nq = 64, 50
    rng = np.random.default_rng(n + k)
    centres = rng.standard_normal((30, d)).astype(np.float32)
    base = (centres[rng.integers(0, 30, n)] + 0.3 * rng.standard_normal((n, d))).astype(np.float32)
    q = (centres[rng.integers(0, 30, nq)] + 0.3 * rng.standard_normal((nq, d))).astype(np.float32)
    index = ix.AscendIndexFlat(d, ix.METRIC_L2, scratch_bytes=scratch)
    index.add(base)
    D, I = index.search(q, k)
    Dr, Ir = oracle.flat_f32(base, q, k, ix.METRIC_L2)
    assert np.array_equal(I, Ir)
    assert np.array_equal(D.view(np.uint32), Dr.view(np.uint32))


def test_flat_rows_of_equal_scores_overflow_the_register_selection(ix, oracle):
    d, n, nq, k = 64, 24000, 20, 100
    rng = np.random.default_rng(5)
    protos = rng.standard_normal((5, d)).astype(np.float32)
    base = protos[rng.integers(0, 5, n)]
    q = (protos[rng.integers(0, 5, nq)] + 0.05 * rng.standard_normal((nq, d))).astype(np.float32)
    index = ix.AscendIndexFlat(d, ix.METRIC_L2)
    index.add(base)
    D, I = index.search(q, k)
    Dr, Ir = oracle.flat_f32(base, q, k, ix.METRIC_L2)
    assert np.array_equal(I, Ir) and np.array_equal(D.view(np.uint32), Dr.view(np.uint32))
    b8 = rng.integers(-127, 128, size=(4, d), dtype=np.int8)[rng.integers(0, 4, n)]
    q8 = rng.integers(-127, 128, size=(nq, d), dtype=np.int8)
    i8 = ix.AscendIndexInt8Flat(d)
    i8.add(b8)
    D, I = i8.search_int32(q8, k)
    Dr, Ir = oracle.flat_i8(b8, q8, k)
    assert np.array_equal(I, Ir) and np.array_equal(D, Dr)


def test_flat_i8_rows_selected_from_registers(ix, oracle):
    d, n, nq, k = 64, 30001, 40, 200
    rng = np.random.default_rng(6)
    base = rng.integers(-127, 128, size=(n, d), dtype=np.int8)
    q = rng.integers(-127, 128, size=(nq, d), dtype=np.int8)
    index = ix.AscendIndexInt8Flat(d)
    index.add(base)
    D, I = index.search_int32(q, k)
    Dr, Ir = oracle.flat_i8(base, q, k)
    assert np.array_equal(I, Ir) and np.array_equal(D, Dr)


@pytest.mark.parametrize("n,nq,scratch", [(9000, 37, 0), (2049, 129, 1 << 20), (50000, 5, 4 << 20), (1500, 3, 0)])
def test_flat_largest_k(ix, oracle, n, nq, scratch):
    """k = 2048, the API's maximum, on all three Flat variants: the streaming selection then runs on two
    scanning wavefronts (four pools of 4096 keys do not fit LDS), over one block of the base or several,
    and with fewer rows than k the tail is padding."""
    d, k = 64, 2048
    rng = np.random.default_rng(n + nq)
    bi = rng.integers(-127, 128, size=(n, d), dtype=np.int8)
    qi = rng.integers(-127, 128, size=(nq, d), dtype=np.int8)
    bi[n // 3] = bi[1]
    index = ix.AscendIndexInt8Flat(d, ix.METRIC_L2, scratch_bytes=scratch)
    index.add(bi)
    D, I = index.search_int32(qi, k)
    Dr, Ir = oracle.flat_i8(bi, qi, k)
    assert np.array_equal(I, Ir) and np.array_equal(D, Dr)
    centres = rng.standard_normal((16, d)).astype(np.float32)
    base = (centres[rng.integers(0, 16, n)] + 0.3 * rng.standard_normal((n, d))).astype(np.float32)
    q = (centres[rng.integers(0, 16, nq)] + 0.3 * rng.standard_normal((nq, d))).astype(np.float32)
    base[n // 3] = base[1]
    for metric in (ix.METRIC_L2, ix.METRIC_INNER_PRODUCT):
        flat = ix.AscendIndexFlat(d, metric, scratch_bytes=scratch)
        flat.add(base)
        D, I = flat.search(q, k)
        Dr, Ir = oracle.flat_f32(base, q, k, metric)
        assert np.array_equal(I, Ir)
        assert np.array_equal(D.view(np.uint32), Dr.view(np.uint32))


@pytest.mark.parametrize("kind", ["fp32_L2", "fp32_IP", "int8"])
def test_flat_remove_ids_follows_the_reference_order(ix, oracle, kind):
    """remove_ids with a batch of ids (some absent, some repeated, some held by two vectors) and with an id
    range: the count, the storage order afterwards (getIdxMap / getBase: every hole, highest first, is
    refilled with the vector that is last at that moment; Index.cpp:86-113) and the searches on what is left
    equal the oracle's, and vectors added afterwards land behind the survivors."""
    rng = np.random.default_rng(31)
    d, n = 48, 30000
    if kind == "int8":
        index = ix.AscendIndexInt8Flat(d, ix.METRIC_L2, scratch_bytes=4 << 20)
        base = rng.integers(-127, 128, size=(n, d), dtype=np.int8)
        q = rng.integers(-127, 128, size=(40, d), dtype=np.int8)
    else:
        metric = ix.METRIC_L2 if kind == "fp32_L2" else ix.METRIC_INNER_PRODUCT
        index = ix.AscendIndexFlat(d, metric, scratch_bytes=4 << 20)
        base = rng.standard_normal((n, d)).astype(np.float32)
        q = rng.standard_normal((40, d)).astype(np.float32)
    ids = rng.permutation(10 * n)[:n].astype(np.int64)
    ids[100] = ids[7]                                   # one id held by two vectors: both leave
    index.add_with_ids(base[:20000], ids[:20000])
    index.add_with_ids(base[20000:], ids[20000:])

    def check(base, ids, k=12):
        assert index.ntotal == len(ids)
        assert np.array_equal(index.getIdxMap(), ids)
        assert np.array_equal(index.getBase(), base)
        if kind == "int8":
            D, I = index.search_int32(q, k)
            Dr, Ir = oracle.flat_i8(base, q, k, ids=ids)
            assert np.array_equal(D, Dr) and np.array_equal(I, Ir)
        else:
            D, I = index.search(q, k)
            Dr, Ir = oracle.flat_f32(base, q, k, index.metric_type, ids=ids)
            assert np.array_equal(I, Ir) and np.array_equal(D.view(np.uint32), Dr.view(np.uint32))

    check(base, ids)
    victims = np.concatenate([rng.choice(ids, 2500, replace=False), ids[-3:], [ids[7]], [-5, 10 * n + 1], ids[:4], ids[:4]])
    gone = np.nonzero(np.isin(ids, victims))[0]
    assert index.remove_ids(victims) == len(gone)
    order = oracle.flat_remove_order(n, gone)
    base, ids = base[order], ids[order]
    check(base, ids)
    assert index.remove_ids(np.array([-5], dtype=np.int64)) == 0 and index.remove_ids(np.empty(0, dtype=np.int64)) == 0
    lo, hi = 1000, 40000
    gone = np.nonzero((ids >= lo) & (ids < hi))[0]
    assert len(gone) > 1000 and index.remove_range(lo, hi) == len(gone)
    order = oracle.flat_remove_order(len(ids), gone)
    base, ids = base[order], ids[order]
    check(base, ids)
    assert index.remove_range(hi, lo) == 0
    extra = base[:50][::-1].copy()
    extra_ids = np.arange(50, dtype=np.int64) + 20 * n
    index.add_with_ids(extra, extra_ids)
    base, ids = np.concatenate([base, extra]), np.concatenate([ids, extra_ids])
    check(base, ids)
    assert index.remove_range(-1, 30 * n) == len(ids) and index.ntotal == 0      # everything leaves
    if kind == "int8":
        D, I = index.search_int32(q[:2], 3)
    else:
        D, I = index.search(q[:2], 3)
    assert (I == -1).all()


@pytest.mark.parametrize("kind", ["fp32_L2", "fp32_IP", "int8"])
def test_flat_search_with_masks(ix, oracle, kind):
    """search_with_masks: every query has its own bit mask over the storage positions (bit p % 8 of byte p / 8;
    FR/test/DTascendhost/TestAscendIndexInt8Flat.cpp:230-240 reads it that way); the answer is the oracle's
    brute force over the vectors that take part, bit for bit, with sentinels when fewer than k do.  A full
    mask gives the plain search; the base has a length that is no multiple of eight and spans several
    stretches of the score scratch."""
    rng = np.random.default_rng(61)
    d, n, nq, k = 40, 20003, 24, 30
    if kind == "int8":
        index = ix.AscendIndexInt8Flat(d, ix.METRIC_L2, scratch_bytes=1 << 20)
        base = rng.integers(-127, 128, size=(n, d), dtype=np.int8)
        q = rng.integers(-127, 128, size=(nq, d), dtype=np.int8)
        base[101] = base[7]                              # a tie across the mask
    else:
        metric = ix.METRIC_L2 if kind == "fp32_L2" else ix.METRIC_INNER_PRODUCT
        index = ix.AscendIndexFlat(d, metric, scratch_bytes=1 << 20)
        base = rng.standard_normal((n, d)).astype(np.float32)
        q = rng.standard_normal((nq, d)).astype(np.float32)
    ids = rng.permutation(5 * n)[:n].astype(np.int64)
    index.add_with_ids(base, ids)
    stride = (n + 7) // 8
    allowed = rng.random((nq, n)) < 0.5
    allowed[0] = True                                    # everything takes part
    allowed[1] = False                                   # nothing does
    allowed[2] = False
    allowed[2, rng.choice(n, 11, replace=False)] = True  # fewer than k
    allowed[3] = False
    allowed[3, -1] = True                                # only the last vector (a bit of the last, partial byte)
    allowed[4, 7] = False                                # of two equal vectors only the later one
    allowed[4, 101] = True
    mask = np.packbits(allowed, axis=1, bitorder="little")
    assert mask.shape == (nq, stride)
    if kind == "int8":
        q[4] = base[7]
        search = lambda qq, m: index.search_with_masks_int32(qq, k, m)
        plain = index.search_int32(q, k)
        brute = lambda sel, qq: oracle.flat_i8(base[sel], qq, k, ids=ids[sel])
    else:
        search = lambda qq, m: index.search_with_masks(qq, k, m)
        plain = index.search(q, k)
        brute = lambda sel, qq: oracle.flat_f32(base[sel], qq, k, index.metric_type, ids=ids[sel])
    D, I = search(q, mask)
    assert np.array_equal(I[0], plain[1][0]) and np.array_equal(D[0], plain[0][0])
    for i in range(nq):
        sel = np.nonzero(allowed[i])[0]
        if len(sel) == 0:
            assert (I[i] == -1).all()
            continue
        Dr, Ir = brute(sel, q[i:i + 1])
        assert np.array_equal(I[i], Ir[0]), i
        assert np.array_equal(D[i].view(np.uint32), Dr[0].view(np.uint32)), i
    assert (I[2, 11:] == -1).all() and (I[2, :11] >= 0).all()
    assert I[3, 0] == ids[-1] and (I[3, 1:] == -1).all()
    if kind == "int8":
        assert I[4, 0] == ids[101] and D[4, 0] == 0
    # the index answers plain searches as before
    again = index.search_int32(q, k) if kind == "int8" else index.search(q, k)
    assert np.array_equal(again[1], plain[1]) and np.array_equal(again[0], plain[0])


def test_flat_int8_mask_precision_recipe(ix, oracle):
    """The reference's own mask test (testMaskPrecision, FR/test/DTascendhost/TestAscendIndexInt8Flat.cpp:287-325):
    300000 vectors of 384 int8 (more than one 262144-row block of the reference), top 100, every second mask
    byte 255 and the others 0, for 1, 32 and 128 queries taken from the base.  Its check -- every label of the
    plain search that passes the mask is among the masked results with the same distance -- and the stricter
    one here: the masked results are the brute-force answer over the vectors that pass, bit for bit."""
    rng = np.random.default_rng(2024)
    n, d, k = 300_000, 384, 100
    base = rng.integers(-127, 128, size=(n, d), dtype=np.int8)
    index = ix.AscendIndexInt8Flat(d, ix.METRIC_L2)
    index.add(base)
    stride = (n + 7) // 8
    row = np.zeros(stride, dtype=np.uint8)
    row[1::2] = 255
    passes = np.unpackbits(row, bitorder="little")[:n].astype(bool)
    sel = np.nonzero(passes)[0]
    for nq in (1, 32, 128):
        q = base[:nq]
        mask = np.ascontiguousarray(np.broadcast_to(row, (nq, stride)))
        D, I = index.search_int32(q, k)
        Dm, Im = index.search_with_masks_int32(q, k, mask)
        for i in range(nq):
            keep = passes[I[i]]
            found = {int(l): int(v) for l, v in zip(Im[i], Dm[i])}
            assert all(found.get(int(l)) == int(v) for l, v in zip(I[i][keep], D[i][keep])), i
        Dr, Ir = oracle.flat_i8(base[sel], q, k, ids=sel.astype(np.int64))
        assert np.array_equal(Im, Ir) and np.array_equal(Dm, Dr)
        assert passes[Im].all()
