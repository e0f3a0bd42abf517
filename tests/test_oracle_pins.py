"""Pins the CPU oracle against independent facts (CPU only, no GPU, no product code).

The reference holds no golden vectors for the IVFPQ search path (its unit tests only assert error
strings and its system tests assert invariants), so each oracle function is pinned by what the
mathematics fixes: closed forms evaluated in float64, brute force, hand-computed cases that a
wrong accumulation order / sign / index would break, and the invariants the reference's own
system tests assert (self-query top-1, FR/test/ascend/TestAscendIndexIVFPQ.cpp:150-166; the AICPU
top-k recipe of random distances against a sorted ground truth, FR/test/aicpu/test_topk_flat.cc:52-187).
"""
import numpy as np
import pytest

FLT_MAX = np.finfo(np.float32).max


def rel_close(a, b, tol):
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    return np.abs(a - b) <= tol * np.maximum(np.maximum(np.abs(a), np.abs(b)), 1e-30)


# ----------------------------------------------------------------------------------------------
def test_f16_to_f32_all_patterns(oracle):
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = np.array([oracle.f16_to_f32(int(b)) for b in bits], dtype=np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_f32_to_f16_matches_numpy_rne(oracle):
    rng = np.random.default_rng(0)
    vals = np.concatenate([
        rng.standard_normal(4000).astype(np.float32) * np.float32(10.0) ** rng.integers(-9, 6, 4000),
        # exact halfway cases between adjacent halves (ties-to-even), subnormals, overflow edge
        np.array([1.0 + 2.0 ** -11, 1.0 + 3 * 2.0 ** -11, 2.0 ** -24, 2.0 ** -25, 3 * 2.0 ** -25, 65504.0, 65519.9,
                  65520.0, 1e9, -1e9, 0.0, -0.0, 6.1e-5, 5.96e-8, 2.98e-8, 2.9802322e-08], dtype=np.float32),
    ])
    with np.errstate(over="ignore"):
        want = vals.astype(np.float16).view(np.uint16)
    got = np.array([oracle.f32_to_f16(v) for v in vals], dtype=np.uint16)
    assert np.array_equal(got, want)


# ----------------------------------------------------------------------------------------------
def test_sqnorm_left_to_right_known_answer(oracle):
    # fp32: 2^24 + 1 rounds back to 2^24, so left-to-right gives 2^24; any pairwise / reversed
    # order that adds 1+1 first gives 2^24 + 2.
    x = np.array([[4096.0, 1.0, 1.0], [1.0, 1.0, 4096.0]], dtype=np.float32)
    got = oracle.sqnorms(x)
    assert got[0] == np.float32(16777216.0)
    assert got[1] == np.float32(16777218.0)


def test_coarse_dist_known_answers_and_closed_form(oracle):
    q = np.array([[1.0, 2.0]], dtype=np.float32)
    c = np.array([[3.0, 4.0], [1.0, 2.0], [-1.0, 0.5]], dtype=np.float32)
    l2 = oracle.coarse_dist(q, c, oracle.METRIC_L2)
    ip = oracle.coarse_dist(q, c, oracle.METRIC_INNER_PRODUCT)
    assert l2.tolist() == [[8.0, 0.0, 6.25]]
    assert ip.tolist() == [[11.0, 5.0, 0.0]]
    rng = np.random.default_rng(1)
    q = rng.standard_normal((37, 48)).astype(np.float32)
    c = rng.standard_normal((211, 48)).astype(np.float32)
    exact = ((q[:, None, :].astype(np.float64) - c[None].astype(np.float64)) ** 2).sum(-1)
    got = oracle.coarse_dist(q, c, oracle.METRIC_L2)
    scale = (q.astype(np.float64) ** 2).sum(1)[:, None] + (c.astype(np.float64) ** 2).sum(1)[None]
    assert np.all(np.abs(got - exact) <= 48 * 2 * np.finfo(np.float32).eps * scale)
    got_ip = oracle.coarse_dist(q, c, oracle.METRIC_INNER_PRODUCT)
    assert np.allclose(got_ip, q.astype(np.float64) @ c.astype(np.float64).T, atol=1e-4)


@pytest.mark.parametrize("metric_name", ["L2", "IP"])
def test_probe_select_is_full_stable_sort(oracle, metric_name):
    metric = oracle.METRIC_L2 if metric_name == "L2" else oracle.METRIC_INNER_PRODUCT
    rng = np.random.default_rng(2)
    c = rng.standard_normal((300, 16)).astype(np.float32)
    c[17] = c[5]           # exact duplicate centroids -> exact ties, smaller id must come first
    c[250] = c[5]
    c[100] = c[99]
    q = rng.standard_normal((50, 16)).astype(np.float32)
    q[0] = c[5]
    dist = oracle.coarse_dist(q, c, metric)
    key = -dist if metric_name == "IP" else dist
    order = np.argsort(key, axis=1, kind="stable")
    for nprobe in (1, 7, 64, 300):
        ids, d = oracle.coarse_probe(q, c, nprobe, metric)
        assert np.array_equal(ids, order[:, :nprobe])
        assert np.array_equal(d, np.take_along_axis(dist, order[:, :nprobe], axis=1))
    assert list(oracle.coarse_probe(q[:1], c, 3, metric)[0][0]) == [5, 17, 250]
    assert np.array_equal(oracle.assign(q, c), np.argsort(oracle.coarse_dist(q, c), axis=1, kind="stable")[:, 0])


def test_probe_select_aicpu_recipe(oracle):
    # d = 1, q = 0  =>  dist_j = c_j^2: arbitrary "random distances", ground truth by sorting
    rng = np.random.default_rng(3)
    c = rng.uniform(0.0, 100.0, size=(4096, 1)).astype(np.float32)
    q = np.zeros((3, 1), dtype=np.float32)
    ids, d = oracle.coarse_probe(q, c, 100)
    truth = np.argsort((c[:, 0] * c[:, 0]), kind="stable")[:100]
    assert np.array_equal(ids[1], truth)
    assert np.all(np.diff(d, axis=1) >= 0)


# ----------------------------------------------------------------------------------------------
def test_pq_encode_hand_cases(oracle):
    # dsub = 1, M = 2: codewords are integers, answers by inspection.
    cb = np.full((2, 256, 1), 1000.0, dtype=np.float32)
    cb[0, 3, 0], cb[0, 9, 0] = 2.0, 2.0        # duplicate codeword: first minimum (k=3) wins
    cb[0, 200, 0] = -5.0
    cb[1, 255, 0], cb[1, 0, 0] = 7.0, 9.0      # equidistant from 8.0: strict '<' keeps k=0
    x = np.array([[2.0, 8.0], [-4.0, 7.4], [2.1, 9.0]], dtype=np.float32)
    assert oracle.pq_encode(x, cb).tolist() == [[3, 0], [200, 255], [3, 0]]


def test_pq_encode_vs_float64_bruteforce(oracle):
    rng = np.random.default_rng(4)
    M, dsub, n = 8, 6, 500
    cb = rng.standard_normal((M, 256, dsub)).astype(np.float32)
    x = rng.standard_normal((n, M * dsub)).astype(np.float32)
    codes = oracle.pq_encode(x, cb)
    xs = x.reshape(n, M, 1, dsub).astype(np.float64)
    dist = ((xs - cb[None].astype(np.float64)) ** 2).sum(-1)          # [n, M, 256]
    best = dist.argmin(-1)
    diff = codes != best
    # any disagreement must be a float32-level near tie in the exact distances
    chosen = np.take_along_axis(dist, codes[..., None].astype(np.int64), -1)[..., 0]
    assert np.all(chosen[diff] - dist.min(-1)[diff] <= 1e-5 * dist.min(-1)[diff] + 1e-12)
    assert diff.mean() < 0.01


# ----------------------------------------------------------------------------------------------
@pytest.mark.parametrize("metric_name", ["L2", "IP"])
def test_lut_closed_form(oracle, metric_name):
    metric = oracle.METRIC_L2 if metric_name == "L2" else oracle.METRIC_INNER_PRODUCT
    rng = np.random.default_rng(5)
    M, dsub = 4, 8
    cb = rng.standard_normal((M, 256, dsub)).astype(np.float32)
    q = rng.standard_normal((9, M * dsub)).astype(np.float32)
    q[0, :dsub] = cb[0, 77]                       # q_m equals a codeword -> entry ~ 0 for L2
    got = oracle.lut(q, cb, metric)
    qs = q.reshape(9, M, 1, dsub).astype(np.float64)
    if metric_name == "L2":
        exact = ((qs - cb[None].astype(np.float64)) ** 2).sum(-1)
        scale = (qs ** 2).sum(-1) + (cb[None].astype(np.float64) ** 2).sum(-1)
        assert np.all(np.abs(got - exact) <= 4 * dsub * np.finfo(np.float32).eps * scale)
        assert abs(got[0, 0, 77]) <= 1e-5
    else:
        exact = (qs * cb[None].astype(np.float64)).sum(-1)
        assert np.allclose(got, exact, atol=1e-5)
    got16 = oracle.lut(q, cb, metric, lut_fp16=True)
    assert np.array_equal(got16, got.astype(np.float16).astype(np.float32))


def test_lut_known_answer(oracle):
    cb = np.zeros((1, 256, 2), dtype=np.float32)
    cb[0, 1] = [3.0, 4.0]
    q = np.array([[1.0, 2.0]], dtype=np.float32)
    l2 = oracle.lut(q, cb, oracle.METRIC_L2)
    assert l2[0, 0, 0] == 5.0 and l2[0, 0, 1] == 8.0       # |q|^2 and |q-c|^2 = 4 + 4
    assert oracle.lut(q, cb, oracle.METRIC_INNER_PRODUCT)[0, 0, 1] == 11.0


# ----------------------------------------------------------------------------------------------
def _small_index(oracle, metric, seed=6, n=3000, d=32, M=8, nlist=24, empty_lists=()):
    rng = np.random.default_rng(seed)
    centres = rng.standard_normal((12, d)).astype(np.float32)
    x = (centres[rng.integers(0, 12, n)] + 0.3 * rng.standard_normal((n, d))).astype(np.float32)
    cent, _ = oracle.kmeans(x, nlist, niter=5, seed=seed)
    cb = oracle.train_pq(x, M, niter=4, seed=seed)
    ids = rng.permutation(10 * n)[:n].astype(np.int64)
    list_no = oracle.assign(x, cent)
    keep = ~np.isin(list_no, list(empty_lists))
    idx = oracle.CsrIndex.from_assignment(d, M, metric, cent, cb, list_no[keep], oracle.pq_encode(x[keep], cb),
                                          ids[keep])
    return idx, x[keep], ids[keep], rng


@pytest.mark.parametrize("metric_name", ["L2", "IP"])
def test_search_against_numpy_ground_truth(oracle, metric_name):
    metric = oracle.METRIC_L2 if metric_name == "L2" else oracle.METRIC_INNER_PRODUCT
    idx, x, ids, rng = _small_index(oracle, metric)
    q = x[rng.integers(0, x.shape[0], 25)] + 0.05 * rng.standard_normal((25, idx.d)).astype(np.float32)
    nprobe, k = 5, 40
    D, I = idx.search(q, k, nprobe)
    probe, _ = oracle.coarse_probe(q, idx.cent, nprobe, metric)
    luts = oracle.lut(q, idx.codebook, metric)
    decode = idx.codebook[np.arange(idx.M)[None, :], idx.codes.astype(np.int64)].reshape(len(idx.codes), -1)
    for i in range(q.shape[0]):
        cand_pos = np.concatenate([np.arange(idx.list_off[l], idx.list_off[l + 1]) for l in probe[i]])
        # sequential fp32 accumulation over m, vectorised over candidates
        s = np.zeros(len(cand_pos), dtype=np.float32)
        for m in range(idx.M):
            s = s + luts[i, m, idx.codes[cand_pos, m]]
        key = -s if metric_name == "IP" else s
        order = np.argsort(key, kind="stable")[:k]       # ties -> (probe rank, position) order
        assert np.array_equal(I[i], idx.ids[cand_pos[order]])
        assert np.array_equal(D[i], s[order])
        # by_residual = false  =>  ADC distance is the distance to the reconstruction
        rec = decode[cand_pos[order]].astype(np.float64)
        qi = q[i].astype(np.float64)
        exact = (rec @ qi) if metric_name == "IP" else ((rec - qi) ** 2).sum(1)
        scale = (qi ** 2).sum() + (rec ** 2).sum(1)
        assert np.all(np.abs(D[i] - exact) <= 1e-5 * scale)
    assert idx.last_scanned == sum(int(idx.list_off[l + 1] - idx.list_off[l]) for l in probe.ravel())


def test_search_sentinels_and_self_query(oracle):
    idx, x, ids, rng = _small_index(oracle, oracle.METRIC_L2, seed=7, n=400, nlist=32)
    # k larger than what two probed lists can hold -> padded with (FLT_MAX, -1)
    D, I = idx.search(x[:6], 300, 2)
    probe, _ = oracle.coarse_probe(x[:6], idx.cent, 2)
    for i in range(6):
        cnt = sum(int(idx.list_off[l + 1] - idx.list_off[l]) for l in probe[i])
        assert cnt < 300
        assert np.all(I[i, cnt:] == -1) and np.all(D[i, cnt:] == FLT_MAX)
        assert np.all(I[i, :cnt] >= 0) and np.all(np.diff(D[i, :cnt]) >= 0)
    # IP pads with -FLT_MAX
    idx_ip, x_ip, _, _ = _small_index(oracle, oracle.METRIC_INNER_PRODUCT, seed=7, n=400, nlist=32)
    D, I = idx_ip.search(x_ip[:3], 300, 2)
    assert np.all(D[I == -1] == -FLT_MAX) and np.any(I == -1)
    # well-separated data: a database vector finds itself (its own code) at rank 1 distance-wise
    idx2, x2, ids2, _ = _small_index(oracle, oracle.METRIC_L2, seed=8, n=2000, d=32, M=16, nlist=16)
    D, I = idx2.search(x2[:200], 1, 16)
    own_code_dist = np.array([oracle.adc_list(oracle.lut(x2[i:i + 1], idx2.codebook)[0],
                                              oracle.pq_encode(x2[i:i + 1], idx2.codebook))[0] for i in range(200)])
    assert np.all(D[:, 0] <= own_code_dist)
    assert (I[:, 0] == ids2[:200]).mean() > 0.9


def test_search_empty_index_and_empty_probed_lists(oracle):
    idx, x, ids, _ = _small_index(oracle, oracle.METRIC_L2, seed=9, n=500, nlist=8, empty_lists=(0, 1, 2, 3, 4, 5, 6))
    D, I = idx.search(x[:4], 5, 8)
    assert np.all(I >= 0)
    empty = oracle.CsrIndex(idx.d, idx.M, idx.metric, idx.cent, idx.codebook, np.zeros(9, np.int64),
                            np.zeros((0, idx.M), np.uint8), np.zeros(0, np.int64))
    D, I = empty.search(x[:4], 5, 8)
    assert np.all(I == -1) and np.all(D == FLT_MAX)


# ----------------------------------------------------------------------------------------------
def test_flat_i8_exact(oracle):
    rng = np.random.default_rng(10)
    base = rng.integers(-127, 128, size=(700, 64), dtype=np.int8)
    base[5] = base[3]
    q = rng.integers(-127, 128, size=(9, 64), dtype=np.int8)
    q[0] = base[3]
    D, I = oracle.flat_i8(base, q, 20)
    exact = ((q[:, None, :].astype(np.int64) - base[None].astype(np.int64)) ** 2).sum(-1)
    order = np.argsort(exact, axis=1, kind="stable")[:, :20]
    assert np.array_equal(I, order)
    assert np.array_equal(D, np.take_along_axis(exact, order, 1).astype(np.int32))
    assert I[0, 0] == 3 and I[0, 1] == 5 and D[0, 0] == 0
    ids = np.arange(700, dtype=np.int64) * 3 + 1
    D2, I2 = oracle.flat_i8(base, q, 800, ids=ids)
    assert np.array_equal(I2[:, :700], ids[np.argsort(exact, axis=1, kind="stable")])
    assert np.all(I2[:, 700:] == -1) and np.all(D2[:, 700:] == np.iinfo(np.int32).max)


def test_flat_i8_extreme_values_fit_int32(oracle):
    base = np.full((2, 512), -127, dtype=np.int8)
    base[1] = 127
    q = np.full((1, 512), 127, dtype=np.int8)
    D, I = oracle.flat_i8(base, q, 2)
    assert D.tolist() == [[0, 512 * 254 * 254]] and I.tolist() == [[1, 0]]


@pytest.mark.parametrize("metric_name", ["L2", "IP"])
def test_flat_f32(oracle, metric_name):
    metric = oracle.METRIC_L2 if metric_name == "L2" else oracle.METRIC_INNER_PRODUCT
    rng = np.random.default_rng(11)
    base = rng.standard_normal((600, 24)).astype(np.float32)
    q = rng.standard_normal((7, 24)).astype(np.float32)
    D, I = oracle.flat_f32(base, q, 15, metric)
    dist = oracle.coarse_dist(q, base, metric)
    order = np.argsort(-dist if metric_name == "IP" else dist, axis=1, kind="stable")[:, :15]
    assert np.array_equal(I, order)
    assert np.array_equal(D, np.take_along_axis(dist, order, 1))


def test_kmeans_objective_decreases(oracle):
    # parity unpinned against faiss::Clustering; only the Lloyd invariant is checked
    rng = np.random.default_rng(12)
    x = rng.standard_normal((2000, 8)).astype(np.float32)
    objs = [oracle.kmeans(x, 16, niter=it, seed=5)[1] for it in (1, 2, 4, 8)]
    assert all(b <= a * (1 + 1e-6) for a, b in zip(objs, objs[1:]))
    cent, _ = oracle.kmeans(x, 16, niter=3, spherical=True, seed=5)
    assert np.allclose(np.linalg.norm(cent, axis=1), 1.0, atol=1e-5)


# ----------------------------------------------------------------------------------------------
def _device_lists(rng, ndev, n, k, metric_l2, ties=False, holes=0.0):
    """ndev sorted result lists per query, optionally with repeated distances and invalid labels."""
    d = rng.standard_normal((ndev, n, k)).astype(np.float32)
    if ties:
        d = np.round(d * 2) / 2
    d = np.sort(d, axis=2)
    if not metric_l2:
        d = d[:, :, ::-1].copy()
    lab = rng.permutation(ndev * n * k).reshape(ndev, n, k).astype(np.int64)
    if holes:
        lab[rng.random(lab.shape) < holes] = -1
    return d, lab


@pytest.mark.parametrize("metric_l2", [True, False])
def test_merge_results_equals_stable_sort_of_the_concatenation(oracle, metric_l2):
    """A k-way merge of sorted lists with a strict comparison, scanning the devices in order, is the
    stable sort of the device-major concatenation (FR/ascend/impl/AscendIndexImpl.cpp:587-640)."""
    rng = np.random.default_rng(7)
    d, lab = _device_lists(rng, 3, 40, 17, metric_l2, ties=True)
    metric = oracle.METRIC_L2 if metric_l2 else oracle.METRIC_INNER_PRODUCT
    got_d, got_l = oracle.merge_results(d, lab, metric)
    cat_d = np.concatenate(list(d), axis=1)
    cat_l = np.concatenate(list(lab), axis=1)
    order = np.argsort(cat_d if metric_l2 else -cat_d, axis=1, kind="stable")[:, :17]
    assert np.array_equal(got_d, np.take_along_axis(cat_d, order, 1))
    assert np.array_equal(got_l, np.take_along_axis(cat_l, order, 1))


def test_merge_results_skips_invalid_labels_anywhere_and_pads(oracle):
    d = np.array([[[1.0, 2.0, 3.0, 9.0]], [[0.5, 2.0, 2.5, 4.0]]], dtype=np.float32)
    lab = np.array([[[10, -1, 12, -1]], [[-1, 21, -1, -1]]], dtype=np.int64)
    got_d, got_l = oracle.merge_results(d, lab, oracle.METRIC_L2)
    assert got_l.tolist() == [[10, 21, 12, -1]]
    assert got_d.tolist() == [[1.0, 2.0, 3.0, float(FLT_MAX)]]
    # inner product: larger first, padding is still (FLT_MAX, -1)
    got_d, got_l = oracle.merge_results(d[:, :, ::-1].copy(), lab[:, :, ::-1].copy(), oracle.METRIC_INNER_PRODUCT)
    assert got_l.tolist() == [[12, 21, 10, -1]]
    assert got_d.tolist() == [[3.0, 2.0, 1.0, float(FLT_MAX)]]


def test_parity_rule_measures_cancelling_sums_against_their_terms(oracle):
    """tests/parity.py: term_scale is the sum of |LUT entries| of an id's code (brute force here), and
    assert_topk_parity accepts association noise on a sum that cancels but not a real error."""
    from tests.parity import assert_topk_parity, term_scale
    rng = np.random.default_rng(5)
    d = M = 8
    x = rng.standard_normal((200, d)).astype(np.float32)
    cent, _ = oracle.kmeans(x, 4, niter=2, seed=1)
    cb = oracle.train_pq(x, M, niter=2, seed=1)
    idx = oracle.CsrIndex.build(d, M, oracle.METRIC_INNER_PRODUCT, cent, cb, x)
    q = rng.standard_normal((3, d)).astype(np.float32)
    D, I = idx.search(q, 20, 4)
    lut = oracle.lut(q[:1], cb, oracle.METRIC_INNER_PRODUCT)[0]
    pos = {int(v): i for i, v in enumerate(idx.ids)}
    want = [sum(abs(float(lut[m, idx.codes[pos[int(i)]][m]])) for m in range(M)) for i in I[0, :5]]
    assert np.allclose(term_scale(oracle, idx, q[0], I[0, :5]), want, rtol=1e-12)
    # the entry closest to zero, moved by a few ulps of its terms: beyond 1e-4 of itself, within 1e-4 of the terms
    r = int(np.argmin(np.abs(D[0])))
    scale = term_scale(oracle, idx, q[0], [I[0, r]])[0]
    noisy = D.copy()
    noisy[0, r] += np.float32(3e-5 * scale)
    if abs(noisy[0, r] - D[0, r]) > 1e-4 * max(abs(noisy[0, r]), abs(D[0, r])):
        assert_topk_parity(oracle, idx, q, noisy, I, D, I, 1e-4)
    wrong = D.copy()
    wrong[0, r] += np.float32(1e-3 * scale)
    with pytest.raises(AssertionError):
        assert_topk_parity(oracle, idx, q, wrong, I, D, I, 1e-4)


def test_flat_remove_order_worked_examples(oracle):
    """The removal order of the Flat indexes, against sequences worked by hand from the reference's loop
    (highest position first, the last vector moves into the hole; Index.cpp:86-113): a vector can move
    twice, a removed last vector just leaves, repeats and positions past the end are ignored."""
    assert oracle.flat_remove_order(10, [2, 7]).tolist() == [0, 1, 8, 3, 4, 5, 6, 9]
    assert oracle.flat_remove_order(10, [8, 2]).tolist() == [0, 1, 9, 3, 4, 5, 6, 7]       # 9 -> 8 -> 2
    assert oracle.flat_remove_order(10, [1, 2]).tolist() == [0, 8, 9, 3, 4, 5, 6, 7]
    assert oracle.flat_remove_order(5, [4, 4, 9, -1]).tolist() == [0, 1, 2, 3]
    assert oracle.flat_remove_order(4, [0, 1, 2, 3]).tolist() == []
    assert oracle.flat_remove_order(6, [0]).tolist() == [5, 1, 2, 3, 4]
    assert oracle.flat_remove_order(3, []).tolist() == [0, 1, 2]
    # survivors are exactly the positions that were not named, each once
    rng = np.random.default_rng(3)
    for _ in range(20):
        n = int(rng.integers(1, 60))
        gone = rng.integers(0, n, int(rng.integers(0, n + 1)))
        order = oracle.flat_remove_order(n, gone)
        assert sorted(order.tolist()) == sorted(set(range(n)) - set(gone.tolist()))
        stay = [p for p in range(n - len(set(gone.tolist()))) if p not in set(gone.tolist())]
        assert all(order[p] == p for p in stay)        # a survivor below the new end never moves
