"""Host-only checks of the C ABI: the library loads, exports every symbol the header declares,
validates constructor parameters with the reference's messages, and refuses to run without a GPU
(no CPU fallback).  No search/add/train entry point is called here; the merge of per-device result
lists is host code in the reference too and is checked against the oracle."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "indexsdk_amd.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b((?:ixa|ivfpq|flat|flat_i8)_[a-z0-9_]+)\s*\(", text)))


@pytest.fixture(scope="module")
def capi():
    from indexsdk_amd import _capi
    if not os.path.exists(_capi.LIB_PATH):
        import __graft_entry__
        __graft_entry__.build()
    _capi.load()
    return _capi


def test_header_declares_the_index_level_boundary():
    names = declared_functions()
    for need in ["ivfpq_create", "ivfpq_destroy", "ivfpq_train", "ivfpq_set_trained", "ivfpq_add_with_ids",
                 "ivfpq_add_codes", "ivfpq_set_nprobe", "ivfpq_get_nprobe", "ivfpq_search", "ivfpq_assign",
                 "ivfpq_coarse_probe", "ivfpq_list_length", "ivfpq_get_list", "ivfpq_remove_ids", "ivfpq_reset",
                 "ixa_last_error", "ivfpq_last_error"]:
        assert need in names


def test_library_exports_every_declared_symbol(capi):
    lib = ctypes.CDLL(capi.LIB_PATH)
    missing = [n for n in declared_functions() if not hasattr(lib, n)]
    assert not missing, f"declared in the header but not exported: {missing}"
    unbound = [n for n in declared_functions() if n not in capi.exported_names()]
    assert not unbound, f"declared in the header but not bound in _capi.py: {unbound}"


def _create(capi, d, metric, nlist, M, nbits, strict=0):
    lib = capi.load()
    cfg = capi.IvfpqConfig()
    lib.ivfpq_config_default(ctypes.byref(cfg))
    cfg.strict_reference_params = strict
    h = ctypes.c_void_p()
    rc = lib.ivfpq_create(d, metric, nlist, M, nbits, ctypes.byref(cfg), ctypes.byref(h))
    return rc, lib.ixa_last_error().decode(), h


# FR/ut/TestAscendIndexUTIVFPQ.cpp:77-184: constructor validation messages
@pytest.mark.parametrize("args,strict,needle", [
    ((64, 1, 1024, 4, 8), 1, "Unsupported dims"),
    ((128, 1, 512, 4, 8), 1, "Unsupported nlists"),
    ((128, 1, 262144, 3, 8), 1, "Unsupported msubs"),
    ((128, 1, 524288, 3, 8), 1, "Unsupported msubs"),
    ((128, 1, 1024, 4, 4), 1, "Unsupported nbits"),
    ((128, 7, 1024, 4, 8), 1, "Unsupported metric type"),
    ((128, 1, 1024, 3, 8), 0, "Unsupported msubs"),       # 3 does not divide 128
    ((0, 1, 1024, 4, 8), 0, "Unsupported dims"),
    ((128, 1, 0, 4, 8), 0, "Unsupported nlists"),
])
def test_constructor_rejects_bad_parameters(capi, args, strict, needle):
    rc, msg, h = _create(capi, *args, strict=strict)
    assert rc == 2001 and needle in msg and not h.value


def test_large_nlist_passes_the_nlist_check(capi):
    # FR/ut/TestAscendIndexUTIVFPQ.cpp:122-145
    for nlist in (262144, 524288):
        rc, msg, _ = _create(capi, 128, 1, nlist, 3, 8, strict=1)
        assert "Unsupported nlists" not in msg and "Unsupported msubs" in msg


def test_null_handle_and_null_out_are_errors_not_crashes(capi):
    lib = capi.load()
    assert lib.ivfpq_search(None, 1, None, 1, None, None) == 2001
    assert "nullptr" in lib.ixa_last_error().decode()
    assert lib.ivfpq_create(128, 1, 1024, 4, 8, None, None) == 2001
    assert lib.ivfpq_destroy(None) == 0


def test_no_cpu_fallback(capi):
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    rc, msg, h = _create(capi, 128, 1, 1024, 4, 8)
    assert rc == 2016 and "no CPU path" in msg and not h.value


def test_product_never_imports_the_oracle():
    for dirpath, _, files in os.walk(os.path.join(ROOT, "indexsdk_amd")):
        for f in files:
            if f.endswith((".py", ".h", ".hip", ".cpp", ".sh")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text.lower(), f"{f} mentions the oracle"


# FR/ascend/impl/AscendIndexImpl.cpp:587-640: the merge of per-device results is host code in the
# reference and here; it is the one entry point that computes without a GPU.
@pytest.mark.parametrize("metric_l2,ndev,holes", [(True, 1, 0.0), (True, 4, 0.3), (False, 3, 0.2), (True, 2, 1.0)])
def test_merge_search_results_matches_the_oracle(capi, oracle, metric_l2, ndev, holes):
    import numpy as np
    import indexsdk_amd as ix
    rng = np.random.default_rng(11 + ndev)
    n, k = 300, 33
    d = np.sort(np.round(rng.standard_normal((ndev, n, k)) * 4).astype(np.float32) / 4, axis=2)
    if not metric_l2:
        d = d[:, :, ::-1].copy()
    lab = rng.permutation(ndev * n * k).reshape(ndev, n, k).astype(np.int64)
    lab[rng.random(lab.shape) < holes] = -1
    metric = ix.METRIC_L2 if metric_l2 else ix.METRIC_INNER_PRODUCT
    got_d, got_l = ix.merge_search_results(list(d), list(lab), metric)
    want_d, want_l = oracle.merge_results(d, lab, metric)
    assert np.array_equal(got_l, want_l) and np.array_equal(got_d.view(np.uint32), want_d.view(np.uint32))


def test_merge_search_results_rejects_bad_arguments(capi):
    lib = capi.load()
    rc = lib.ixa_merge_search_results(0, 1, 1, 1, None, None, None, None)
    assert rc != 0 and "ndev" in lib.ixa_last_error().decode()


def test_evaluate_counts_queries_whose_true_neighbour_is_in_the_first_r_results():
    """indexsdk_amd.datasets.evaluate (the reference harness's recall@r, FR/test/python/datasets.py:71-84)
    on a hand-made result list: true neighbours 7, 8, 9, 10; found at ranks 1, 3, 11 and never."""
    import numpy as np
    from indexsdk_amd.datasets import evaluate

    class Canned:
        def search(self, xq, k):
            lab = np.full((4, k), -1, dtype=np.int64)
            lab[0, 0] = 7
            lab[1, 2] = 8
            lab[2, 10] = 9
            lab[3, :] = np.arange(100, 100 + k)
            return np.zeros((4, k), dtype=np.float32), lab

    gt = np.array([[7, 1], [8, 2], [9, 3], [10, 4]], dtype=np.int64)
    ms, rec = evaluate(Canned(), np.zeros((4, 2), dtype=np.float32), gt, 100)
    assert ms >= 0 and rec == {1: 0.25, 10: 0.5, 100: 0.75}
    assert set(evaluate(Canned(), np.zeros((4, 2), dtype=np.float32), gt, 50)[1]) == {1, 10}


def _pool_capacity(k, waves, shared):
    """Keys a candidate pool must hold (the rule the selection code states: k plus two rounds of what the
    wavefronts that share the pool can append between prunes), as a power of two."""
    cap, need = (1024, k + 2 * waves * 64) if shared else (256, k + 2 * 64)
    while cap < need:
        cap *= 2
    return cap


def test_scan_lds_plan_keeps_every_region_inside_the_allocation(capi):
    """The fused scan kernel addresses its dynamic LDS through offsets the launcher computes by hand.  Over
    sub-quantizer counts, k, probe counts, splits, workgroup sizes, both pool kinds, both LUT types and every
    code layout: each region (LUT, query, candidate pools, list table, histogram, per-wave words + control
    block), sized here from what the kernel stores in it, ends inside the allocation, starts 16-byte aligned,
    and overlaps no other region."""
    lib = capi.load()
    plan = capi.ScanLdsPlan()
    checked = 0
    for M in (4, 8, 16, 32, 48, 64, 96, 128):
        for lut_fp16 in (0, 1):
            layouts = [0]
            if M in (32, 64, 96):
                layouts.append(1)
            if M == 48 and not lut_fp16:
                layouts.append(2)
            for layout in layouts:
                for k in (1, 10, 100, 128, 129, 160, 256, 300, 320, 384, 385, 1000, 1024, 1408, 1409, 2048):
                    for nprobe, nsplit in ((1, 1), (16, 1), (64, 8), (256, 1), (2048, 1), (2048, 8), (100, 3)):
                        for waves, shared in ((0, 0), (4, 0), (8, 0), (8, 1), (16, 1)):
                            d = M * 4
                            rc = lib.ivfpq_plan_scan_lds(d, M, lut_fp16, layout, nprobe, nsplit, k, waves, shared,
                                                         ctypes.byref(plan))
                            assert rc == 0, lib.ixa_last_error()
                            W, sh = plan.waves, plan.shared_pool
                            if waves:
                                assert (W, sh) == (waves, shared)
                            assert plan.cap == _pool_capacity(k, W, sh)
                            assert plan.table_n == -(-nprobe // nsplit)
                            lut = 64 * 256 * 4 if layout == 2 else M * 256 * (2 if lut_fp16 else 4)
                            if layout == 1 and lut_fp16:
                                lut += 64          # the upper half of the last row's sub-quantizers 16..31
                            regions = [
                                ("lut", 0, lut),
                                ("query", plan.off_query, d * 4),
                                ("pools", plan.off_pools, (plan.cap if sh else W * plan.cap) * 8),
                                ("table", plan.off_table, plan.table_n * 12),
                                ("misc", plan.off_misc, 8 * W + plan.ctl_bytes),
                            ]
                            if sh:
                                regions.append(("hist", plan.off_hist, 1024 * 4))
                            assert plan.ctl_bytes >= 32
                            spans = sorted((off, off + size, name) for name, off, size in regions)
                            for off, end, name in spans:
                                assert off % 16 == 0 or name == "misc" and off % 8 == 0, (name, off)
                                assert end <= plan.total_bytes, (name, end, plan.total_bytes, M, k, nprobe, W, sh)
                            for (a0, a1, an), (b0, b1, bn) in zip(spans, spans[1:]):
                                assert a1 <= b0, (an, bn, M, k, nprobe, W, sh)
                            checked += 1
    assert checked > 5000


def _faiss_file(tmp_path, name, d=4, nlist=1, ntotal=0, M=2, code_size=None, nbits=8, map_n=0, cent_floats=None,
                metric=1):
    """The leading part of a faiss IndexIVFPQ file (fourcc IwPQ, IndexFlat quantizer, product quantizer), as
    faiss 1.10's write_index lays it out, with the given -- possibly absurd -- sizes."""
    import struct
    hdr = lambda dd, nt: struct.pack("<iqqqBi", dd, nt, 1 << 20, 1 << 20, 1, metric)
    n_cent = nlist * d if cent_floats is None else cent_floats
    out = b"IwPQ" + hdr(d, ntotal) + struct.pack("<QQ", nlist, 1)
    out += (b"IxF2" if metric == 1 else b"IxFI") + hdr(d, nlist) + struct.pack("<Q", nlist * d)
    out += b"\0" * (4 * min(n_cent, 1 << 16))
    out += struct.pack("<BQ", 0, map_n) + struct.pack("<B", 0)
    out += struct.pack("<QQQQ", M if code_size is None else code_size, d, M, nbits)
    out += struct.pack("<Q", 256 * d) + b"\0" * (4 * 256 * min(d, 64))
    p = tmp_path / name
    p.write_bytes(out)
    return str(p).encode()


@pytest.mark.parametrize("kw,needle", [
    (dict(d=100000), "outside what an index holds"),
    (dict(d=0), "outside what an index holds"),
    (dict(nlist=1 << 21), "outside what an index holds"),
    (dict(nlist=0), "outside what an index holds"),
    (dict(ntotal=-5), "outside what an index holds"),
    (dict(d=4096, nlist=1 << 20), "shorter than its coarse quantizer"),
    (dict(M=1 << 32, code_size=1 << 32), "product quantizer"),          # d % (int)M would divide by zero
    (dict(M=3), "product quantizer"),                                    # 3 does not divide 4
    (dict(M=2, code_size=3), "product quantizer"),
    (dict(M=256, d=256, code_size=256), "product quantizer"),            # more sub-quantizers than the index takes
    (dict(nbits=4), "product quantizer"),
    (dict(map_n=1 << 61), "truncated"),
])
def test_reader_of_faiss_files_rejects_absurd_headers_before_using_them(capi, tmp_path, kw, needle):
    """Sizes a file states are checked against the index's limits and the file's own length before they are
    allocated, cast or divided by: every one of these comes back as an error message (no crash, no GPU needed,
    no huge allocation)."""
    lib = capi.load()
    path = _faiss_file(tmp_path, "bad.index", **kw)
    h = ctypes.c_void_p()
    rc = lib.ivfpq_read_faiss(path, None, ctypes.byref(h))
    msg = lib.ixa_last_error().decode()
    assert rc == 2001 and needle in msg and not h.value, (rc, msg)
