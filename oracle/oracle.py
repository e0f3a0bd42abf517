"""ctypes loader for the CPU parity oracle (``oracle/ivfpq_oracle.c``).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py``.  The product package never imports this module.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libivfpq_oracle.so")

METRIC_INNER_PRODUCT = 0
METRIC_L2 = 1

_c_f32p = ctypes.POINTER(ctypes.c_float)
_c_i64p = ctypes.POINTER(ctypes.c_int64)
_c_u8p = ctypes.POINTER(ctypes.c_uint8)
_c_i8p = ctypes.POINTER(ctypes.c_int8)
_c_i32p = ctypes.POINTER(ctypes.c_int32)


def build(force=False):
    """Compile the oracle shared object with gcc (no GPU involved)."""
    if force or not os.path.exists(_LIB_PATH) or (
        os.path.getmtime(_LIB_PATH) < os.path.getmtime(os.path.join(_HERE, "ivfpq_oracle.c"))
    ):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libivfpq_oracle.so"], stdout=subprocess.DEVNULL)
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.orc_f32_to_f16.restype = ctypes.c_uint16
        _lib.orc_f32_to_f16.argtypes = [ctypes.c_float]
        _lib.orc_f16_to_f32.restype = ctypes.c_float
        _lib.orc_f16_to_f32.argtypes = [ctypes.c_uint16]
        _lib.orc_kmeans.restype = ctypes.c_double
        _lib.orc_num_threads.restype = ctypes.c_int
    return _lib


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _p(a, t):
    return a.ctypes.data_as(t)


def num_threads():
    return int(lib().orc_num_threads())


def f32_to_f16(x):
    return int(lib().orc_f32_to_f16(ctypes.c_float(float(x))))


def f16_to_f32(h):
    return float(lib().orc_f16_to_f32(ctypes.c_uint16(int(h))))


def sqnorms(x):
    x = _f32(x)
    out = np.empty(x.shape[0], dtype=np.float32)
    lib().orc_sqnorms(_p(x, _c_f32p), ctypes.c_int64(x.shape[0]), ctypes.c_int(x.shape[1]), _p(out, _c_f32p))
    return out


def coarse_dist(q, cent, metric=METRIC_L2):
    q, cent = _f32(q), _f32(cent)
    out = np.empty((q.shape[0], cent.shape[0]), dtype=np.float32)
    lib().orc_coarse_dist(_p(q, _c_f32p), ctypes.c_int64(q.shape[0]), _p(cent, _c_f32p),
                          ctypes.c_int64(cent.shape[0]), ctypes.c_int(q.shape[1]), ctypes.c_int(metric),
                          _p(out, _c_f32p))
    return out


def coarse_probe(q, cent, nprobe, metric=METRIC_L2):
    q, cent = _f32(q), _f32(cent)
    nprobe = min(int(nprobe), cent.shape[0])
    ids = np.empty((q.shape[0], nprobe), dtype=np.int64)
    dist = np.empty((q.shape[0], nprobe), dtype=np.float32)
    lib().orc_coarse_probe(_p(q, _c_f32p), ctypes.c_int64(q.shape[0]), _p(cent, _c_f32p),
                           ctypes.c_int64(cent.shape[0]), ctypes.c_int(q.shape[1]), ctypes.c_int(metric),
                           ctypes.c_int64(nprobe), _p(ids, _c_i64p), _p(dist, _c_f32p))
    return ids, dist


def assign(x, cent):
    x, cent = _f32(x), _f32(cent)
    out = np.empty(x.shape[0], dtype=np.int64)
    lib().orc_assign(_p(x, _c_f32p), ctypes.c_int64(x.shape[0]), _p(cent, _c_f32p), ctypes.c_int64(cent.shape[0]),
                     ctypes.c_int(x.shape[1]), _p(out, _c_i64p))
    return out


def pq_encode(x, codebook):
    """codebook: [M, 256, dsub] float32 -> codes [n, M] uint8."""
    x, codebook = _f32(x), _f32(codebook)
    M = codebook.shape[0]
    assert codebook.shape[1] == 256 and codebook.shape[2] * M == x.shape[1]
    codes = np.empty((x.shape[0], M), dtype=np.uint8)
    lib().orc_pq_encode(_p(x, _c_f32p), ctypes.c_int64(x.shape[0]), ctypes.c_int(x.shape[1]), ctypes.c_int(M),
                        _p(codebook, _c_f32p), _p(codes, _c_u8p))
    return codes


def lut(q, codebook, metric=METRIC_L2, lut_fp16=False):
    q, codebook = _f32(q), _f32(codebook)
    M = codebook.shape[0]
    out = np.empty((q.shape[0], M, 256), dtype=np.float32)
    lib().orc_lut(_p(q, _c_f32p), ctypes.c_int64(q.shape[0]), ctypes.c_int(q.shape[1]), ctypes.c_int(M),
                  _p(codebook, _c_f32p), ctypes.c_int(metric), ctypes.c_int(int(lut_fp16)), _p(out, _c_f32p))
    return out


def adc_list(lut_q, codes):
    lut_q = _f32(lut_q)
    codes = np.ascontiguousarray(codes, dtype=np.uint8)
    out = np.empty(codes.shape[0], dtype=np.float32)
    lib().orc_adc_list(_p(lut_q, _c_f32p), _p(codes, _c_u8p), ctypes.c_int64(codes.shape[0]),
                       ctypes.c_int(codes.shape[1]), _p(out, _c_f32p))
    return out


class CsrIndex:
    """Host-side IVFPQ index in CSR form: what the oracle searches."""

    def __init__(self, d, M, metric, cent, codebook, list_off, codes, ids):
        self.d, self.M, self.metric = int(d), int(M), int(metric)
        self.cent = _f32(cent)
        self.codebook = _f32(codebook)
        self.nlist = self.cent.shape[0]
        self.list_off = np.ascontiguousarray(list_off, dtype=np.int64)
        self.codes = np.ascontiguousarray(codes, dtype=np.uint8).reshape(-1, self.M)
        self.ids = np.ascontiguousarray(ids, dtype=np.int64)

    @classmethod
    def from_assignment(cls, d, M, metric, cent, codebook, list_no, codes, ids):
        """Bucket rows by list keeping insertion order inside each list (reference add order,
        FR/ascend/impl/AscendIndexIVFPQImpl.cpp:715-753)."""
        list_no = np.asarray(list_no, dtype=np.int64)
        nlist = np.asarray(cent).shape[0]
        order = np.argsort(list_no, kind="stable")
        counts = np.bincount(list_no, minlength=nlist)
        off = np.zeros(nlist + 1, dtype=np.int64)
        np.cumsum(counts, out=off[1:])
        return cls(d, M, metric, cent, codebook, off, np.asarray(codes)[order], np.asarray(ids)[order])

    @classmethod
    def build(cls, d, M, metric, cent, codebook, x, ids=None):
        x = _f32(x)
        if ids is None:
            ids = np.arange(x.shape[0], dtype=np.int64)
        return cls.from_assignment(d, M, metric, cent, codebook, assign(x, cent), pq_encode(x, codebook), ids)

    def search(self, q, k, nprobe, lut_fp16=False):
        q = _f32(q)
        nq = q.shape[0]
        dist = np.empty((nq, k), dtype=np.float32)
        labels = np.empty((nq, k), dtype=np.int64)
        scanned = ctypes.c_int64(0)
        lib().orc_search(ctypes.c_int(self.d), ctypes.c_int(self.M), ctypes.c_int64(self.nlist),
                         ctypes.c_int(self.metric), _p(self.cent, _c_f32p), _p(self.codebook, _c_f32p),
                         _p(self.list_off, _c_i64p), _p(self.codes, _c_u8p), _p(self.ids, _c_i64p),
                         _p(q, _c_f32p), ctypes.c_int64(nq), ctypes.c_int64(nprobe), ctypes.c_int64(k),
                         ctypes.c_int(int(lut_fp16)), _p(dist, _c_f32p), _p(labels, _c_i64p),
                         ctypes.byref(scanned))
        self.last_scanned = int(scanned.value)
        return dist, labels


def flat_f32(base, q, k, metric=METRIC_L2, ids=None):
    base, q = _f32(base), _f32(q)
    dist = np.empty((q.shape[0], k), dtype=np.float32)
    labels = np.empty((q.shape[0], k), dtype=np.int64)
    idp = _p(np.ascontiguousarray(ids, dtype=np.int64), _c_i64p) if ids is not None else None
    lib().orc_flat_f32(_p(base, _c_f32p), ctypes.c_int64(base.shape[0]), ctypes.c_int(base.shape[1]),
                       ctypes.c_int(metric), idp, _p(q, _c_f32p), ctypes.c_int64(q.shape[0]), ctypes.c_int64(k),
                       _p(dist, _c_f32p), _p(labels, _c_i64p))
    return dist, labels


def flat_i8(base, q, k, ids=None):
    base = np.ascontiguousarray(base, dtype=np.int8)
    q = np.ascontiguousarray(q, dtype=np.int8)
    dist = np.empty((q.shape[0], k), dtype=np.int32)
    labels = np.empty((q.shape[0], k), dtype=np.int64)
    idp = _p(np.ascontiguousarray(ids, dtype=np.int64), _c_i64p) if ids is not None else None
    lib().orc_flat_i8(_p(base, _c_i8p), ctypes.c_int64(base.shape[0]), ctypes.c_int(base.shape[1]), idp,
                      _p(q, _c_i8p), ctypes.c_int64(q.shape[0]), ctypes.c_int64(k), _p(dist, _c_i32p),
                      _p(labels, _c_i64p))
    return dist, labels


def flat_remove_order(ntotal, positions):
    """Storage order of a Flat index after the reference removes the vectors at ``positions``: original
    positions of the survivors, in their new order.  The reference's loop as it stands
    (Index::removeIdsBatch, FR/ascenddaemon/impl/Index.cpp:86-113; the host id map is edited the same way,
    AscendIndexImpl::removeIdx, FR/ascend/impl/AscendIndexImpl.cpp:253-270): positions outside the index and
    repeats are dropped, the rest are visited from the highest to the lowest, each is overwritten with the
    vector that is last at that moment, and the index shrinks by one."""
    order = list(range(int(ntotal)))
    for pos in sorted({int(p) for p in positions if 0 <= int(p) < ntotal}, reverse=True):
        order[pos] = order[-1]
        order.pop()
    return np.asarray(order, dtype=np.int64)


def merge_results(dist, labels, metric=METRIC_L2):
    """dist/labels: [ndev][n][k] per-device result lists -> merged ([n][k], [n][k])."""
    dist = _f32(dist)
    labels = np.ascontiguousarray(labels, dtype=np.int64)
    ndev, n, k = dist.shape
    out_d = np.empty((n, k), dtype=np.float32)
    out_l = np.empty((n, k), dtype=np.int64)
    lib().orc_merge_results(ctypes.c_int(ndev), _p(dist, _c_f32p), _p(labels, _c_i64p), ctypes.c_int64(n),
                            ctypes.c_int64(k), ctypes.c_int(metric), _p(out_d, _c_f32p), _p(out_l, _c_i64p))
    return out_d, out_l


def kmeans(x, k, niter=25, spherical=False, seed=1234):
    x = _f32(x)
    cent = np.empty((k, x.shape[1]), dtype=np.float32)
    obj = lib().orc_kmeans(_p(x, _c_f32p), ctypes.c_int64(x.shape[0]), ctypes.c_int(x.shape[1]), ctypes.c_int64(k),
                           ctypes.c_int(niter), ctypes.c_int(int(spherical)), ctypes.c_uint64(seed),
                           _p(cent, _c_f32p))
    return cent, float(obj)


def train_pq(x, M, niter=25, spherical=False, seed=1234):
    """Per-sub-space k-means with 256 codewords -> codebook [M, 256, dsub]."""
    x = _f32(x)
    d = x.shape[1]
    dsub = d // M
    cb = np.empty((M, 256, dsub), dtype=np.float32)
    for m in range(M):
        cb[m], _ = kmeans(x[:, m * dsub:(m + 1) * dsub], 256, niter, spherical, seed + 17 * m)
    return cb
