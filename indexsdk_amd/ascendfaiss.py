"""Python face of the MI355X IVFPQ / Flat search path with the array contracts of the reference's
SWIG module ``ascendfaiss`` (examples/faiss-python/ascendfaiss.py:63-104): ``index.train(xb)``,
``index.add(xb)``, ``D, I = index.search(xq, k)`` on C-contiguous float32 ``[n, d]`` arrays,
returning ``D`` float32 ``[n, k]`` and ``I`` int64 ``[n, k]``.  Everything runs through the C ABI.
"""
import ctypes

import numpy as np

from . import _capi
from ._capi import IndexSdkError  # noqa: F401  (re-export)

METRIC_INNER_PRODUCT = 0
METRIC_L2 = 1


def _as(a, dtype, ndim, name):
    a = np.ascontiguousarray(a, dtype=dtype)
    if a.ndim != ndim:
        raise ValueError(f"{name} must have {ndim} dimensions, got shape {a.shape}")
    return a


def _ptr(a):
    return ctypes.c_void_p(a.ctypes.data)


class AscendIndexIVFPQConfig:
    """AscendIndexIVFPQConfig (FR/ascend/AscendIndexIVFPQ.h:32-68) plus the knobs of this build."""

    def __init__(self, **kw):
        self._c = _capi.IvfpqConfig()
        _capi.load().ivfpq_config_default(ctypes.byref(self._c))
        aliases = {"trainSamplesPerList": "train_samples_per_list", "maxTrainSamples": "max_train_samples",
                   "pqNiter": "pq_niter", "resourceSize": "scratch_bytes"}
        for key, val in kw.items():
            key = aliases.get(key, key)
            if key not in dict(self._c._fields_):
                raise TypeError(f"unknown config field {key}")
            setattr(self._c, key, val)

    def __getattr__(self, name):
        return getattr(self.__dict__["_c"], name)


class AscendIndexIVFPQ:
    """AscendIndexIVFPQ(dims, metric, nlist, msubs, nbits, config) -- FR/ascend/AscendIndexIVFPQ.h:71-96."""

    def __init__(self, dims, metric, nlist, msubs, nbits=8, config=None):
        self._lib = _capi.load()
        self._h = ctypes.c_void_p()
        self.d, self.metric_type, self.nlist, self.msubs, self.nbits = dims, metric, nlist, msubs, nbits
        cfg = ctypes.byref(config._c) if config is not None else None
        _capi.check(self._lib.ivfpq_create(dims, metric, nlist, msubs, nbits, cfg, ctypes.byref(self._h)))

    def __del__(self):
        h = getattr(self, "_h", None)
        if h:
            self._lib.ivfpq_destroy(h)
            self._h = None

    # ---- interchange with faiss (file form of copyTo / copyFrom, AscendIndexIVFPQImpl.cpp:392-508) --
    def write_faiss(self, path):
        """Writes the index in faiss.write_index's layout for an IndexIVFPQ (by_residual = False)."""
        _capi.check(self._lib.ivfpq_write_faiss(self._h, str(path).encode()))

    @classmethod
    def read_faiss(cls, path, config=None):
        """Loads a file written by write_faiss or by faiss.write_index(IndexIVFPQ with by_residual = False)."""
        self = cls.__new__(cls)
        self._lib = _capi.load()
        self._h = ctypes.c_void_p()
        cfg = ctypes.byref(config._c) if config is not None else None
        _capi.check(self._lib.ivfpq_read_faiss(str(path).encode(), cfg, ctypes.byref(self._h)))
        d, metric, nlist, m = ctypes.c_int(), ctypes.c_int(), ctypes.c_int64(), ctypes.c_int()
        _capi.check(self._lib.ivfpq_get_shape(self._h, ctypes.byref(d), ctypes.byref(metric), ctypes.byref(nlist),
                                              ctypes.byref(m)))
        self.d, self.metric_type, self.nlist, self.msubs, self.nbits = d.value, metric.value, nlist.value, m.value, 8
        return self

    # ---- training -----------------------------------------------------------------------------
    @property
    def is_trained(self):
        out = ctypes.c_int()
        _capi.check(self._lib.ivfpq_is_trained(self._h, ctypes.byref(out)))
        return bool(out.value)

    @property
    def ntotal(self):
        out = ctypes.c_int64()
        _capi.check(self._lib.ivfpq_ntotal(self._h, ctypes.byref(out)))
        return out.value

    def train(self, x):
        x = _as(x, np.float32, 2, "x")
        assert x.shape[1] == self.d
        _capi.check(self._lib.ivfpq_train(self._h, x.shape[0], _ptr(x)))

    def set_trained(self, centroids, codebook):
        """Injects quantizers (the role of copyFrom); codebook is [msubs, 256, dsub]."""
        c = _as(centroids, np.float32, 2, "centroids")
        cb = np.ascontiguousarray(codebook, dtype=np.float32)
        assert c.shape == (self.nlist, self.d) and cb.size == self.msubs * 256 * (self.d // self.msubs)
        _capi.check(self._lib.ivfpq_set_trained(self._h, _ptr(c), _ptr(cb)))

    def get_trained(self):
        c = np.empty((self.nlist, self.d), dtype=np.float32)
        cb = np.empty((self.msubs, 256, self.d // self.msubs), dtype=np.float32)
        _capi.check(self._lib.ivfpq_get_trained(self._h, _ptr(c), _ptr(cb)))
        return c, cb

    # ---- add ----------------------------------------------------------------------------------
    def add(self, x):
        self.add_with_ids(x, None)

    def add_with_ids(self, x, ids):
        x = _as(x, np.float32, 2, "x")
        assert x.shape[1] == self.d
        idp = None
        if ids is not None:
            ids = _as(ids, np.int64, 1, "ids")
            assert ids.shape[0] == x.shape[0]
            idp = _ptr(ids)
        _capi.check(self._lib.ivfpq_add_with_ids(self._h, x.shape[0], _ptr(x), idp))

    def add_codes(self, list_id, codes, ids):
        codes = _as(codes, np.uint8, 2, "codes")
        ids = _as(ids, np.int64, 1, "ids")
        assert codes.shape == (ids.shape[0], self.msubs)
        _capi.check(self._lib.ivfpq_add_codes(self._h, list_id, ids.shape[0], _ptr(codes), _ptr(ids)))

    # ---- search -------------------------------------------------------------------------------
    def setNumProbes(self, nprobe):
        _capi.check(self._lib.ivfpq_set_nprobe(self._h, nprobe))

    def getNumProbes(self):
        out = ctypes.c_int()
        _capi.check(self._lib.ivfpq_get_nprobe(self._h, ctypes.byref(out)))
        return out.value

    def search(self, x, k):
        x = _as(x, np.float32, 2, "x")
        assert x.shape[1] == self.d
        D = np.empty((x.shape[0], k), dtype=np.float32)
        I = np.empty((x.shape[0], k), dtype=np.int64)
        _capi.check(self._lib.ivfpq_search(self._h, x.shape[0], _ptr(x), k, _ptr(D), _ptr(I)))
        return D, I

    def assign(self, x):
        x = _as(x, np.float32, 2, "x")
        out = np.empty(x.shape[0], dtype=np.int64)
        _capi.check(self._lib.ivfpq_assign(self._h, x.shape[0], _ptr(x), _ptr(out)))
        return out

    def coarse_probe(self, x):
        x = _as(x, np.float32, 2, "x")
        nprobe = self.getNumProbes()
        ids = np.empty((x.shape[0], nprobe), dtype=np.int64)
        dist = np.empty((x.shape[0], nprobe), dtype=np.float32)
        _capi.check(self._lib.ivfpq_coarse_probe(self._h, x.shape[0], _ptr(x), _ptr(ids), _ptr(dist)))
        return ids, dist

    def encode(self, x):
        x = _as(x, np.float32, 2, "x")
        codes = np.empty((x.shape[0], self.msubs), dtype=np.uint8)
        _capi.check(self._lib.ivfpq_encode(self._h, x.shape[0], _ptr(x), _ptr(codes)))
        return codes

    # ---- lists --------------------------------------------------------------------------------
    def getListLength(self, list_id):
        out = ctypes.c_int64()
        _capi.check(self._lib.ivfpq_list_length(self._h, list_id, ctypes.byref(out)))
        return out.value

    def getListCodesAndIds(self, list_id):
        n = self.getListLength(list_id)
        codes = np.empty((n, self.msubs), dtype=np.uint8)
        ids = np.empty(n, dtype=np.int64)
        _capi.check(self._lib.ivfpq_get_list(self._h, list_id, _ptr(codes), _ptr(ids)))
        return codes, ids

    def remove_ids(self, ids):
        ids = _as(ids, np.int64, 1, "ids")
        out = ctypes.c_int64()
        _capi.check(self._lib.ivfpq_remove_ids(self._h, ids.shape[0], _ptr(ids), ctypes.byref(out)))
        return out.value

    def remove_range(self, imin, imax):
        """remove_ids(IDSelectorRange(imin, imax)): the vectors whose id lies in [imin, imax); returns how many."""
        removed = ctypes.c_int64()
        _capi.check(self._lib.ivfpq_remove_range(self._h, imin, imax, ctypes.byref(removed)))
        return removed.value

    def update(self, x, ids):
        """Replaces the vectors of existing ids; returns the ids that were not found."""
        x = _as(x, np.float32, 2, "x")
        ids = _as(ids, np.int64, 1, "ids")
        assert x.shape == (ids.shape[0], self.d)
        missing = np.empty(ids.shape[0], dtype=np.int64)
        nm = ctypes.c_int64()
        _capi.check(self._lib.ivfpq_update(self._h, ids.shape[0], _ptr(x), _ptr(ids), _ptr(missing), ctypes.byref(nm)))
        return missing[: nm.value].copy()

    def reset(self):
        _capi.check(self._lib.ivfpq_reset(self._h))

    def code_layout(self):
        """0 = row-major codes, 1 = bank-rotated, 2 = xor-rotated (what the index chose, or was told)."""
        out = ctypes.c_int()
        _capi.check(self._lib.ivfpq_get_code_layout(self._h, ctypes.byref(out)))
        return out.value

    def reserveMemory(self, num_vecs):
        """AscendIndexIVF::reserveMemory: room for num_vecs more vectors without replacing the code arena."""
        _capi.check(self._lib.ivfpq_reserve_memory(self._h, int(num_vecs)))

    def reclaimMemory(self):
        """AscendIndexIVF::reclaimMemory: shrinks the code arena to what the lists hold; returns the bytes released."""
        out = ctypes.c_int64()
        _capi.check(self._lib.ivfpq_reclaim_memory(self._h, ctypes.byref(out)))
        return out.value

    def arena_state(self):
        """(slots allocated, slots handed out, slots abandoned by lists that moved) of the code arena."""
        a, u, h = ctypes.c_int64(), ctypes.c_int64(), ctypes.c_int64()
        _capi.check(self._lib.ivfpq_arena_state(self._h, ctypes.byref(a), ctypes.byref(u), ctypes.byref(h)))
        return a.value, u.value, h.value

    def search_lanes(self):
        """Streams with workspaces of their own that searches of this index have needed so far (1 to 4)."""
        out = ctypes.c_int()
        _capi.check(self._lib.ivfpq_search_lanes(self._h, ctypes.byref(out)))
        return out.value

    def set_stage_timings(self, mode):
        """Stage events of a search (ms_coarse / ms_scan): 1 always, 0 never, -1 for pages of >= 256 queries."""
        _capi.check(self._lib.ivfpq_set_stage_timings(self._h, mode))

    def last_search_timings(self):
        """(ms_coarse, ms_scan) of the last search (0, 0 when it recorded no stage events); no device work, usable
        inside a timed loop."""
        a, b = ctypes.c_double(), ctypes.c_double()
        _capi.check(self._lib.ivfpq_last_search_timings(self._h, ctypes.byref(a), ctypes.byref(b)))
        return a.value, b.value

    def last_search_stats(self):
        s = _capi.IvfpqSearchStats()
        _capi.check(self._lib.ivfpq_last_search_stats(self._h, ctypes.byref(s)))
        return {n: getattr(s, n) for n, _ in s._fields_}


def merge_search_results(distances, labels, metric=METRIC_L2):
    """AscendIndexImpl::mergeSearchResult (FR/ascend/impl/AscendIndexImpl.cpp:587-640): merges the
    [n, k] result lists of several devices or shards (sequences of arrays, best first) into one."""
    dist = [_as(a, np.float32, 2, "distances") for a in distances]
    lab = [_as(a, np.int64, 2, "labels") for a in labels]
    assert len(dist) == len(lab) >= 1 and all(a.shape == dist[0].shape for a in dist + lab)
    n, k = dist[0].shape
    out_d = np.empty((n, k), dtype=np.float32)
    out_l = np.empty((n, k), dtype=np.int64)
    dp = (ctypes.c_void_p * len(dist))(*[a.ctypes.data for a in dist])
    lp = (ctypes.c_void_p * len(lab))(*[a.ctypes.data for a in lab])
    _capi.check(_capi.load().ixa_merge_search_results(len(dist), n, k, metric, dp, lp, _ptr(out_d), _ptr(out_l)))
    return out_d, out_l


class _FlatCommon:
    _pfx = None
    _dtype = None

    def __init__(self, dims, metric=METRIC_L2, scratch_bytes=0):
        self._lib = _capi.load()
        self._h = ctypes.c_void_p()
        self.d, self.metric_type = dims, metric
        _capi.check(self._fn("create")(dims, metric, scratch_bytes, ctypes.byref(self._h)))

    def _fn(self, name):
        return getattr(self._lib, f"{self._pfx}_{name}")

    def __del__(self):
        h = getattr(self, "_h", None)
        if h:
            self._fn("destroy")(h)
            self._h = None

    @property
    def ntotal(self):
        out = ctypes.c_int64()
        _capi.check(self._fn("ntotal")(self._h, ctypes.byref(out)))
        return out.value

    is_trained = True

    def add(self, x):
        self.add_with_ids(x, None)

    def add_with_ids(self, x, ids):
        x = _as(x, self._dtype, 2, "x")
        assert x.shape[1] == self.d
        idp = None
        if ids is not None:
            ids = _as(ids, np.int64, 1, "ids")
            assert ids.shape[0] == x.shape[0]
            idp = _ptr(ids)
        _capi.check(self._fn("add_with_ids")(self._h, x.shape[0], _ptr(x), idp))

    def getBase(self, offset=0, n=None):
        n = self.ntotal - offset if n is None else n
        out = np.empty((n, self.d), dtype=self._dtype)
        _capi.check(self._fn("get_base")(self._h, offset, n, _ptr(out)))
        return out

    def getIdxMap(self, offset=0, n=None):
        """The id of every stored vector, in storage order (getIdxMap, FR/ascend/AscendIndexFlat.h:76)."""
        n = self.ntotal - offset if n is None else n
        out = np.empty(n, dtype=np.int64)
        _capi.check(self._fn("get_ids")(self._h, offset, n, _ptr(out)))
        return out

    def remove_ids(self, ids):
        """remove_ids(IDSelectorBatch(ids)) -- FR/ascend/AscendIndex.h:78; returns the number of vectors removed."""
        ids = _as(ids, np.int64, 1, "ids")
        removed = ctypes.c_int64()
        _capi.check(self._fn("remove_ids")(self._h, ids.shape[0], _ptr(ids), ctypes.byref(removed)))
        return removed.value

    def remove_range(self, imin, imax):
        """remove_ids(IDSelectorRange(imin, imax)): the vectors whose id lies in [imin, imax)."""
        removed = ctypes.c_int64()
        _capi.check(self._fn("remove_range")(self._h, imin, imax, ctypes.byref(removed)))
        return removed.value

    def reset(self):
        _capi.check(self._fn("reset")(self._h))

    def last_search_stats(self):
        s = _capi.FlatSearchStats()
        _capi.check(self._fn("last_search_stats")(self._h, ctypes.byref(s)))
        return {n: getattr(s, n) for n, _ in s._fields_}


class AscendIndexFlat(_FlatCommon):
    """AscendIndexFlat(dims, metric, config) -- FR/ascend/AscendIndexFlat.h:48-90; fp32 distances."""
    _pfx = "flat"
    _dtype = np.float32

    def search(self, x, k):
        x = _as(x, np.float32, 2, "x")
        assert x.shape[1] == self.d
        D = np.empty((x.shape[0], k), dtype=np.float32)
        I = np.empty((x.shape[0], k), dtype=np.int64)
        _capi.check(self._lib.flat_search(self._h, x.shape[0], _ptr(x), k, _ptr(D), _ptr(I)))
        return D, I


    def search_with_masks(self, x, k, mask):
        """search_with_masks (FR/ascend/AscendIndexFlat.h:78-82): mask uint8 [n, ceil(ntotal / 8)], bit p % 8 of
        byte p / 8 of row i set = query i may return the vector at storage position p."""
        x = _as(x, np.float32, 2, "x")
        mask = _as(mask, np.uint8, 2, "mask")
        assert x.shape[1] == self.d and mask.shape == (x.shape[0], (self.ntotal + 7) // 8)
        D = np.empty((x.shape[0], k), dtype=np.float32)
        I = np.empty((x.shape[0], k), dtype=np.int64)
        _capi.check(self._lib.flat_search_with_masks(self._h, x.shape[0], _ptr(x), k, _ptr(mask), _ptr(D), _ptr(I)))
        return D, I


class AscendIndexFlatL2(AscendIndexFlat):
    def __init__(self, dims, scratch_bytes=0):
        super().__init__(dims, METRIC_L2, scratch_bytes)


class AscendIndexInt8Flat(_FlatCommon):
    """AscendIndexInt8Flat(dims, metric, config) -- FR/ascend/AscendIndexInt8.h:53-96; L2 only.
    ``search_int32`` returns the exact int32 distances; ``search`` returns them as float32 like the
    reference's signature (exact below 2**24, rounded to nearest above)."""
    _pfx = "flat_i8"
    _dtype = np.int8

    def search_int32(self, x, k):
        x = _as(x, np.int8, 2, "x")
        assert x.shape[1] == self.d
        D = np.empty((x.shape[0], k), dtype=np.int32)
        I = np.empty((x.shape[0], k), dtype=np.int64)
        _capi.check(self._lib.flat_i8_search(self._h, x.shape[0], _ptr(x), k, _ptr(D), _ptr(I)))
        return D, I

    def search_with_masks_int32(self, x, k, mask):
        """search_with_masks (FR/ascend/AscendIndexInt8Flat.h:98-99) with the exact int32 distances."""
        x = _as(x, np.int8, 2, "x")
        mask = _as(mask, np.uint8, 2, "mask")
        assert x.shape[1] == self.d and mask.shape == (x.shape[0], (self.ntotal + 7) // 8)
        D = np.empty((x.shape[0], k), dtype=np.int32)
        I = np.empty((x.shape[0], k), dtype=np.int64)
        _capi.check(self._lib.flat_i8_search_with_masks(self._h, x.shape[0], _ptr(x), k, _ptr(mask), _ptr(D), _ptr(I)))
        return D, I

    def search(self, x, k):
        D, I = self.search_int32(x, k)
        Df = D.astype(np.float32)
        Df[I == -1] = np.finfo(np.float32).max
        return Df, I
