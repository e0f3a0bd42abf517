"""ctypes binding of ``libindexsdk_amd.so`` (the C ABI declared in ``include/indexsdk_amd.h``).

The library is built in-tree by ``indexsdk_amd/csrc/build.sh``; importing this module never
compiles anything and never falls back to a CPU implementation: if the shared object is missing,
``load()`` raises.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libindexsdk_amd.so")

c_f32p = ctypes.POINTER(ctypes.c_float)
c_i64p = ctypes.POINTER(ctypes.c_int64)
c_i32p = ctypes.POINTER(ctypes.c_int32)
c_u8p = ctypes.POINTER(ctypes.c_uint8)
c_i8p = ctypes.POINTER(ctypes.c_int8)


class IvfpqConfig(ctypes.Structure):
    _fields_ = [
        ("niter", ctypes.c_int32),
        ("pq_niter", ctypes.c_int32),
        ("spherical", ctypes.c_int32),
        ("train_samples_per_list", ctypes.c_int32),
        ("max_train_samples", ctypes.c_int64),
        ("lut_fp16", ctypes.c_int32),
        ("code_layout", ctypes.c_int32),
        ("scratch_bytes", ctypes.c_int64),
        ("seed", ctypes.c_uint64),
        ("strict_reference_params", ctypes.c_int32),
        ("coarse_fp32_only", ctypes.c_int32),
        ("scan_locality", ctypes.c_int32),
        ("coarse_sampled_bound", ctypes.c_int32),
        ("pq_spherical", ctypes.c_int32),
        ("coarse_exact_small", ctypes.c_int32),
        ("stage_timings", ctypes.c_int32),
        ("coarse_resident", ctypes.c_int32),
    ]


class IvfpqSearchStats(ctypes.Structure):
    _fields_ = [(n, ctypes.c_double) for n in
                ("scanned_codes", "ms_coarse", "ms_scan", "ms_total", "scan_launches", "nsplit", "scan_waves",
                 "shared_pool", "coarse_reruns", "ordered", "coarse_plan", "pages")]


class ScanLdsPlan(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int32) for n in
                ("waves", "shared_pool", "cap", "merge_n", "table_n", "off_query", "off_pools", "off_table", "off_hist",
                 "off_misc", "ctl_bytes", "total_bytes")]


class FlatSearchStats(ctypes.Structure):
    _fields_ = [(n, ctypes.c_double) for n in ("ms_score", "ms_select", "ms_total", "score_launches",
                                                     "exact_reruns")]


# every exported symbol of include/indexsdk_amd.h: name -> (restype, argtypes)
_H = ctypes.c_void_p
_SIGNATURES = {
    "ixa_last_error": (ctypes.c_char_p, []),
    "ivfpq_last_error": (ctypes.c_char_p, []),
    "ixa_copy_probe": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64]),
    "ixa_read_probe": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.POINTER(ctypes.c_double)]),
    "ixa_merge_search_results": (ctypes.c_int, [ctypes.c_int, ctypes.c_int64, ctypes.c_int64, ctypes.c_int,
                                                ctypes.POINTER(ctypes.c_void_p), ctypes.POINTER(ctypes.c_void_p),
                                                ctypes.c_void_p, ctypes.c_void_p]),
    "ixa_op_distance_flat_l2_mins_fp32": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p,
                                                         ctypes.c_int64, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p,
                                                         ctypes.c_void_p, ctypes.c_void_p]),
    "ixa_op_topk_flat_fp32": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_int64,
                                             ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p,
                                             ctypes.c_void_p]),
    "ixa_op_ivfpq_search_distance_topk": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_void_p,
                                                         ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int,
                                                         ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p,
                                                         ctypes.c_void_p, ctypes.c_void_p]),
    "ixa_op_topk_ivfpq_l3": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_int,
                                            ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]),
    "ixa_op_ivfpq_subspace_distance": (ctypes.c_int, [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_void_p,
                                                      ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]),
    "ivfpq_search_probes_device": (ctypes.c_int, [_H, ctypes.c_int64, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int,
                                                  ctypes.c_int64, ctypes.c_void_p, ctypes.c_void_p]),
    "ivfpq_search_probes_device_noalloc": (ctypes.c_int, [_H, ctypes.c_int64, ctypes.c_void_p, ctypes.c_void_p,
                                                          ctypes.c_int, ctypes.c_int64, ctypes.c_void_p,
                                                          ctypes.c_void_p]),
    "ivfpq_reserve_memory": (ctypes.c_int, [_H, ctypes.c_int64]),
    "ivfpq_reclaim_memory": (ctypes.c_int, [_H, c_i64p]),
    "ivfpq_arena_state": (ctypes.c_int, [_H, c_i64p, c_i64p, c_i64p]),
    "ivfpq_search_lanes": (ctypes.c_int, [_H, ctypes.POINTER(ctypes.c_int)]),
    "ivfpq_plan_scan_lds": (ctypes.c_int, [ctypes.c_int] * 9 + [ctypes.POINTER(ScanLdsPlan)]),
    "ivfpq_get_code_layout": (ctypes.c_int, [_H, ctypes.POINTER(ctypes.c_int)]),
    "ivfpq_config_default": (None, [ctypes.POINTER(IvfpqConfig)]),
    "ivfpq_create": (ctypes.c_int, [ctypes.c_int, ctypes.c_int, ctypes.c_int64, ctypes.c_int, ctypes.c_int,
                                    ctypes.POINTER(IvfpqConfig), ctypes.POINTER(_H)]),
    "ivfpq_destroy": (ctypes.c_int, [_H]),
    "ivfpq_train": (ctypes.c_int, [_H, ctypes.c_int64, ctypes.c_void_p]),
    "ivfpq_train_device": (ctypes.c_int, [_H, ctypes.c_int64, ctypes.c_void_p]),
    "ivfpq_set_trained": (ctypes.c_int, [_H, ctypes.c_void_p, ctypes.c_void_p]),
    "ivfpq_get_trained": (ctypes.c_int, [_H, ctypes.c_void_p, ctypes.c_void_p]),
    "ivfpq_is_trained": (ctypes.c_int, [_H, ctypes.POINTER(ctypes.c_int)]),
    "ivfpq_add_with_ids": (ctypes.c_int, [_H, ctypes.c_int64, ctypes.c_void_p, ctypes.c_void_p]),
    "ivfpq_add_with_ids_device": (ctypes.c_int, [_H, ctypes.c_int64, ctypes.c_void_p, ctypes.c_void_p]),
    "ivfpq_add_codes": (ctypes.c_int, [_H, ctypes.c_int64, ctypes.c_int64, ctypes.c_void_p, ctypes.c_void_p]),
    "ivfpq_set_nprobe": (ctypes.c_int, [_H, ctypes.c_int]),
    "ivfpq_set_stage_timings": (ctypes.c_int, [_H, ctypes.c_int]),
    "ivfpq_get_nprobe": (ctypes.c_int, [_H, ctypes.POINTER(ctypes.c_int)]),
    "ivfpq_search": (ctypes.c_int, [_H, ctypes.c_int64, ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p,
                                    ctypes.c_void_p]),
    "ivfpq_search_device": (ctypes.c_int, [_H, ctypes.c_int64, ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p,
                                           ctypes.c_void_p]),
    "ivfpq_assign": (ctypes.c_int, [_H, ctypes.c_int64, ctypes.c_void_p, ctypes.c_void_p]),
    "ivfpq_coarse_probe": (ctypes.c_int, [_H, ctypes.c_int64, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]),
    "ivfpq_write_faiss": (ctypes.c_int, [_H, ctypes.c_char_p]),
    "ivfpq_read_faiss": (ctypes.c_int, [ctypes.c_char_p, ctypes.c_void_p, ctypes.POINTER(ctypes.c_void_p)]),
    "ivfpq_get_shape": (ctypes.c_int, [_H, ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_int),
                                       ctypes.POINTER(ctypes.c_int64), ctypes.POINTER(ctypes.c_int)]),
    "ivfpq_encode": (ctypes.c_int, [_H, ctypes.c_int64, ctypes.c_void_p, ctypes.c_void_p]),
    "ivfpq_list_length": (ctypes.c_int, [_H, ctypes.c_int64, ctypes.POINTER(ctypes.c_int64)]),
    "ivfpq_get_list": (ctypes.c_int, [_H, ctypes.c_int64, ctypes.c_void_p, ctypes.c_void_p]),
    "ivfpq_remove_ids": (ctypes.c_int, [_H, ctypes.c_int64, ctypes.c_void_p, ctypes.POINTER(ctypes.c_int64)]),
    "ivfpq_remove_range": (ctypes.c_int, [_H, ctypes.c_int64, ctypes.c_int64, ctypes.POINTER(ctypes.c_int64)]),
    "ivfpq_update": (ctypes.c_int, [_H, ctypes.c_int64, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                    ctypes.POINTER(ctypes.c_int64)]),
    "ivfpq_reset": (ctypes.c_int, [_H]),
    "ivfpq_ntotal": (ctypes.c_int, [_H, ctypes.POINTER(ctypes.c_int64)]),
    "ivfpq_last_search_stats": (ctypes.c_int, [_H, ctypes.POINTER(IvfpqSearchStats)]),
    "ivfpq_last_search_timings": (ctypes.c_int, [_H, ctypes.POINTER(ctypes.c_double), ctypes.POINTER(ctypes.c_double)]),
}

for _pfx, _dist in (("flat", ctypes.c_void_p), ("flat_i8", ctypes.c_void_p)):
    _SIGNATURES.update({
        f"{_pfx}_create": (ctypes.c_int, [ctypes.c_int, ctypes.c_int, ctypes.c_int64, ctypes.POINTER(_H)]),
        f"{_pfx}_destroy": (ctypes.c_int, [_H]),
        f"{_pfx}_add_with_ids": (ctypes.c_int, [_H, ctypes.c_int64, ctypes.c_void_p, ctypes.c_void_p]),
        f"{_pfx}_add_with_ids_device": (ctypes.c_int, [_H, ctypes.c_int64, ctypes.c_void_p, ctypes.c_void_p]),
        f"{_pfx}_search": (ctypes.c_int, [_H, ctypes.c_int64, ctypes.c_void_p, ctypes.c_int64, _dist,
                                          ctypes.c_void_p]),
        f"{_pfx}_search_with_masks": (ctypes.c_int, [_H, ctypes.c_int64, ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p,
                                                     _dist, ctypes.c_void_p]),
        f"{_pfx}_search_device": (ctypes.c_int, [_H, ctypes.c_int64, ctypes.c_void_p, ctypes.c_int64, _dist,
                                                 ctypes.c_void_p]),
        f"{_pfx}_get_base": (ctypes.c_int, [_H, ctypes.c_int64, ctypes.c_int64, ctypes.c_void_p]),
        f"{_pfx}_get_ids": (ctypes.c_int, [_H, ctypes.c_int64, ctypes.c_int64, ctypes.c_void_p]),
        f"{_pfx}_remove_ids": (ctypes.c_int, [_H, ctypes.c_int64, ctypes.c_void_p, ctypes.POINTER(ctypes.c_int64)]),
        f"{_pfx}_remove_range": (ctypes.c_int, [_H, ctypes.c_int64, ctypes.c_int64, ctypes.POINTER(ctypes.c_int64)]),
        f"{_pfx}_ntotal": (ctypes.c_int, [_H, ctypes.POINTER(ctypes.c_int64)]),
        f"{_pfx}_reset": (ctypes.c_int, [_H]),
        f"{_pfx}_last_search_stats": (ctypes.c_int, [_H, ctypes.POINTER(FlatSearchStats)]),
    })

_lib = None


def load():
    """Load the shared library; raises OSError when it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise OSError(f"{LIB_PATH} is missing: build it with indexsdk_amd/csrc/build.sh "
                          "(there is no CPU fallback)")
        # PyTorch-ROCm brings its own copy of the HIP runtime: when it initialises after this library has
        # started the system's runtime, torch.cuda reports no GPU.  If the caller has imported torch
        # already, let it start first (it costs nothing when it has).
        import sys
        torch = sys.modules.get("torch")
        if torch is not None and hasattr(torch, "cuda") and torch.cuda.device_count() > 0:
            try:
                torch.cuda.init()
            except Exception:
                pass
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def exported_names():
    return list(_SIGNATURES)


class IndexSdkError(RuntimeError):
    """Raised for a non-zero status of the C ABI (the reference throws faiss::FaissException)."""

    def __init__(self, code, message):
        super().__init__(f"[{code}] {message}")
        self.code = code
        self.message = message


def check(status):
    if status != 0:
        raise IndexSdkError(status, load().ixa_last_error().decode("utf-8", "replace"))
