"""ctypes binding of ``libkge_hip.so`` (C ABI declared in ``include/kge_hip.h``)."""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libkge_hip.so")

KGE_OK = 0
MODEL_IDS = {"DistMult": 0, "ComplEx": 1, "QMult": 2, "Keci": 3, "CKeci": 3, "OMult": 4, "DeCaL": 5}
DTYPE_F32, DTYPE_BF16, DTYPE_I8 = 0, 1, 2
NORM_NONE, NORM_LAYERNORM, NORM_BATCHNORM1D = 0, 1, 2

_c_i64 = ctypes.c_int64
_c_int = ctypes.c_int
_c_f = ctypes.c_float
_vp = ctypes.c_void_p
_sz = ctypes.c_size_t


class NormParams(ctypes.Structure):
    _fields_ = [("kind", ctypes.c_int32), ("eps", ctypes.c_float),
                ("h_a", _vp), ("h_b", _vp), ("r_a", _vp), ("r_b", _vp)]


class DropoutParams(ctypes.Structure):
    _fields_ = [("keep_h", _vp), ("keep_r", _vp), ("keep_q", _vp), ("scale_in", ctypes.c_float),
                ("scale_hidden", ctypes.c_float)]


class NormGrads(ctypes.Structure):
    _fields_ = [("h_a", _vp), ("h_b", _vp), ("r_a", _vp), ("r_b", _vp)]


SIGNATURES = {
    "kge_last_error": (ctypes.c_char_p, []),
    "kge_abi_version": (_c_int, []),
    "kge_build_query": (_c_int, [_c_int, _c_int, _c_int, _vp, _c_int, _vp, _vp, _c_int, _vp, _vp, _c_int,
                                 ctypes.POINTER(NormParams), _vp, _c_i64, _c_i64, _c_i64, _c_i64, _vp, _vp, _vp]),
    "kge_build_query_head": (_c_int, [_c_int, _c_int, _c_int, _vp, _c_int, _vp, _vp, _c_int, _vp, _vp, _c_int,
                                      ctypes.POINTER(NormParams), _vp, _c_i64, _c_i64, _c_i64, _c_i64, _vp, _vp, _vp]),
    "kge_build_query_decal": (_c_int, [_c_int, _c_int, _c_int, _c_int, _vp, _c_int, _vp, _vp, _c_int, _vp, _vp, _vp,
                                       ctypes.POINTER(NormParams), _vp, _c_i64, _c_i64, _c_i64, _c_i64, _vp, _vp, _vp]),
    "kge_build_query_backward": (_c_int, [_c_int, _c_int, _c_int, _c_int, _vp, _vp, _vp, _vp, _vp, _c_int, _vp, _c_i64,
                                          _c_i64, _c_i64, _c_i64, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "kge_build_query_dropout": (_c_int, [_c_int, _c_int, _c_int, _c_int, _vp, _c_int, _vp, _vp, _c_int, _vp, _vp, _vp,
                                         _c_int, ctypes.POINTER(NormParams), ctypes.POINTER(DropoutParams), _vp, _c_i64,
                                         _c_i64, _c_i64, _c_i64, _vp, _vp, _vp]),
    "kge_build_query_backward_norm": (_c_int, [_c_int, _c_int, _c_int, _c_int, _vp, _vp, _vp, _vp, _vp, _c_int,
                                               ctypes.POINTER(NormParams), ctypes.POINTER(NormGrads),
                                               ctypes.POINTER(DropoutParams), _vp, _c_i64, _c_i64, _c_i64, _c_i64, _vp,
                                               _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "kge_batchnorm_workspace_bytes": (_sz, [_c_i64, _c_i64]),
    "kge_batchnorm_stats": (_c_int, [_vp, _vp, _vp, _c_i64, _c_i64, _c_i64, _c_i64, ctypes.POINTER(DropoutParams), _c_f,
                                     _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _sz, _vp]),
    "kge_build_query_backward_batchnorm": (_c_int, [_c_int, _c_int, _c_int, _c_int, _vp, _vp, _vp, _vp, _vp, _c_int,
                                                    ctypes.POINTER(NormParams), ctypes.POINTER(DropoutParams), _vp,
                                                    _c_i64, _c_i64, _c_i64, _c_i64, _vp, _vp, _vp, _vp, _vp, _vp, _vp,
                                                    _vp, _sz, _vp]),
    "kge_scores": (_c_int, [_vp, _vp, _vp, _c_int, _vp, _c_i64, _c_i64, _c_i64, _vp, _c_i64, _vp]),
    "kge_triple_scores": (_c_int, [_vp, _vp, _vp, _c_int, _vp, _c_i64, _c_i64, _c_i64, _vp, _vp, _vp]),
    "kge_sample_scores": (_c_int, [_vp, _vp, _vp, _c_int, _vp, _c_i64, _c_i64, _c_i64, _vp, _c_i64, _vp, _vp]),
    "kge_csr_lookup": (_c_int, [_vp, _c_i64, _vp, _c_i64, _c_i64, _vp, _vp]),
    "kge_csr_build_workspace_bytes": (_sz, [_c_i64]),
    "kge_csr_build": (_c_int, [_vp, _c_i64, _c_int, _c_int, _c_int, _c_i64, _c_i64, _c_i64, _vp, _vp, _vp, _vp, _vp,
                               _sz, _vp]),
    "kge_rank_workspace_bytes": (_sz, [_c_i64]),
    "kge_rank_filtered": (_c_int, [_vp, _vp, _vp, _c_int, _vp, _c_i64, _c_i64, _c_i64, _vp, _vp, _vp, _vp, _c_i64,
                                   _vp, _vp, _vp, _vp, _vp, _sz, _vp]),
    "kge_rank_thresholds": (_c_int, [_vp, _vp, _vp, _c_int, _vp, _c_i64, _c_i64, _c_i64, _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "kge_rank_filtered_with_thresholds": (_c_int, [_vp, _vp, _c_int, _vp, _c_i64, _c_i64, _c_i64, _vp, _vp, _vp, _vp, _vp,
                                                   _c_i64, _c_int, _vp, _vp, _vp, _vp, _sz, _vp]),
    "kge_rank_static_init": (_c_int, []),
    "kge_rank_filtered_static": (_c_int, [_vp, _vp, _vp, _c_int, _vp, _c_i64, _c_i64, _c_i64, _vp, _vp, _vp, _vp, _c_i64,
                                          _vp, _vp, _vp, _vp, _vp]),
    "kge_topk_workspace_bytes": (_sz, [_c_i64, _c_i64, _c_i64]),
    "kge_topk": (_c_int, [_vp, _vp, _vp, _c_int, _vp, _c_i64, _c_i64, _c_i64, _c_i64, _vp, _vp, _c_int, _vp, _sz,
                          _vp]),
    "kge_topk_prepared_bytes": (_sz, [_c_int, _c_i64, _c_i64]),
    "kge_topk_prepare": (_c_int, [_vp, _c_int, _vp, _c_i64, _c_i64, _vp, _sz, _vp]),
    "kge_topk_prepared_workspace_bytes": (_sz, [_c_i64, _c_i64, _c_i64]),
    "kge_topk_prepared": (_c_int, [_vp, _vp, _vp, _c_int, _vp, _c_i64, _c_i64, _c_i64, _c_i64, _vp, _vp, _c_int, _vp,
                                   _sz, _vp, _sz, _vp]),
    "kge_profile_begin": (_c_int, []),
    "kge_profile_end": (_c_int, [ctypes.POINTER(ctypes.c_double), ctypes.POINTER(ctypes.c_int64)]),
    "kge_profile_kernel": (ctypes.c_char_p, []),
    "kge_probe_mfma": (_c_int, [_c_int, _c_int, ctypes.c_double, ctypes.POINTER(ctypes.c_double),
                                ctypes.POINTER(ctypes.c_double), _vp]),
    "kge_probe_walk": (_c_int, [_vp, _vp, _c_i64, _c_i64, ctypes.c_double, ctypes.POINTER(ctypes.c_double),
                                ctypes.POINTER(ctypes.c_double), _vp]),
    "kge_probe_i8_scan": (_c_int, [_vp, _vp, _c_i64, _c_i64, ctypes.c_double, ctypes.POINTER(ctypes.c_double),
                                   ctypes.POINTER(ctypes.c_double), _vp]),
    "kge_row_minmax": (_c_int, [_vp, _vp, _vp, _c_int, _vp, _c_i64, _c_i64, _c_i64, _vp, _vp, _vp]),
    "kge_bce_workspace_bytes": (_sz, []),
    "kge_bce_multihot": (_c_int, [_vp, _vp, _vp, _c_int, _vp, _c_i64, _c_i64, _c_i64, _vp, _vp, _vp, _c_i64, _c_f,
                                  _vp, _vp, _sz, _vp]),
    "kge_bce_backward_workspace_bytes": (_sz, [_c_i64, _c_i64, _c_i64]),
    "kge_bce_multihot_backward": (_c_int, [_vp, _vp, _vp, _c_int, _c_i64, _c_i64, _c_i64, _vp, _vp, _vp, _c_i64,
                                           ctypes.c_float, ctypes.c_float, _vp, _vp, _vp, _vp, _vp, _sz, _vp]),
}

_lib = None


class KgeError(RuntimeError):
    def __init__(self, code, text):
        super().__init__(f"libkge_hip error {code}: {text}")
        self.code = code


def load():
    """Load the HIP library; raises if it has not been built (there is no fallback path)."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `python -m dicee_amd.build` "
            "(hipcc --offload-arch=gfx950). There is no CPU fallback for the scoring path.")
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(rc):
    if rc != KGE_OK:
        raise KgeError(rc, load().kge_last_error().decode("utf-8", "replace"))
