"""ctypes binding of libhipress_amd.so (the C ABI declared in include/hipress_amd.h).

There is no CPU fallback: if the library is missing or a call fails, an
exception is raised.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# HIPRESS_AMD_LIB names another build of the same library (a variant made with
# `python -m hipress_amd.build --define ... --output ...` for an A/B measurement)
LIB_PATH = os.environ.get("HIPRESS_AMD_LIB") or os.path.join(_HERE, "libhipress_amd.so")

ONEBIT, TBQ, TERNGRAD, DGC, GRADDROP, ONEBIT_DEFERRED = range(6)
ALG_IDS = {"onebit": ONEBIT, "tbq": TBQ, "terngrad": TERNGRAD, "dgc": DGC, "graddrop": GRADDROP,
           "onebit_deferred": ONEBIT_DEFERRED}
MAX_PEERS = 16
HEADER_BYTES = 16

_i32, _i64, _f32, _f64, _vp = ctypes.c_int32, ctypes.c_int64, ctypes.c_float, ctypes.c_double, ctypes.c_void_p


class HipressError(RuntimeError):
    def __init__(self, code, where):
        self.code = code
        super().__init__(f"{where}: {strerror(code)} (code {code})")


class Tensor(ctypes.Structure):
    _fields_ = [
        ("grad", _vp), ("state0", _vp), ("state1", _vp), ("uniform", _vp),
        ("payload", _vp), ("out", _vp), ("n", _i64), ("payload_bytes", _i64),
    ]


class Params(ctypes.Structure):
    _fields_ = [("threshold", _f32), ("bucket", _i32), ("momentum_factor", _f32), ("reserved", _f32), ("ratio", _f64)]


class MergeChunk(ctypes.Structure):
    _fields_ = [
        ("payloads", _vp * MAX_PEERS), ("payload_bytes", _i64 * MAX_PEERS),
        ("aggregate", _vp), ("state", _vp), ("out_payload", _vp), ("out_payload_bytes", _i64), ("n", _i64),
        ("local", _vp),
    ]


# name -> (restype, argtypes); every symbol include/hipress_amd.h declares
SIGNATURES = {
    "hipress_version": (ctypes.c_int, []),
    "hipress_strerror": (ctypes.c_char_p, [ctypes.c_int]),
    "hipress_onebit_payload_bytes": (_i64, [_i64]),
    "hipress_tbq_payload_bytes": (_i64, [_i64]),
    "hipress_terngrad_payload_bytes": (_i64, [_i64, _i32]),
    "hipress_sparse_capacity": (_i64, [_i64, _f64]),
    "hipress_sparse_payload_bytes": (_i64, [_i64, _f64]),
    "hipress_onebit_workspace_bytes": (_i64, [_i64]),
    "hipress_sparse_workspace_bytes": (_i64, [_i64, _f64]),
    "hipress_sparse_merge_workspace_bytes": (_i64, [_i64, _i32, _f64, _i32]),
    "hipress_tbq_encode": (ctypes.c_int, [_vp, _vp, _i64, _vp, _i64, _f32, _vp]),
    "hipress_tbq_decode": (ctypes.c_int, [_vp, _i64, _vp, _i64, _vp]),
    "hipress_onebit_encode": (ctypes.c_int, [_vp, _vp, _i64, _vp, _i64, _vp, _i64, _vp]),
    "hipress_onebit_encode_static": (ctypes.c_int, [_vp, _vp, _i64, _vp, _i64, _vp]),
    "hipress_onebit_decode": (ctypes.c_int, [_vp, _i64, _vp, _i64, _vp]),
    "hipress_onebit_encode_deferred": (ctypes.c_int, [_vp, _vp, _vp, _i64, _vp, _i64, _vp, _i64, _vp]),
    "hipress_onebit_residual": (ctypes.c_int, [_vp, _vp, _i64, _vp, _vp]),
    "hipress_terngrad_encode": (ctypes.c_int, [_vp, _vp, _i64, _vp, _i64, _i32, _vp]),
    "hipress_terngrad_encode_seeded": (ctypes.c_int, [_vp, _i64, _vp, _i64, _i32, ctypes.c_uint64, _vp]),
    "hipress_uniform_fill": (ctypes.c_int, [_vp, _i64, ctypes.c_uint64, ctypes.c_uint32, _vp]),
    "hipress_terngrad_decode": (ctypes.c_int, [_vp, _i64, _vp, _i64, _vp]),
    "hipress_compll_payload_bytes": (_i64, [_i64, _i32]),
    "hipress_compll_workspace_bytes": (_i64, [_i64]),
    "hipress_compll_decoded_count": (_i64, [_i64, _i32]),
    "hipress_compll_encode": (ctypes.c_int, [_vp, _vp, _i64, _vp, _i64, _i32, _vp, _i64, _vp]),
    "hipress_compll_encode_seeded": (ctypes.c_int, [_vp, _i64, _vp, _i64, _i32, ctypes.c_uint64, _vp, _i64, _vp]),
    "hipress_compll_decode": (ctypes.c_int, [_vp, _i64, _vp, _i64, _vp]),
    "hipress_dgc_encode": (ctypes.c_int, [_vp, _vp, _vp, _i64, _vp, _i64, _f32, _f64, _vp, _i64, _vp]),
    "hipress_graddrop_encode": (ctypes.c_int, [_vp, _vp, _i64, _vp, _i64, _f64, _vp, _i64, _vp]),
    "hipress_sparse_decode": (ctypes.c_int, [_vp, _i64, _vp, _i64, _vp]),
    "hipress_tbq_decode_merge": (ctypes.c_int, [_vp, _vp, _i32, _vp, _i64, _vp, _vp, _i64, _f32, _vp]),
    "hipress_onebit_decode_merge": (ctypes.c_int, [_vp, _vp, _i32, _vp, _i64, _vp]),
    "hipress_terngrad_decode_merge": (ctypes.c_int, [_vp, _vp, _i32, _vp, _i64, _vp]),
    "hipress_sparse_decode_merge": (ctypes.c_int, [_vp, _vp, _i32, _vp, _i64, _vp, _vp, _i64, _f64, _vp, _i64, _vp]),
    "hipress_tbq_decode_merge_local": (ctypes.c_int, [_vp, _vp, _i32, _vp, _vp, _i64, _vp, _vp, _i64, _f32, _vp]),
    "hipress_onebit_decode_merge_local": (ctypes.c_int, [_vp, _vp, _i32, _vp, _vp, _i64, _vp]),
    "hipress_terngrad_decode_merge_local": (ctypes.c_int, [_vp, _vp, _i32, _vp, _vp, _i64, _vp]),
    "hipress_sparse_decode_merge_local": (ctypes.c_int, [_vp, _vp, _i32, _vp, _vp, _i64, _vp, _vp, _i64, _f64, _vp, _i64, _vp]),
    "hipress_batch_create": (ctypes.c_int, [ctypes.POINTER(_vp), _i32, ctypes.POINTER(Tensor), _i32, ctypes.POINTER(Params)]),
    "hipress_batch_encode": (ctypes.c_int, [_vp, _vp]),
    "hipress_batch_encode_seeded": (ctypes.c_int, [_vp, ctypes.c_uint64, _vp]),
    "hipress_batch_decode": (ctypes.c_int, [_vp, _vp]),
    "hipress_batch_encode_phase": (ctypes.c_int, [_vp, _i32, _vp]),
    "hipress_batch_destroy": (ctypes.c_int, [_vp]),
    "hipress_merge_batch_create": (ctypes.c_int, [ctypes.POINTER(_vp), _i32, ctypes.POINTER(MergeChunk), _i32, _i32, ctypes.POINTER(Params)]),
    "hipress_merge_batch_run": (ctypes.c_int, [_vp, _vp]),
    "hipress_merge_batch_run_phase": (ctypes.c_int, [_vp, _i32, _vp]),
    "hipress_merge_batch_destroy": (ctypes.c_int, [_vp]),
}

_lib = None


def lib():
    """The loaded library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `python -m hipress_amd.build` "
                "(hipcc, gfx950). hipress_amd has no CPU fallback."
            )
        L = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def strerror(code):
    return lib().hipress_strerror(code).decode()


def check(code, where):
    if code != 0:
        raise HipressError(code, where)


def size(value, where):
    """Size queries return a non-negative byte/element count or a negative error code."""
    if value < 0:
        raise HipressError(int(value), where)
    return int(value)
