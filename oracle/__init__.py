"""ctypes front end of the CPU oracle (``oracle/hipress_oracle.c``).

Test infrastructure only: imported by ``tests/``, by ``__graft_entry__.smoke``
and by the CPU-baseline leg of ``bench.py`` as the checker.  The shipped package
``hipress_amd`` never imports it.

Every wrapper takes and returns numpy arrays; state buffers (residual,
momentum, accumulator) are copied, updated and returned, so the caller's
arrays are never modified.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libhipress_oracle.so")
_SO_OMP = os.path.join(_HERE, "libhipress_oracle_omp.so")
HEADER_BYTES = 16


def build(force=False):
    """Compile the oracle with gcc (a second or so)."""
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(
        os.path.join(_HERE, "hipress_oracle.c")
    ):
        subprocess.check_call(["make", "-C", _HERE, "-B", "all"], stdout=subprocess.DEVNULL)
    return _SO


def omp_lib():
    """The all-cores (OpenMP) build of the same source, for the CPU-baseline timing only:
    same entry points, every loop with independent iterations shared between the cores."""
    global _omp
    if _omp is None:
        build()
        if not os.path.exists(_SO_OMP):
            subprocess.check_call(["make", "-C", _HERE, "libhipress_oracle_omp.so"], stdout=subprocess.DEVNULL)
        L = ctypes.CDLL(_SO_OMP)
        _bind(L)
        L.hpo_threads.restype = ctypes.c_int
        _omp = L
    return _omp


_omp = None
_lib = None

_i64 = ctypes.c_int64
_f32 = ctypes.c_float
_f64 = ctypes.c_double
_ptr = ctypes.c_void_p


_SIG = {
    "hpo_get_code": (ctypes.c_uint32, [_ptr, _i64, ctypes.c_int]),
    "hpo_put_code": (None, [_ptr, _i64, ctypes.c_int, ctypes.c_uint32]),
    "hpo_onebit_payload_bytes": (_i64, [_i64]),
    "hpo_tbq_payload_bytes": (_i64, [_i64]),
    "hpo_terngrad_scale_bytes": (_i64, [_i64, _i64]),
    "hpo_terngrad_payload_bytes": (_i64, [_i64, _i64]),
    "hpo_sparse_capacity": (_i64, [_i64, _f64]),
    "hpo_sparse_payload_bytes": (_i64, [_i64, _f64]),
    "hpo_tbq_encode": (None, [_ptr, _ptr, _i64, _ptr, _f32]),
    "hpo_tbq_decode": (None, [_ptr, _ptr, _i64]),
    "hpo_onebit_scale": (_f32, [_ptr, _ptr, _i64]),
    "hpo_onebit_encode_with_scale": (None, [_ptr, _ptr, _i64, _ptr, _f32]),
    "hpo_onebit_encode": (None, [_ptr, _ptr, _i64, _ptr]),
    "hpo_onebit_decode": (None, [_ptr, _ptr, _i64]),
    "hpo_terngrad_encode": (None, [_ptr, _ptr, _i64, _ptr, _i64]),
    "hpo_terngrad_decode": (None, [_ptr, _ptr, _i64]),
    "hpo_sparse_sample_stride": (_i64, [_i64]),
    "hpo_sparse_sample_count": (_i64, [_i64]),
    "hpo_sparse_sample_k": (_i64, [_i64, _f64]),
    "hpo_sparse_threshold": (_f32, [_ptr, _i64, _f64]),
    "hpo_dgc_encode": (None, [_ptr, _ptr, _ptr, _i64, _ptr, _f32, _f64]),
    "hpo_graddrop_encode": (None, [_ptr, _ptr, _i64, _ptr, _f64]),
    "hpo_sparse_decode": (None, [_ptr, _ptr, _i64]),
    "hpo_tbq_decode_merge": (None, [_ptr, ctypes.c_int, _ptr, _i64, _ptr, _ptr, _f32]),
    "hpo_onebit_decode_merge": (None, [_ptr, ctypes.c_int, _ptr, _i64]),
    "hpo_terngrad_decode_merge": (None, [_ptr, ctypes.c_int, _ptr, _i64]),
    "hpo_sparse_decode_merge": (None, [_ptr, ctypes.c_int, _ptr, _i64, _ptr, _ptr, _f64]),
    "hpo_tbq_decode_merge_local": (None, [_ptr, ctypes.c_int, _ptr, _ptr, _i64, _ptr, _ptr, _f32]),
    "hpo_onebit_decode_merge_local": (None, [_ptr, ctypes.c_int, _ptr, _ptr, _i64]),
    "hpo_terngrad_decode_merge_local": (None, [_ptr, ctypes.c_int, _ptr, _ptr, _i64]),
    "hpo_sparse_decode_merge_local": (None, [_ptr, ctypes.c_int, _ptr, _ptr, _i64, _ptr, _ptr, _f64]),
    "hpo_compll_decode": (_i64, [_ptr, _i64, _ptr, _i64]),
    "hpo_compll_payload_bytes": (_i64, [_i64, ctypes.c_int]),
    "hpo_compll_encode": (_i64, [_ptr, _ptr, _i64, _ptr, ctypes.c_int]),
    "hpo_lcg_uniform": (None, [ctypes.c_uint32, _f32, _f32, _ptr, _i64]),
    "hpo_uniform_tensor_key": (ctypes.c_uint32, [ctypes.c_uint64, ctypes.c_uint32]),
    "hpo_uniform_draws": (None, [ctypes.c_uint64, ctypes.c_uint32, _ptr, _i64]),
}


def _bind(L):
    for name, (res, args) in _SIG.items():
        fn = getattr(L, name)
        fn.restype = res
        fn.argtypes = args


def lib():
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_SO)
        _bind(L)
        _lib = L
    return _lib


def _f32c(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _payload(nbytes):
    return np.zeros(int(nbytes), dtype=np.uint8)


def _peer_array(payloads):
    keep = [np.ascontiguousarray(p, dtype=np.uint8) for p in payloads]
    arr = (ctypes.c_void_p * len(keep))(*[p.ctypes.data for p in keep])
    return keep, arr


# -- wire rule -------------------------------------------------------------
def get_code(words, i, b):
    words = np.ascontiguousarray(words, dtype=np.uint32)
    return int(lib().hpo_get_code(_p(words), i, b))


def put_code(words, i, b, code):
    assert words.dtype == np.uint32 and words.flags.c_contiguous
    lib().hpo_put_code(_p(words), i, b, code)


# -- sizes -------------------------------------------------------------------
def onebit_payload_bytes(n):
    return int(lib().hpo_onebit_payload_bytes(n))


def tbq_payload_bytes(n):
    return int(lib().hpo_tbq_payload_bytes(n))


def terngrad_scale_bytes(n, bucket):
    return int(lib().hpo_terngrad_scale_bytes(n, bucket))


def terngrad_payload_bytes(n, bucket):
    return int(lib().hpo_terngrad_payload_bytes(n, bucket))


def sparse_capacity(n, ratio):
    return int(lib().hpo_sparse_capacity(n, ratio))


def sparse_payload_bytes(n, ratio):
    return int(lib().hpo_sparse_payload_bytes(n, ratio))


def sparse_sample_stride(n):
    return int(lib().hpo_sparse_sample_stride(n))


def sparse_sample_k(n, ratio):
    return int(lib().hpo_sparse_sample_k(n, ratio))


# -- TBQ ---------------------------------------------------------------------
def tbq_encode(g, r, tau):
    """-> (payload uint8[], residual')"""
    g, r = _f32c(g), _f32c(r).copy()
    pay = _payload(tbq_payload_bytes(g.size))
    lib().hpo_tbq_encode(_p(g), _p(r), g.size, _p(pay), tau)
    return pay, r


def tbq_decode(payload, n):
    payload = np.ascontiguousarray(payload, dtype=np.uint8)
    out = np.empty(n, dtype=np.float32)
    lib().hpo_tbq_decode(_p(payload), _p(out), n)
    return out


# -- onebit ------------------------------------------------------------------
def onebit_scale(g, r):
    g, r = _f32c(g), _f32c(r)
    return np.float32(lib().hpo_onebit_scale(_p(g), _p(r), g.size))


def onebit_encode(g, r, scale=None):
    """-> (payload, residual'); with ``scale`` given, that scale is used verbatim."""
    g, r = _f32c(g), _f32c(r).copy()
    pay = _payload(onebit_payload_bytes(g.size))
    if scale is None:
        lib().hpo_onebit_encode(_p(g), _p(r), g.size, _p(pay))
    else:
        lib().hpo_onebit_encode_with_scale(_p(g), _p(r), g.size, _p(pay), float(scale))
    return pay, r


def onebit_decode(payload, n):
    payload = np.ascontiguousarray(payload, dtype=np.uint8)
    out = np.empty(n, dtype=np.float32)
    lib().hpo_onebit_decode(_p(payload), _p(out), n)
    return out


# -- TernGrad ------------------------------------------------------------------
def terngrad_encode(g, u, bucket=512):
    g, u = _f32c(g), _f32c(u)
    pay = _payload(terngrad_payload_bytes(g.size, bucket))
    lib().hpo_terngrad_encode(_p(g), _p(u), g.size, _p(pay), bucket)
    return pay


def terngrad_decode(payload, n):
    payload = np.ascontiguousarray(payload, dtype=np.uint8)
    out = np.empty(n, dtype=np.float32)
    lib().hpo_terngrad_decode(_p(payload), _p(out), n)
    return out


# -- DGC / GradDrop ------------------------------------------------------------
def sparse_threshold(a, ratio):
    a = _f32c(a)
    return np.float32(lib().hpo_sparse_threshold(_p(a), a.size, ratio))


def dgc_encode(g, mom, acc, m, ratio):
    """-> (payload, mom', acc')"""
    g, mom, acc = _f32c(g), _f32c(mom).copy(), _f32c(acc).copy()
    pay = _payload(sparse_payload_bytes(g.size, ratio))
    lib().hpo_dgc_encode(_p(g), _p(mom), _p(acc), g.size, _p(pay), m, ratio)
    return pay, mom, acc


def graddrop_encode(g, acc, ratio):
    """-> (payload, acc')"""
    g, acc = _f32c(g), _f32c(acc).copy()
    pay = _payload(sparse_payload_bytes(g.size, ratio))
    lib().hpo_graddrop_encode(_p(g), _p(acc), g.size, _p(pay), ratio)
    return pay, acc


def sparse_decode(payload, n):
    payload = np.ascontiguousarray(payload, dtype=np.uint8)
    out = np.empty(n, dtype=np.float32)
    lib().hpo_sparse_decode(_p(payload), _p(out), n)
    return out


def sparse_unpack(payload):
    """-> (nnz, n, capacity, thr, idx[nnz], val[nnz]) from a sparse payload."""
    payload = np.ascontiguousarray(payload, dtype=np.uint8)
    hdr = payload[:16].view(np.uint32)
    nnz, n, cap = int(hdr[0]), int(hdr[1]), int(hdr[2])
    thr = payload[12:16].view(np.float32)[0]
    idx = payload[16 : 16 + 4 * cap].view(np.int32)[: min(nnz, cap)].copy()
    val = payload[16 + 4 * cap : 16 + 8 * cap].view(np.float32)[: min(nnz, cap)].copy()
    return nnz, n, cap, thr, idx, val


# -- decode-and-merge ----------------------------------------------------------
def _local(local, n):
    """The aggregator's own uncompressed gradient the sum starts from, or None (zero)."""
    if local is None:
        return None, None
    local = _f32c(local)
    assert local.size == n
    return local, _p(local)


def tbq_decode_merge(payloads, n, r=None, tau=0.0, local=None):
    """-> aggregate, or (aggregate, out_payload, residual') when r is given."""
    keep, arr = _peer_array(payloads)
    agg = np.empty(n, dtype=np.float32)
    local, lp = _local(local, n)
    if r is None:
        lib().hpo_tbq_decode_merge_local(arr, len(keep), lp, _p(agg), n, None, None, tau)
        return agg
    r = _f32c(r).copy()
    out = _payload(tbq_payload_bytes(n))
    lib().hpo_tbq_decode_merge_local(arr, len(keep), lp, _p(agg), n, _p(r), _p(out), tau)
    return agg, out, r


def onebit_decode_merge(payloads, n, local=None):
    keep, arr = _peer_array(payloads)
    agg = np.empty(n, dtype=np.float32)
    local, lp = _local(local, n)
    lib().hpo_onebit_decode_merge_local(arr, len(keep), lp, _p(agg), n)
    return agg


def terngrad_decode_merge(payloads, n, local=None):
    keep, arr = _peer_array(payloads)
    agg = np.empty(n, dtype=np.float32)
    local, lp = _local(local, n)
    lib().hpo_terngrad_decode_merge_local(arr, len(keep), lp, _p(agg), n)
    return agg


def sparse_decode_merge(payloads, n, acc=None, ratio=0.0, local=None):
    """-> aggregate, or (aggregate, out_payload, acc') when acc is given."""
    keep, arr = _peer_array(payloads)
    agg = np.empty(n, dtype=np.float32)
    local, lp = _local(local, n)
    if acc is None:
        lib().hpo_sparse_decode_merge_local(arr, len(keep), lp, _p(agg), n, None, None, ratio)
        return agg
    acc = _f32c(acc).copy()
    out = _payload(sparse_payload_bytes(n, ratio))
    lib().hpo_sparse_decode_merge_local(arr, len(keep), lp, _p(agg), n, _p(acc), _p(out), ratio)
    return agg, out, acc


# -- CompLL generated-operator format -------------------------------------------
def compll_decode(compressed, out_cap):
    compressed = np.ascontiguousarray(compressed, dtype=np.uint8)
    out = np.zeros(out_cap, dtype=np.float32)
    cnt = lib().hpo_compll_decode(_p(compressed), compressed.size, _p(out), out_cap)
    return out[:cnt]


def compll_payload_bytes(n, b):
    return int(lib().hpo_compll_payload_bytes(n, b))


def compll_encode(g, u, b):
    g, u = _f32c(g), _f32c(u)
    pay = _payload(compll_payload_bytes(g.size, b))
    lib().hpo_compll_encode(_p(g), _p(u), g.size, _p(pay), b)
    return pay


def lcg_uniform(seed, n, lo=0.0, hi=1.0):
    out = np.empty(n, dtype=np.float32)
    lib().hpo_lcg_uniform(seed, lo, hi, _p(out), n)
    return out


def uniform_draws(seed, n, tensor=0):
    """The noise an encoder called with `seed` draws for the n elements of tensor `tensor`
    of its launch (0 for a per-tensor call)."""
    out = np.empty(n, dtype=np.float32)
    lib().hpo_uniform_draws(seed, tensor, _p(out), n)
    return out


def uniform_tensor_key(seed, tensor=0):
    return int(lib().hpo_uniform_tensor_key(seed, tensor))
