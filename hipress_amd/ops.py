"""In-place PyTorch operators over the C ABI.

The surface follows the reference's operator convention
(/root/reference/src/CompLL/GCGen/output/TernGradEncode/TernGradEncode.cc:10-24,
 /root/reference/src/CompLL/GCGen/output/TernGradDecode/TernGradDecode.cc:10-24):
encode takes ``(gradient, [state...], compressed, *scalars)``, decode takes
``(compressed, gradient)``; every buffer is allocated by the caller, updated in
place, and nothing is returned.  ``gradient`` must be float32 and ``compressed``
uint8, the two type checks the reference makes
(TernGradEncode_wrapper.h:35-38); here a violation raises ``TypeError`` instead
of aborting the process.

Operator names are ``<alg>_encode`` / ``<alg>_decode`` / ``<alg>_decode_merge``
for the algorithm tokens the reference's launch lines use (onebit, tbq,
terngrad, dgc, graddrop; /root/reference/README.md:9,45,160,276), with
CompLL-style aliases (``TernGradEncode`` ...: TernGradEncode.cc:10) kept in
``ALIASES``.  All of them are also registered as ``torch.ops.hipress.<name>``.
"""
import contextlib
import ctypes

import torch

from . import _lib
from ._lib import ALG_IDS, MAX_PEERS, MergeChunk, Params, Tensor, check, size

__all__ = [
    "onebit_payload_bytes", "tbq_payload_bytes", "terngrad_payload_bytes", "sparse_capacity",
    "sparse_payload_bytes", "dgc_payload_bytes", "graddrop_payload_bytes",
    "onebit_encode", "onebit_decode", "onebit_encode_deferred", "onebit_residual", "tbq_encode", "tbq_decode", "terngrad_encode", "terngrad_decode",
    "dgc_encode", "dgc_decode", "graddrop_encode", "graddrop_decode",
    "terngrad_encode_seeded", "uniform_fill", "compll_terngrad_encode_seeded",
    "compll_payload_bytes", "compll_decoded_count", "compll_terngrad_encode", "compll_terngrad_decode",
    "onebit_decode_merge", "tbq_decode_merge", "terngrad_decode_merge", "dgc_decode_merge",
    "graddrop_decode_merge", "Batch", "MergeBatch", "PlannedSet", "PlannedMerge", "ALIASES",
]


# ---------------------------------------------------------------- sizes
def onebit_payload_bytes(n):
    return size(_lib.lib().hipress_onebit_payload_bytes(n), "onebit_payload_bytes")


def tbq_payload_bytes(n):
    return size(_lib.lib().hipress_tbq_payload_bytes(n), "tbq_payload_bytes")


def terngrad_payload_bytes(n, bucket=512):
    return size(_lib.lib().hipress_terngrad_payload_bytes(n, bucket), "terngrad_payload_bytes")


def sparse_capacity(n, ratio):
    return size(_lib.lib().hipress_sparse_capacity(n, ratio), "sparse_capacity")


def sparse_payload_bytes(n, ratio):
    return size(_lib.lib().hipress_sparse_payload_bytes(n, ratio), "sparse_payload_bytes")


dgc_payload_bytes = sparse_payload_bytes
graddrop_payload_bytes = sparse_payload_bytes


# ---------------------------------------------------------------- argument checks
def _f32(t, name, like=None):
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{name} must be a torch.Tensor")
    if t.dtype != torch.float32:
        raise TypeError(f"type of {name} should be float")
    _common(t, name, like)
    return t


def _u8(t, name, like=None):
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{name} must be a torch.Tensor")
    if t.dtype != torch.uint8:
        raise TypeError(f"type of {name} should be uint8")
    _common(t, name, like)
    return t


def _common(t, name, like):
    if not t.is_cuda:
        raise ValueError(f"{name} must live on the GPU (hipress_amd has no CPU path)")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous")
    if like is not None:
        if t.device != like.device:
            raise ValueError(f"{name} is on {t.device}, expected {like.device}")


def _same_numel(a, b, na, nb):
    if a.numel() != b.numel():
        raise ValueError(f"{na} has {a.numel()} elements, {nb} has {b.numel()}")


_NO_SWITCH = contextlib.nullcontext()


def _on(device):
    """Makes `device` current for a call; costs nothing when it already is (the usual case,
    and the one where a few microseconds per call matter: small tensors are launch-bound)."""
    return _NO_SWITCH if torch.cuda.current_device() == device.index else torch.cuda.device(device)


# torch's own extensions read the current stream's handle through this accessor; it skips
# the Stream object that torch.cuda.current_stream builds (about 2 microseconds a call,
# which shows on launch-bound tensors)
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _device_stream(device):
    if _raw_stream is not None:
        return _raw_stream(device.index)
    return torch.cuda.current_stream(device).cuda_stream


def _stream(t):
    return _device_stream(t.device)


_workspaces = {}


def _workspace(t, nbytes):
    """Scratch buffer per (device, stream), grown on demand and reused."""
    key = (t.device.index, _stream(t))
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = torch.empty(max(int(nbytes), 1 << 16), dtype=torch.uint8, device=t.device)
        _workspaces[key] = ws
    return ws


def _p(t):
    return t.data_ptr() if t is not None else None


# ---------------------------------------------------------------- TBQ
def tbq_encode(gradient, residual, compressed, threshold):
    """Threshold two-bit quantisation with error feedback; residual is updated in place."""
    _f32(gradient, "gradient"); _f32(residual, "residual", gradient); _u8(compressed, "compressed", gradient)
    _same_numel(gradient, residual, "gradient", "residual")
    with _on(gradient.device):
        check(_lib.lib().hipress_tbq_encode(_p(gradient), _p(residual), gradient.numel(), _p(compressed),
                                            compressed.numel(), float(threshold), _stream(gradient)), "tbq_encode")


def tbq_decode(compressed, gradient):
    _u8(compressed, "compressed"); _f32(gradient, "gradient", compressed)
    with _on(gradient.device):
        check(_lib.lib().hipress_tbq_decode(_p(compressed), compressed.numel(), _p(gradient), gradient.numel(),
                                            _stream(gradient)), "tbq_decode")


# ---------------------------------------------------------------- onebit
def onebit_encode(gradient, residual, compressed):
    """Sign bits + mean-magnitude scale with error feedback; residual is updated in place."""
    _f32(gradient, "gradient"); _f32(residual, "residual", gradient); _u8(compressed, "compressed", gradient)
    _same_numel(gradient, residual, "gradient", "residual")
    L = _lib.lib()
    n = gradient.numel()
    with _on(gradient.device):
        need = size(L.hipress_onebit_workspace_bytes(n), "onebit_workspace_bytes")
        ws = _workspace(gradient, need)
        check(L.hipress_onebit_encode(_p(gradient), _p(residual), n, _p(compressed), compressed.numel(),
                                      _p(ws), ws.numel(), _stream(gradient)), "onebit_encode")


def onebit_encode_deferred(gradient, state, scale_state, compressed):
    """onebit_encode in one pass per step: `state` holds v = residual + gradient of the
    previous step (initially the residual) and `scale_state` (1 float, initially 0) its
    scale; the payloads equal onebit_encode's.  Use onebit_residual to read the residual."""
    _f32(gradient, "gradient"); _f32(state, "state", gradient); _f32(scale_state, "scale_state", gradient)
    _u8(compressed, "compressed", gradient)
    _same_numel(gradient, state, "gradient", "state")
    if scale_state.numel() != 1:
        raise ValueError("scale_state must hold exactly one float")
    L = _lib.lib()
    n = gradient.numel()
    with _on(gradient.device):
        ws = _workspace(gradient, size(L.hipress_onebit_workspace_bytes(n), "onebit_workspace_bytes"))
        check(L.hipress_onebit_encode_deferred(_p(gradient), _p(state), _p(scale_state), n, _p(compressed),
                                               compressed.numel(), _p(ws), ws.numel(), _stream(gradient)),
              "onebit_encode_deferred")


def onebit_residual(state, scale_state, residual):
    """residual = the error-feedback residual onebit_encode would hold after the same steps."""
    _f32(state, "state"); _f32(scale_state, "scale_state", state); _f32(residual, "residual", state)
    _same_numel(state, residual, "state", "residual")
    with _on(state.device):
        check(_lib.lib().hipress_onebit_residual(_p(state), _p(scale_state), state.numel(), _p(residual),
                                                 _stream(state)), "onebit_residual")


def onebit_decode(compressed, gradient):
    _u8(compressed, "compressed"); _f32(gradient, "gradient", compressed)
    with _on(gradient.device):
        check(_lib.lib().hipress_onebit_decode(_p(compressed), compressed.numel(), _p(gradient), gradient.numel(),
                                               _stream(gradient)), "onebit_decode")


# ---------------------------------------------------------------- TernGrad
def terngrad_encode(gradient, uniform, compressed, bucket=512):
    """Stochastic ternarisation; `uniform` holds one U[0,1) draw per element."""
    _f32(gradient, "gradient"); _f32(uniform, "uniform", gradient); _u8(compressed, "compressed", gradient)
    _same_numel(gradient, uniform, "gradient", "uniform")
    with _on(gradient.device):
        check(_lib.lib().hipress_terngrad_encode(_p(gradient), _p(uniform), gradient.numel(), _p(compressed),
                                                 compressed.numel(), int(bucket), _stream(gradient)), "terngrad_encode")


def _seed(seed):
    """A caller's seed as the C ABI takes it (64 bits); None draws one from torch's CPU
    generator, so that torch.manual_seed makes a run repeatable and every call differs."""
    if seed is None:
        return int(torch.randint(0, 2 ** 62, (1,)).item())
    return int(seed) & 0xFFFFFFFFFFFFFFFF


def terngrad_encode_seeded(gradient, compressed, bucket=512, seed=None):
    """terngrad_encode with the noise drawn inside the kernel from `seed` (a new one every
    step; None takes one from torch's CPU generator): no noise tensor is made, kept or read.
    The payload equals that of terngrad_encode with uniform_fill(seed)'s values."""
    _f32(gradient, "gradient"); _u8(compressed, "compressed", gradient)
    with _on(gradient.device):
        check(_lib.lib().hipress_terngrad_encode_seeded(_p(gradient), gradient.numel(), _p(compressed), compressed.numel(),
                                                        int(bucket), _seed(seed), _stream(gradient)), "terngrad_encode_seeded")


def uniform_fill(out, seed, tensor=0):
    """out[i] = the noise a seeded encoder draws for element i of tensor number `tensor` of its
    launch (0 for a per-tensor call, the place in the table for a Batch)."""
    _f32(out, "out")
    with _on(out.device):
        check(_lib.lib().hipress_uniform_fill(_p(out), out.numel(), _seed(seed), int(tensor), _stream(out)), "uniform_fill")


def terngrad_decode(compressed, gradient):
    _u8(compressed, "compressed"); _f32(gradient, "gradient", compressed)
    with _on(gradient.device):
        check(_lib.lib().hipress_terngrad_decode(_p(compressed), compressed.numel(), _p(gradient), gradient.numel(),
                                                 _stream(gradient)), "terngrad_decode")


# ---------------------------------------------------------------- the in-tree CompLL operator
def compll_payload_bytes(n, bitwidth=2):
    return size(_lib.lib().hipress_compll_payload_bytes(n, int(bitwidth)), "compll_payload_bytes")


def compll_decoded_count(n, bitwidth=2):
    """Elements compll_terngrad_decode writes for a payload encoded from n elements: the
    reference's count (8 * code bytes / bitwidth - tail, tail = n mod 2**bitwidth), which is
    smaller than n for some n; the rest of the output buffer is left untouched."""
    return size(_lib.lib().hipress_compll_decoded_count(n, int(bitwidth)), "compll_decoded_count")


def compll_terngrad_encode(gradient, uniform, compressed, bitwidth=2):
    """The operator CompLL generates from pse/TernGradEncode.pse: min/max `bitwidth`-bit
    stochastic quantiser with the 10-byte header; `uniform` replaces random<float>(0,1)."""
    _f32(gradient, "gradient"); _f32(uniform, "uniform", gradient); _u8(compressed, "compressed", gradient)
    _same_numel(gradient, uniform, "gradient", "uniform")
    L = _lib.lib()
    n = gradient.numel()
    with _on(gradient.device):
        ws = _workspace(gradient, size(L.hipress_compll_workspace_bytes(n), "compll_workspace_bytes"))
        check(L.hipress_compll_encode(_p(gradient), _p(uniform), n, _p(compressed), compressed.numel(), int(bitwidth),
                                      _p(ws), ws.numel(), _stream(gradient)), "compll_encode")


def compll_terngrad_encode_seeded(gradient, compressed, bitwidth=2, seed=None):
    """compll_terngrad_encode with the noise drawn inside the kernel from `seed`, as the
    reference's operator draws its own: the signature the reference registers, plus the seed."""
    _f32(gradient, "gradient"); _u8(compressed, "compressed", gradient)
    L = _lib.lib()
    n = gradient.numel()
    with _on(gradient.device):
        ws = _workspace(gradient, size(L.hipress_compll_workspace_bytes(n), "compll_workspace_bytes"))
        check(L.hipress_compll_encode_seeded(_p(gradient), n, _p(compressed), compressed.numel(), int(bitwidth), _seed(seed),
                                             _p(ws), ws.numel(), _stream(gradient)), "compll_encode_seeded")


def compll_terngrad_decode(compressed, gradient):
    """Decode of that format; the element count comes from the payload length and its tail
    byte as in the reference and can fall short of gradient.numel() (see compll_decoded_count):
    elements past it keep what the caller put there, so pass a zeroed buffer if that matters."""
    _u8(compressed, "compressed"); _f32(gradient, "gradient", compressed)
    with _on(gradient.device):
        check(_lib.lib().hipress_compll_decode(_p(compressed), compressed.numel(), _p(gradient), gradient.numel(),
                                               _stream(gradient)), "compll_decode")


# ---------------------------------------------------------------- DGC / GradDrop
def dgc_encode(gradient, momentum, accumulator, compressed, momentum_factor=0.9, ratio=0.001):
    """Deep gradient compression: momentum correction, local accumulation,
    sampled-threshold top-`ratio` selection; momentum and accumulator are updated in place."""
    _f32(gradient, "gradient"); _f32(momentum, "momentum", gradient); _f32(accumulator, "accumulator", gradient)
    _u8(compressed, "compressed", gradient)
    _same_numel(gradient, momentum, "gradient", "momentum"); _same_numel(gradient, accumulator, "gradient", "accumulator")
    L = _lib.lib()
    n = gradient.numel()
    with _on(gradient.device):
        need = size(L.hipress_sparse_workspace_bytes(n, float(ratio)), "sparse_workspace_bytes")
        ws = _workspace(gradient, need)
        check(L.hipress_dgc_encode(_p(gradient), _p(momentum), _p(accumulator), n, _p(compressed), compressed.numel(),
                                   float(momentum_factor), float(ratio), _p(ws), ws.numel(), _stream(gradient)), "dgc_encode")


def graddrop_encode(gradient, accumulator, compressed, ratio=0.01):
    """Gradient dropping: `ratio` is the kept fraction (drop ratio 0.99 = ratio 0.01)."""
    _f32(gradient, "gradient"); _f32(accumulator, "accumulator", gradient); _u8(compressed, "compressed", gradient)
    _same_numel(gradient, accumulator, "gradient", "accumulator")
    L = _lib.lib()
    n = gradient.numel()
    with _on(gradient.device):
        need = size(L.hipress_sparse_workspace_bytes(n, float(ratio)), "sparse_workspace_bytes")
        ws = _workspace(gradient, need)
        check(L.hipress_graddrop_encode(_p(gradient), _p(accumulator), n, _p(compressed), compressed.numel(),
                                        float(ratio), _p(ws), ws.numel(), _stream(gradient)), "graddrop_encode")


def dgc_decode(compressed, gradient):
    _u8(compressed, "compressed"); _f32(gradient, "gradient", compressed)
    with _on(gradient.device):
        check(_lib.lib().hipress_sparse_decode(_p(compressed), compressed.numel(), _p(gradient), gradient.numel(),
                                               _stream(gradient)), "sparse_decode")


graddrop_decode = dgc_decode


# ---------------------------------------------------------------- the reference's own operator names
def TernGradEncode(gradient, compressed, bitwidth=2, uniform=None, seed=None):
    """The operator the reference registers under this name
    (/root/reference/src/CompLL/GCGen/output/TernGradEncode/TernGradEncode.cc:10-24):
    arguments (gradient, compressed, bitwidth), the min/max `bitwidth`-bit stochastic
    quantiser with the 10-byte [bitwidth][tail][min][max] header.  The reference draws its
    rounding noise inside the operator from a clock-seeded generator
    (TernGradEncode_body.h:49,119); here `uniform` supplies it, and when it is left out the
    kernel draws it itself from `seed` (None: a seed from torch's CPU generator, a new one
    every call)."""
    if uniform is None:
        compll_terngrad_encode_seeded(gradient, compressed, bitwidth, seed)
    else:
        compll_terngrad_encode(gradient, uniform, compressed, bitwidth)


def TernGradDecode(compressed, gradient):
    """Decode of TernGradEncode's format, arguments as the reference registers them
    (/root/reference/src/CompLL/GCGen/output/TernGradDecode/TernGradDecode.cc:10-24)."""
    compll_terngrad_decode(compressed, gradient)


# ---------------------------------------------------------------- decode-and-merge
def _peers(compressed_list, like):
    if not 1 <= len(compressed_list) <= MAX_PEERS:
        raise ValueError(f"between 1 and {MAX_PEERS} peer payloads are supported, got {len(compressed_list)}")
    for i, c in enumerate(compressed_list):
        _u8(c, f"compressed[{i}]", like)
    P = len(compressed_list)
    ptrs = (ctypes.c_void_p * P)(*[c.data_ptr() for c in compressed_list])
    lens = (ctypes.c_int64 * P)(*[c.numel() for c in compressed_list])
    return ptrs, lens, P


def _local_of(local, like):
    """The aggregator's own uncompressed gradient a merge starts from, or None (zero)."""
    if local is not None:
        _f32(local, "local", like)
        _same_numel(like, local, "aggregate", "local")
    return local


def tbq_decode_merge(compressed_list, aggregate, residual=None, out_compressed=None, threshold=0.0, local=None):
    """aggregate = sum of the decoded peers; with `residual` given the aggregate is
    re-encoded into `out_compressed` with the aggregator's own residual, and `aggregate`
    may then be None (only the re-encoded payload is produced).  With `local` (fp32, the
    aggregator's own gradient) the sum starts from it instead of zero: one hop of a ring."""
    like = aggregate if aggregate is not None else residual
    if like is None:
        raise TypeError("aggregate may only be None when residual and out_compressed are given")
    if aggregate is not None:
        _f32(aggregate, "aggregate")
    ptrs, lens, P = _peers(compressed_list, like)
    if residual is not None:
        _f32(residual, "residual", like); _u8(out_compressed, "out_compressed", like)
        _same_numel(like, residual, "aggregate", "residual")
    _local_of(local, like)
    with _on(like.device):
        check(_lib.lib().hipress_tbq_decode_merge_local(
            ptrs, lens, P, _p(local), _p(aggregate), like.numel(), _p(residual), _p(out_compressed),
            out_compressed.numel() if out_compressed is not None else 0, float(threshold), _stream(like)),
            "tbq_decode_merge")


def onebit_decode_merge(compressed_list, aggregate, local=None):
    _f32(aggregate, "aggregate")
    ptrs, lens, P = _peers(compressed_list, aggregate)
    _local_of(local, aggregate)
    with _on(aggregate.device):
        check(_lib.lib().hipress_onebit_decode_merge_local(ptrs, lens, P, _p(local), _p(aggregate), aggregate.numel(),
                                                           _stream(aggregate)), "onebit_decode_merge")


def terngrad_decode_merge(compressed_list, aggregate, local=None):
    _f32(aggregate, "aggregate")
    ptrs, lens, P = _peers(compressed_list, aggregate)
    _local_of(local, aggregate)
    with _on(aggregate.device):
        check(_lib.lib().hipress_terngrad_decode_merge_local(ptrs, lens, P, _p(local), _p(aggregate), aggregate.numel(),
                                                             _stream(aggregate)), "terngrad_decode_merge")


def dgc_decode_merge(compressed_list, aggregate, accumulator=None, out_compressed=None, ratio=0.001, local=None):
    """Scatter-add of the peers' (index, value) pairs; with `accumulator` given the
    aggregate is re-sparsified into `out_compressed` (accumulator = aggregator residual),
    and `aggregate` may then be None (only the re-encoded payload is produced).  With
    `local` (fp32, the aggregator's own gradient) the sum starts from it instead of zero."""
    like = aggregate if aggregate is not None else accumulator
    if like is None:
        raise TypeError("aggregate may only be None when accumulator and out_compressed are given")
    if aggregate is not None:
        _f32(aggregate, "aggregate")
    ptrs, lens, P = _peers(compressed_list, like)
    L = _lib.lib()
    n = like.numel()
    ws = None
    if accumulator is not None:
        _f32(accumulator, "accumulator", like); _u8(out_compressed, "out_compressed", like)
        _same_numel(like, accumulator, "aggregate", "accumulator")
    _local_of(local, like)
    with _on(like.device):
        ws = _workspace(like, size(L.hipress_sparse_merge_workspace_bytes(n, P, float(ratio), int(accumulator is not None)),
                                   "sparse_merge_workspace_bytes"))
        check(L.hipress_sparse_decode_merge_local(
            ptrs, lens, P, _p(local), _p(aggregate), n, _p(accumulator), _p(out_compressed),
            out_compressed.numel() if out_compressed is not None else 0, float(ratio),
            _p(ws), ws.numel() if ws is not None else 0, _stream(like)), "sparse_decode_merge")


graddrop_decode_merge = dgc_decode_merge


# ---------------------------------------------------------------- batched launches
class Batch:
    """All tensors of a gradient set behind one launch sequence.

    ``tensors`` is a list of dicts with the keys the algorithm needs:
    gradient, residual (onebit, tbq), momentum + accumulator (dgc), accumulator
    (graddrop), uniform (terngrad), compressed, and ``out`` for decode.  The
    tensors must stay alive and keep their addresses for the life of the batch.
    A terngrad batch none of whose tensors has ``uniform`` draws its noise in the
    kernel: ``encode(seed=...)``.
    """

    def __init__(self, alg, tensors, threshold=0.0, bucket=512, momentum_factor=0.9, ratio=0.001):
        self.alg = alg
        self._keep = tensors
        alg_id = ALG_IDS[alg]
        arr = (Tensor * max(len(tensors), 1))()
        dev = None
        for i, t in enumerate(tensors):
            c = _u8(t["compressed"], "compressed")
            dev = dev or c.device
            g = t.get("gradient")
            if alg in ("onebit", "tbq"):
                s0, s1 = t.get("residual"), None
            elif alg == "onebit_deferred":
                s0, s1 = t.get("state"), t.get("scale_state")
            elif alg == "dgc":
                s0, s1 = t.get("momentum"), t.get("accumulator")
            elif alg == "graddrop":
                s0, s1 = t.get("accumulator"), None
            else:
                s0, s1 = None, None
            u, o = t.get("uniform"), t.get("out")
            for name, x in (("gradient", g), ("state", s0), ("state", s1), ("uniform", u), ("out", o)):
                if x is not None:
                    _f32(x, name, c)
            n = (g if g is not None else o).numel()
            arr[i] = Tensor(_p(g), _p(s0), _p(s1), _p(u), _p(c), _p(o), n, c.numel())
        self.device = dev
        pr = Params(float(threshold), int(bucket), float(momentum_factor), 0.0, float(ratio))
        h = ctypes.c_void_p()
        with _on(dev):
            check(_lib.lib().hipress_batch_create(ctypes.byref(h), alg_id, arr, len(tensors), ctypes.byref(pr)), "batch_create")
        self._h = h
        # as the library decides it: some tensor with elements comes without a noise tensor (all of them, or the
        # library has refused the batch)
        self.seeded = alg == "terngrad" and any(
            t.get("gradient") is not None and t["gradient"].numel() > 0 and t.get("uniform") is None for t in tensors)

    def encode(self, seed=None):
        """``seed``: for a terngrad batch without noise tensors (None: one from torch's CPU
        generator); tensor k of the table draws with tensor = k."""
        with _on(self.device):
            if self.seeded:
                check(_lib.lib().hipress_batch_encode_seeded(self._h, _seed(seed), _device_stream(self.device)),
                      "batch_encode_seeded")
            else:
                check(_lib.lib().hipress_batch_encode(self._h, _device_stream(self.device)), "batch_encode")

    def encode_phase(self, phase):
        """One launch of the encode sequence (measurement aid)."""
        with _on(self.device):
            check(_lib.lib().hipress_batch_encode_phase(self._h, int(phase), _device_stream(self.device)), "batch_encode_phase")

    def decode(self):
        with _on(self.device):
            check(_lib.lib().hipress_batch_decode(self._h, _device_stream(self.device)), "batch_decode")

    def close(self):
        if getattr(self, "_h", None):
            _lib.lib().hipress_batch_destroy(self._h)
            self._h = None

    def __del__(self):
        # at interpreter shutdown the library module may already be gone
        try:
            self.close()
        except Exception:
            pass


class MergeBatch:
    """Decode-and-merge of many chunks in one launch sequence.

    ``chunks``: list of dicts with ``compressed`` (list of peer payload tensors),
    ``aggregate``, and optionally ``state`` + ``out_compressed`` for the fused
    re-encode (tbq: aggregator residual; dgc/graddrop: aggregator accumulator).
    With the re-encode a chunk's ``aggregate`` may be None: the sum is then not
    written as fp32, only the re-encoded payload and the state are produced.  A chunk's
    ``local`` (fp32, the aggregator's own gradient for that chunk) makes its sum start
    from there instead of zero.
    """

    def __init__(self, alg, chunks, threshold=0.0, bucket=512, ratio=0.001):
        self._keep = chunks
        npeers = len(chunks[0]["compressed"]) if chunks else 1
        arr = (MergeChunk * max(len(chunks), 1))()
        dev = None
        for i, c in enumerate(chunks):
            st, oc = c.get("state"), c.get("out_compressed")
            agg = c.get("aggregate")
            like = agg if agg is not None else st
            if like is None:
                raise TypeError("a chunk needs an aggregate, or a state and out_compressed to re-encode into")
            if agg is not None:
                _f32(agg, "aggregate")
            dev = dev or like.device
            if len(c["compressed"]) != npeers:
                raise ValueError("every chunk must have the same number of peers")
            mc = MergeChunk()
            for p, pay in enumerate(c["compressed"]):
                _u8(pay, "compressed", like)
                mc.payloads[p] = pay.data_ptr()
                mc.payload_bytes[p] = pay.numel()
            mc.aggregate = agg.data_ptr() if agg is not None else None
            if st is not None:
                _f32(st, "state", like); _u8(oc, "out_compressed", like)
                mc.state, mc.out_payload, mc.out_payload_bytes = st.data_ptr(), oc.data_ptr(), oc.numel()
            loc = _local_of(c.get("local"), like)
            mc.local = loc.data_ptr() if loc is not None else None
            mc.n = like.numel()
            arr[i] = mc
        self.device = dev
        pr = Params(float(threshold), int(bucket), 0.0, 0.0, float(ratio))
        h = ctypes.c_void_p()
        with _on(dev):
            check(_lib.lib().hipress_merge_batch_create(ctypes.byref(h), ALG_IDS[alg], arr, len(chunks), npeers,
                                                        ctypes.byref(pr)), "merge_batch_create")
        self._h = h

    def run(self):
        with _on(self.device):
            check(_lib.lib().hipress_merge_batch_run(self._h, _device_stream(self.device)), "merge_batch_run")

    def run_phase(self, phase):
        """One part of the launch sequence (measurement aid)."""
        with _on(self.device):
            check(_lib.lib().hipress_merge_batch_run_phase(self._h, int(phase), _device_stream(self.device)),
                  "merge_batch_run_phase")

    def close(self):
        if getattr(self, "_h", None):
            _lib.lib().hipress_merge_batch_destroy(self._h)
            self._h = None

    def __del__(self):
        # at interpreter shutdown the library module may already be gone
        try:
            self.close()
        except Exception:
            pass

class PlannedSet:
    """A model's gradients under a SeCoPa plan, on one GPU.

    The plan (`name,size,y|n,K` lines, /root/reference/src/SeCoPa/SeCoPa.py:139-151, or the
    tuples ``planner.read_plan`` returns) says for every gradient whether to compress it
    and into how many partitions to cut it.  A gradient marked ``y`` is cut with
    ``planner.partition_bounds`` and every partition is compressed on its own - its own
    payload, header and statistics - since the partition is the unit the runtime encodes,
    sends and merges (/root/reference/README.md:134).  A gradient marked ``n`` is left
    alone and listed in ``uncompressed``.  All partitions of the set run in one launch
    sequence (a ``Batch``).

    ``gradients``: dict name -> contiguous float32 tensor, which must keep its address.
    The set allocates what the algorithm needs beside them and exposes it by gradient
    name: ``state[name]`` (dict of whole-gradient tensors: residual / momentum,
    accumulator / state, scale_state per partition), ``compressed[name]`` (one uint8
    payload per partition), ``out[name]`` (the decoded gradient, whole).  TernGrad reads
    its rounding noise from ``uniform[name]``, one float32 tensor per compressed gradient,
    or, with ``uniform=None``, draws it in the kernel: ``encode(seed=...)``.
    """

    def __init__(self, alg, plan, gradients, uniform=None, threshold=0.0, bucket=512, momentum_factor=0.9,
                 ratio=0.001):
        from . import planner

        if alg not in ALG_IDS:
            raise ValueError(f"unknown algorithm {alg!r}")
        self.alg = alg
        self.parts, self.uncompressed = [], []
        self.state, self.compressed, self.out = {}, {}, {}
        nbytes = {"onebit": onebit_payload_bytes, "onebit_deferred": onebit_payload_bytes, "tbq": tbq_payload_bytes,
                  "terngrad": lambda n: terngrad_payload_bytes(n, bucket),
                  "dgc": lambda n: sparse_payload_bytes(n, ratio),
                  "graddrop": lambda n: sparse_payload_bytes(n, ratio)}[alg]
        state_names = {"onebit": ("residual",), "tbq": ("residual",), "onebit_deferred": ("state",),
                       "dgc": ("momentum", "accumulator"), "graddrop": ("accumulator",), "terngrad": ()}[alg]
        tensors = []
        for entry in plan:
            name, size_, compress, k = planner.parse_plan_line(entry) if isinstance(entry, str) else entry
            if name not in gradients:
                raise KeyError(f"the plan names {name!r}, which is not among the gradients")
            g = gradients[name]
            if g.numel() != size_:
                raise ValueError(f"{name}: the plan says {size_} elements, the gradient has {g.numel()}")
            if not compress:
                self.uncompressed.append(name)
                continue
            _f32(g, name)
            flat = g.view(-1)
            st = {s: torch.zeros_like(flat) for s in state_names}
            out = torch.empty_like(flat)
            bounds = planner.partition_bounds(size_, k)
            if alg == "onebit_deferred":
                st["scale_state"] = torch.zeros(max(len(bounds), 1), device=g.device)
            u = None
            if alg == "terngrad" and uniform is not None:
                if name not in uniform:
                    raise KeyError(f"terngrad needs uniform[{name!r}]")
                u = _f32(uniform[name], "uniform", g).view(-1)
                _same_numel(u, flat, "uniform", name)
            pays = []
            for i, (off, length) in enumerate(bounds):
                pay = torch.zeros(nbytes(length), dtype=torch.uint8, device=g.device)
                t = {"gradient": flat[off:off + length], "out": out[off:off + length], "compressed": pay}
                for s in state_names:
                    t[s] = st[s][off:off + length]
                if alg == "onebit_deferred":
                    t["scale_state"] = st["scale_state"][i:i + 1]
                if u is not None:
                    t["uniform"] = u[off:off + length]
                tensors.append(t)
                pays.append(pay)
                self.parts.append({"name": name, "index": i, "offset": off, "length": length})
            self.state[name], self.compressed[name], self.out[name] = st, pays, out
        self.elements = sum(p["length"] for p in self.parts)
        self._batch = Batch(alg, tensors, threshold=threshold, bucket=bucket, momentum_factor=momentum_factor,
                            ratio=ratio) if tensors else None

    def encode(self, seed=None):
        if self._batch is not None:
            self._batch.encode(seed)

    def decode(self):
        if self._batch is not None:
            self._batch.decode()

    def close(self):
        if getattr(self, "_batch", None) is not None:
            self._batch.close()
            self._batch = None

class PlannedMerge:
    """The aggregator's side of a SeCoPa plan on one GPU: for every partition of every
    gradient the plan marks ``y``, the peers' payloads are decoded and summed in peer order
    and, with ``reencode=True`` (tbq, dgc, graddrop), the sum is compressed again for the next
    hop with the aggregator's own residual / accumulator - all partitions of the model in
    one launch sequence (a ``MergeBatch``).

    ``peers``: one entry per peer, each a dict name -> list of that gradient's partition
    payloads, as ``PlannedSet.compressed`` of the sending side holds them.  The object
    allocates and exposes by gradient name ``aggregate[name]`` (the fp32 sum, whole
    gradient), and with the re-encode ``state[name]`` and ``out_compressed[name]`` (one
    payload per partition).  ``local``: dict name -> the aggregator's own uncompressed
    gradient; the sums of those gradients start from it instead of zero.
    """

    def __init__(self, alg, plan, peers, reencode=False, local=None, threshold=0.0, bucket=512, ratio=0.001):
        from . import planner

        if alg not in ALG_IDS or alg == "onebit_deferred":
            raise ValueError(f"no decode-and-merge for algorithm {alg!r}")
        if reencode and alg not in ("tbq", "dgc", "graddrop"):
            raise ValueError(f"{alg} has no fused re-encode")
        if not peers:
            raise ValueError("at least one peer is needed")
        nbytes = {"tbq": tbq_payload_bytes, "dgc": lambda n: sparse_payload_bytes(n, ratio),
                  "graddrop": lambda n: sparse_payload_bytes(n, ratio)}.get(alg)
        self.alg = alg
        self.parts, self.uncompressed = [], []
        self.aggregate, self.state, self.out_compressed = {}, {}, {}
        chunks = []
        for entry in plan:
            name, size_, compress, k = planner.parse_plan_line(entry) if isinstance(entry, str) else entry
            if not compress:
                self.uncompressed.append(name)
                continue
            bounds = planner.partition_bounds(size_, k)
            for p, peer in enumerate(peers):
                if name not in peer or len(peer[name]) != len(bounds):
                    raise ValueError(f"peer {p} does not hold the {len(bounds)} partition payloads of {name!r}")
            if not bounds:
                continue
            dev = peers[0][name][0].device
            agg = torch.empty(size_, device=dev)
            self.aggregate[name] = agg
            if reencode:
                self.state[name] = torch.zeros(size_, device=dev)
                self.out_compressed[name] = [torch.zeros(nbytes(ln), dtype=torch.uint8, device=dev) for _, ln in bounds]
            mine = None
            if local is not None and name in local:
                mine = _f32(local[name], "local").view(-1)
                _same_numel(agg, mine, name, "local")
            for i, (off, ln) in enumerate(bounds):
                c = {"compressed": [peer[name][i] for peer in peers], "aggregate": agg[off:off + ln]}
                if mine is not None:
                    c["local"] = mine[off:off + ln]
                if reencode:
                    c["state"] = self.state[name][off:off + ln]
                    c["out_compressed"] = self.out_compressed[name][i]
                chunks.append(c)
                self.parts.append({"name": name, "index": i, "offset": off, "length": ln})
        self._batch = MergeBatch(alg, chunks, threshold=threshold, bucket=bucket, ratio=ratio) if chunks else None

    def run(self):
        if self._batch is not None:
            self._batch.run()

    def close(self):
        if getattr(self, "_batch", None) is not None:
            self._batch.close()
            self._batch = None


# ---------------------------------------------------------------- aliases + torch.ops registration
# CompLL names its generated operators <Func>Encode / <Func>Decode
# (TernGradEncode.cc:10); one line per name maps them onto the operators above.
# TernGradEncode / TernGradDecode are the reference's own registered operator (the
# min/max quantiser, arguments gradient, compressed, bitwidth); the bucketed max-abs
# ternariser, which the reference names only as the algorithm token "terngrad", goes by
# BucketTernGradEncode / BucketTernGradDecode here.
ALIASES = {
    "OnebitEncode": onebit_encode, "OnebitDecode": onebit_decode,
    "TBQEncode": tbq_encode, "TBQDecode": tbq_decode,
    "TernGradEncode": TernGradEncode, "TernGradDecode": TernGradDecode,
    "BucketTernGradEncode": terngrad_encode, "BucketTernGradDecode": terngrad_decode,
    "DGCEncode": dgc_encode, "DGCDecode": dgc_decode,
    "GradDropEncode": graddrop_encode, "GradDropDecode": graddrop_decode,
}
globals().update(ALIASES)
__all__ += list(ALIASES)

_SCHEMAS = {
    "onebit_encode": "(Tensor gradient, Tensor(a!) residual, Tensor(b!) compressed) -> ()",
    "onebit_decode": "(Tensor compressed, Tensor(a!) gradient) -> ()",
    "tbq_encode": "(Tensor gradient, Tensor(a!) residual, Tensor(b!) compressed, float threshold) -> ()",
    "tbq_decode": "(Tensor compressed, Tensor(a!) gradient) -> ()",
    "terngrad_encode": "(Tensor gradient, Tensor uniform, Tensor(a!) compressed, int bucket=512) -> ()",
    "terngrad_decode": "(Tensor compressed, Tensor(a!) gradient) -> ()",
    "terngrad_encode_seeded": "(Tensor gradient, Tensor(a!) compressed, int bucket=512, int? seed=None) -> ()",
    "uniform_fill": "(Tensor(a!) out, int seed, int tensor=0) -> ()",
    "dgc_encode": "(Tensor gradient, Tensor(a!) momentum, Tensor(b!) accumulator, Tensor(c!) compressed, "
                  "float momentum_factor=0.9, float ratio=0.001) -> ()",
    "dgc_decode": "(Tensor compressed, Tensor(a!) gradient) -> ()",
    "graddrop_encode": "(Tensor gradient, Tensor(a!) accumulator, Tensor(b!) compressed, float ratio=0.01) -> ()",
    "graddrop_decode": "(Tensor compressed, Tensor(a!) gradient) -> ()",
    "compll_terngrad_encode": "(Tensor gradient, Tensor uniform, Tensor(a!) compressed, int bitwidth=2) -> ()",
    "compll_terngrad_decode": "(Tensor compressed, Tensor(a!) gradient) -> ()",
    "compll_terngrad_encode_seeded": "(Tensor gradient, Tensor(a!) compressed, int bitwidth=2, int? seed=None) -> ()",
    "TernGradEncode": "(Tensor gradient, Tensor(a!) compressed, int bitwidth=2, Tensor? uniform=None, int? seed=None) -> ()",
    "TernGradDecode": "(Tensor compressed, Tensor(a!) gradient) -> ()",
    "onebit_decode_merge": "(Tensor[] compressed, Tensor(a!) aggregate, Tensor? local=None) -> ()",
    "terngrad_decode_merge": "(Tensor[] compressed, Tensor(a!) aggregate, Tensor? local=None) -> ()",
    "tbq_decode_merge": "(Tensor[] compressed, Tensor(a!) aggregate, Tensor(b!)? residual=None, "
                        "Tensor(c!)? out_compressed=None, float threshold=0.0, Tensor? local=None) -> ()",
    "dgc_decode_merge": "(Tensor[] compressed, Tensor(a!) aggregate, Tensor(b!)? accumulator=None, "
                        "Tensor(c!)? out_compressed=None, float ratio=0.001, Tensor? local=None) -> ()",
    "graddrop_decode_merge": "(Tensor[] compressed, Tensor(a!) aggregate, Tensor(b!)? accumulator=None, "
                             "Tensor(c!)? out_compressed=None, float ratio=0.01, Tensor? local=None) -> ()",
}
_ALIAS_OF = {
    "OnebitEncode": "onebit_encode", "OnebitDecode": "onebit_decode", "TBQEncode": "tbq_encode",
    "TBQDecode": "tbq_decode", "BucketTernGradEncode": "terngrad_encode", "BucketTernGradDecode": "terngrad_decode",
    "DGCEncode": "dgc_encode", "DGCDecode": "dgc_decode", "GradDropEncode": "graddrop_encode",
    "GradDropDecode": "graddrop_decode",
}


def _register():
    lib = torch.library.Library("hipress", "DEF")
    for name, schema in _SCHEMAS.items():
        lib.define(name + schema)
        lib.impl(name, globals()[name], "CUDA")
    for alias, target in _ALIAS_OF.items():
        lib.define(alias + _SCHEMAS[target])
        lib.impl(alias, globals()[target], "CUDA")
    return lib


_torch_lib = _register()
