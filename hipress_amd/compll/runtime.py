"""Calls operators generated from the shipped programs (hipress_amd/compll/programs)
on torch tensors: in-place operators over caller-allocated buffers, vectors first in
the order the operator declares them, then its scalars, as the reference's generated
operators are called (`TernGradEncode(gradient, compressed, bitwidth=b)`,
/root/reference/src/CompLL/GCGen/output/TernGradEncode/TernGradEncode.cc:10-24).
An operator that draws random numbers takes the uniform[0,1) tensor as `uniform=`, or,
without one, draws in its kernels from `seed=` (left out: a seed from torch's CPU generator).
There is no CPU path: loading fails loudly if the generated library was not built.
"""
import ctypes
import os

from .build import LIB, manifests

_C = {"float": ctypes.c_float, "int": ctypes.c_int32, "int32": ctypes.c_int32, "uint8": ctypes.c_uint8,
      "uint16": ctypes.c_uint16, "uint32": ctypes.c_uint32}
_ERRORS = {-1: "null pointer", -2: "bad size (a buffer is too small)", -3: "misaligned workspace", -4: "bad parameter",
           -5: "HIP error", -6: "workspace missing or too small"}


class GeneratedOpError(RuntimeError):
    pass


class Operators:
    """The operators of a generated library as Python callables.  path: the library
    (default: the one built from the shipped programs); manifest: name -> parameter list,
    by default the file `path + ".json"` that the build writes beside the library."""

    def __init__(self, path=LIB, manifest=None):
        if not os.path.exists(path):
            raise GeneratedOpError(f"{path} is missing: run `python -m hipress_amd.compll.build` "
                                   "(or `python -m hipress_amd.compll prog.pse --library {path}` for a program of your own)")
        self._lib = ctypes.CDLL(path)
        self._workspaces = {}
        if manifest is None:
            if os.path.exists(path + ".json"):
                import json

                with open(path + ".json") as f:
                    manifest = json.load(f)
            elif os.path.abspath(path) == os.path.abspath(LIB):
                manifest = manifests()
            else:
                raise GeneratedOpError(f"{path}.json (the operators' parameter lists) is missing")
        self.manifest = manifest
        for name, m in self.manifest.items():
            fn = getattr(self._lib, name)
            argtypes = []
            for p in m["params"]:
                if p["kind"].endswith("*"):
                    argtypes += [ctypes.c_void_p, ctypes.c_int32]
            argtypes += [_C[p["kind"]] for p in m["params"] if not p["kind"].endswith("*")]
            if m["uniform"]:
                argtypes += [ctypes.c_void_p, ctypes.c_uint64]
            argtypes += [ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p]
            fn.argtypes, fn.restype = argtypes, ctypes.c_int
            ws = getattr(self._lib, name + "_workspace_bytes")
            ws.argtypes, ws.restype = [ctypes.c_int64], ctypes.c_int64
            setattr(self, name, self._bind(name, m, fn, ws))

    def _bind(self, name, m, fn, ws_bytes):
        import torch

        _raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)  # the handle without building a Stream object
        vectors = [p for p in m["params"] if p["kind"].endswith("*")]
        scalars = [p for p in m["params"] if not p["kind"].endswith("*")]

        def call(*args, uniform=None, seed=None, **kw):
            if len(args) > len(vectors) + len(scalars):
                raise TypeError(f"{name} takes {len(vectors) + len(scalars)} positional arguments")
            values = dict(zip([p["name"] for p in vectors + scalars], args))
            for k, v in kw.items():
                if k in values or k not in {p["name"] for p in scalars}:
                    raise TypeError(f"{name}: unexpected argument {k!r}")
                values[k] = v
            missing = [p["name"] for p in vectors + scalars if p["name"] not in values]
            if missing:
                raise TypeError(f"{name}: missing {', '.join(missing)}")
            cargs, biggest, floats, device = [], 0, 0, None
            for p in vectors:
                t = values[p["name"]]
                want = torch.float32 if p["kind"] == "float*" else torch.uint8
                if not isinstance(t, torch.Tensor) or t.dtype != want:
                    raise TypeError(f"{name}: {p['name']} must be a {want} tensor")
                if not t.is_cuda or not t.is_contiguous():
                    raise ValueError(f"{name}: {p['name']} must be a contiguous tensor on the GPU")
                if t.numel() >= 2**31:
                    raise ValueError(f"{name}: {p['name']} is too long")
                device = device or t.device
                biggest = max(biggest, t.numel())
                if p["kind"] == "float*":
                    floats = max(floats, t.numel())
                cargs += [t.data_ptr(), t.numel()]
            cargs += [values[p["name"]] for p in scalars]
            if m["uniform"] and uniform is None:
                # no noise tensor: the kernels draw from a seed (the caller's, or one from torch's CPU generator)
                if seed is None:
                    seed = int(torch.randint(0, 2 ** 62, (1,)).item())
                cargs += [None, int(seed) & 0xFFFFFFFFFFFFFFFF]
            elif m["uniform"]:
                if not isinstance(uniform, torch.Tensor) or uniform.dtype != torch.float32 or not uniform.is_cuda or not uniform.is_contiguous():
                    raise TypeError(f"{name}: uniform= must be a contiguous float32 tensor on the GPU")
                if uniform.numel() < floats:
                    raise ValueError(f"{name}: uniform= is shorter than the float vectors")
                cargs += [uniform.data_ptr(), 0]
            need = ws_bytes(biggest)
            stream = _raw_stream(device.index) if _raw_stream is not None else torch.cuda.current_stream(device).cuda_stream
            key = (device, stream, name)  # scratch is per stream: calls on one stream are ordered, others are not
            ws = self._workspaces.get(key)
            if ws is None or ws.numel() < need:
                ws = self._workspaces[key] = torch.empty(need, dtype=torch.uint8, device=device)
            cargs += [ws.data_ptr(), ws.numel(), stream]
            if torch.cuda.current_device() == device.index:
                rc = fn(*cargs)
            else:
                with torch.cuda.device(device):
                    rc = fn(*cargs)
            if rc != 0:
                raise GeneratedOpError(f"{name}: {_ERRORS.get(rc, rc)}")

        call.__name__ = name
        return call


_ops = None


def load():
    """The operators of the shipped programs, bound to the generated library."""
    global _ops
    if _ops is None:
        _ops = Operators()
    return _ops
