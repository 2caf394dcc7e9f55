"""CPU-side checks of the C ABI: the library loads, exports every function
include/hipress_amd.h declares, the ctypes binding covers them all, and the
host-only size arithmetic agrees with the oracle's.  No GPU work is issued."""
import ctypes
import os
import re

import pytest

import oracle

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "hipress_amd.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(hipress_[a-z0-9_]+)\s*\(", text)))


@pytest.fixture(scope="module")
def lib():
    from hipress_amd import _lib

    return _lib


def test_header_declares_the_expected_surface():
    names = declared_functions()
    for alg in ("onebit", "tbq", "terngrad"):
        assert f"hipress_{alg}_encode" in names and f"hipress_{alg}_decode" in names
        assert f"hipress_{alg}_decode_merge" in names
    for n in ("hipress_dgc_encode", "hipress_graddrop_encode", "hipress_sparse_decode", "hipress_sparse_decode_merge",
              "hipress_batch_create", "hipress_batch_encode", "hipress_batch_decode", "hipress_merge_batch_run"):
        assert n in names


def test_library_exports_every_declared_symbol(lib):
    raw = ctypes.CDLL(lib.LIB_PATH)
    for name in declared_functions():
        assert hasattr(raw, name), f"{name} is declared in the header but not exported"
        assert name in lib.SIGNATURES, f"{name} has no ctypes signature"
    assert set(lib.SIGNATURES) == set(declared_functions())


def test_version_and_strerror(lib):
    L = lib.lib()
    assert L.hipress_version() >= 100
    assert lib.strerror(0) == "ok"
    for code in range(-6, 0):
        assert lib.strerror(code) not in ("ok", "unknown error")


@pytest.mark.parametrize("n", [0, 1, 15, 16, 17, 31, 32, 33, 512, 513, 4096, 262143, 262144, 102760448])
def test_sizes_match_oracle(lib, n):
    L = lib.lib()
    assert L.hipress_onebit_payload_bytes(n) == oracle.onebit_payload_bytes(n)
    assert L.hipress_tbq_payload_bytes(n) == oracle.tbq_payload_bytes(n)
    for bucket in (1, 16, 100, 512, 1024):
        assert L.hipress_terngrad_payload_bytes(n, bucket) == oracle.terngrad_payload_bytes(n, bucket)
    for ratio in (0.001, 0.01, 0.5, 1.0):
        assert L.hipress_sparse_capacity(n, ratio) == oracle.sparse_capacity(n, ratio)
        assert L.hipress_sparse_payload_bytes(n, ratio) == oracle.sparse_payload_bytes(n, ratio)
        assert L.hipress_sparse_workspace_bytes(n, ratio) > 0
    assert L.hipress_onebit_workspace_bytes(n) >= 4 * max(1, (n + 4095) // 4096)


def test_size_errors(lib):
    L = lib.lib()
    assert L.hipress_tbq_payload_bytes(-1) == -2
    assert L.hipress_tbq_payload_bytes(1 << 33) == -2
    assert L.hipress_terngrad_payload_bytes(10, 0) == -4
    assert L.hipress_sparse_capacity(10, 0.0) == -4
    assert L.hipress_sparse_capacity(10, 1.5) == -4


def test_null_and_range_checks_need_no_gpu(lib):
    """Argument validation happens before any HIP call."""
    L = lib.lib()
    assert L.hipress_tbq_encode(None, None, 10, None, 100, 0.05, None) == -1
    assert L.hipress_tbq_encode(None, None, -1, None, 100, 0.05, None) == -2
    assert L.hipress_tbq_decode(None, 100, None, 10, None) == -1
    assert L.hipress_batch_encode(None, None) == -1
    assert L.hipress_batch_encode_seeded(None, 1, None) == -1
    assert L.hipress_terngrad_encode_seeded(None, 10, None, 100, 512, 1, None) == -1
    assert L.hipress_terngrad_encode_seeded(None, -1, None, 100, 512, 1, None) == -2
    assert L.hipress_uniform_fill(None, 10, 1, 0, None) == -1
    assert L.hipress_uniform_fill(None, -1, 1, 0, None) == -2
    assert L.hipress_compll_encode_seeded(None, 10, None, 100, 2, 1, None, 0, None) == -1
    assert L.hipress_compll_encode_seeded(None, 10, None, 100, 3, 1, None, 0, None) == -4
    assert L.hipress_merge_batch_run(None, None) == -1
    # a merge without the re-encode needs its aggregate
    import ctypes
    pay = (ctypes.c_void_p * 1)(64)
    nb = (ctypes.c_int64 * 1)(1 << 20)
    assert L.hipress_tbq_decode_merge(pay, nb, 1, None, 16, None, None, 0, 0.05, None) == -1
    assert L.hipress_onebit_decode_merge(pay, nb, 1, None, 16, None) == -1
    # a peer count outside 1 .. 16 is refused before anything is allocated, also for an empty chunk list
    pr = lib.Params(0.05, 512, 0.9, 0.0, 0.001)
    h = ctypes.c_void_p()
    for alg in (lib.TBQ, lib.DGC):
        for npeers in (0, -1, 17):
            assert L.hipress_merge_batch_create(ctypes.byref(h), alg, None, 0, npeers, ctypes.byref(pr)) == -4
            assert not h.value


def test_sparse_entry_points_reject_what_int32_indices_cannot_address(lib):
    """DGC / GradDrop payloads carry int32 indices: n above 2^31 - 1 is refused on the host,
    before any launch (the pointers below are never touched)."""
    L = lib.lib()
    big, ok = (1 << 31), (1 << 31) - 1
    fake = ctypes.c_void_p(1 << 20)
    assert L.hipress_sparse_capacity(big, 0.001) == -2
    assert L.hipress_sparse_payload_bytes(big, 0.001) == -2
    assert L.hipress_sparse_workspace_bytes(big, 0.001) == -2
    assert L.hipress_sparse_merge_workspace_bytes(big, 8, 0.001, 1) == -2
    assert L.hipress_sparse_capacity(ok, 0.001) > 0
    assert L.hipress_sparse_capacity(ok, 1.0) == 1 << 31  # whole tensor, rounded up to 64: still fits u32
    nbytes = 1 << 40
    assert L.hipress_dgc_encode(fake, fake, fake, big, fake, nbytes, 0.9, 0.001, fake, nbytes, None) == -2
    assert L.hipress_graddrop_encode(fake, fake, big, fake, nbytes, 0.01, fake, nbytes, None) == -2
    assert L.hipress_sparse_decode(fake, nbytes, fake, big, None) == -2
    pay = (ctypes.c_void_p * 1)(1 << 20)
    nb = (ctypes.c_int64 * 1)(nbytes)
    assert L.hipress_sparse_decode_merge(pay, nb, 1, fake, big, None, None, 0, 0.001, fake, nbytes, None) == -2
    # batches: the check precedes every allocation
    t = lib.Tensor(fake.value, fake.value, fake.value, None, fake.value, fake.value, big, nbytes)
    pr = lib.Params(0.0, 512, 0.9, 0.0, 0.001)
    h = ctypes.c_void_p()
    for alg in (lib.DGC, lib.GRADDROP):
        assert L.hipress_batch_create(ctypes.byref(h), alg, ctypes.byref(t), 1, ctypes.byref(pr)) == -2
        assert not h.value
    mc = lib.MergeChunk()
    mc.payloads[0], mc.payload_bytes[0] = fake.value, nbytes
    mc.aggregate, mc.n = fake.value, big
    assert L.hipress_merge_batch_create(ctypes.byref(h), lib.DGC, ctypes.byref(mc), 1, 1, ctypes.byref(pr)) == -2
    # the dense formats carry no indices and keep the u32 limit
    assert L.hipress_tbq_payload_bytes(big) > 0


@pytest.mark.parametrize("b", [1, 2, 4, 8])
def test_compll_decoded_count_is_the_reference_formula(lib, b):
    """count = (8 * code bytes) / b - n mod 2^b (TernGradDecode_body.h:70-72 with the
    encoder's tail, TernGradEncode_body.h:118), clamped to n; checked against the oracle's
    decoder, which writes exactly that many elements."""
    import numpy as np

    L = lib.lib()
    for n in (0, 1, 3, 4, 5, 7, 255, 256, 257, 1000, 4097):
        want = min(n, max(0, 8 * ((n * b + 7) // 8) // b - n % (1 << b)))
        assert L.hipress_compll_decoded_count(n, b) == want
        pay = oracle.compll_encode(np.linspace(-1, 1, n, dtype=np.float32), np.zeros(n, np.float32), b)
        assert oracle.compll_decode(pay, n).size == want
    assert L.hipress_compll_decoded_count(10, 3) == -4


def test_reference_operator_names_keep_the_reference_signature():
    """TernGradEncode(gradient, compressed, bitwidth) / TernGradDecode(compressed, gradient) as
    registered in the reference (TernGradEncode.cc:16,21-23; TernGradDecode.cc:16)."""
    import inspect

    import torch

    from hipress_amd import ops

    enc = list(inspect.signature(ops.ALIASES["TernGradEncode"]).parameters)
    assert enc[:3] == ["gradient", "compressed", "bitwidth"]
    assert list(inspect.signature(ops.ALIASES["TernGradDecode"]).parameters) == ["compressed", "gradient"]
    schema = torch.ops.hipress.TernGradEncode.default._schema
    assert [a.name for a in schema.arguments][:3] == ["gradient", "compressed", "bitwidth"]
    assert [a.name for a in torch.ops.hipress.TernGradDecode.default._schema.arguments] == ["compressed", "gradient"]
    assert len(schema.returns) == 0  # in place, zero outputs (TernGradEncode.cc:12-13)
    # the bucketed ternariser keeps its own name
    assert ops.ALIASES["BucketTernGradEncode"] is ops.terngrad_encode


def test_missing_library_is_an_error_not_a_fallback(monkeypatch, tmp_path):
    """Without libhipress_amd.so the operators raise; nothing computes on the CPU instead."""
    import torch

    from hipress_amd import _lib, ops

    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "libhipress_amd.so"))
    with pytest.raises(ImportError, match="no CPU fallback"):
        _lib.lib()
    with pytest.raises(ImportError):
        ops.tbq_payload_bytes(16)
    # and a CPU tensor is refused before any library call
    monkeypatch.undo()
    with pytest.raises(ValueError, match="GPU"):
        ops.tbq_encode(torch.zeros(16), torch.zeros(16), torch.zeros(32, dtype=torch.uint8), 0.05)
    # the package never imports the oracle
    import hipress_amd
    import os
    import re

    root = os.path.dirname(hipress_amd.__file__)
    for dirpath, _, files in os.walk(root):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cpp")):
                text = open(os.path.join(dirpath, f), errors="ignore").read()
                assert not re.search(r"^\s*(import oracle|from oracle)", text, re.M), f
                assert "libhipress_oracle" not in text, f
