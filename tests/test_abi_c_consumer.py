"""include/hipress_amd.h used from C: a C99 program (tests/csrc/abi_consumer.c) is compiled with
gcc against the header, linked with libhipress_amd.so and run.  It reports the size functions at
fixed element counts, the layout of every struct of the ABI and the host-side argument checks;
the figures are held against constants worked out from the wire format, against the CPU oracle's
own size functions and against the structures hipress_amd/_lib.py declares to ctypes.  No GPU
work is issued (a NULL pointer is refused before any launch)."""
import ctypes
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIBDIR = os.path.join(ROOT, "hipress_amd")


@pytest.fixture(scope="module")
def report(tmp_path_factory):
    if not os.path.exists(os.path.join(LIBDIR, "libhipress_amd.so")):
        pytest.fail("libhipress_amd.so is not built (python -m hipress_amd.build)")
    exe = str(tmp_path_factory.mktemp("abi") / "abi_consumer")
    subprocess.check_call(["gcc", "-std=c99", "-pedantic", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"),
                           os.path.join(ROOT, "tests", "csrc", "abi_consumer.c"), "-o", exe, "-L", LIBDIR, "-lhipress_amd",
                           "-Wl,-rpath," + LIBDIR, "-Wl,-rpath-link,/opt/rocm/lib"])
    r = subprocess.run([exe], capture_output=True, text=True, timeout=60)
    assert r.returncode == 0, r.stderr
    return [l.split() for l in r.stdout.splitlines()]


def test_the_consumer_is_short():
    assert len(open(os.path.join(ROOT, "tests", "csrc", "abi_consumer.c")).read().splitlines()) <= 40


def test_size_functions_from_c(report):
    import oracle

    rows = {int(l[1]): [int(x) for x in l[2:]] for l in report if l[0] == "sizes"}
    # n: onebit, tbq, terngrad(512), sparse capacity(0.001), sparse payload(0.001), min/max quantiser(b=2)
    want = {
        0: [16, 16, 16, 64, 528, 10],
        1: [16 + 4, 16 + 4, 16 + 16 + 4, 64, 528, 11],
        262144: [16 + 4 * 8192, 16 + 4 * 16384, 16 + 4 * 512 + 4 * 16384, 1088, 16 + 8 * 1088, 10 + 65536],
        102760448: [16 + 4 * 3211264, 16 + 4 * 6422528, 16 + 4 * 200704 + 4 * 6422528, 411072, 16 + 8 * 411072, 10 + 25690112],
    }
    assert rows == want
    for n, (ob, tbq, tg, cap, sp, cl) in rows.items():  # the oracle states the same formats on its own
        assert ob == oracle.onebit_payload_bytes(n) and tbq == oracle.tbq_payload_bytes(n)
        assert tg == oracle.terngrad_payload_bytes(n, 512) and sp == oracle.sparse_payload_bytes(n, 0.001)


def test_struct_layout_matches_what_ctypes_declares(report):
    from hipress_amd import _lib

    sizes = {l[1]: int(l[2]) for l in report if l[0] == "sizeof"}
    offsets = {l[1]: int(l[2]) for l in report if l[0] == "offset"}
    structs = {"hipress_tensor": _lib.Tensor, "hipress_params": _lib.Params, "hipress_merge_chunk": _lib.MergeChunk}
    assert set(sizes) == set(structs)
    seen = 0
    for cname, cls in structs.items():
        assert sizes[cname] == ctypes.sizeof(cls), cname
        for field, _ in cls._fields_:
            assert offsets[f"{cname}.{field}"] == getattr(cls, field).offset, (cname, field)
            seen += 1
    assert seen == len(offsets)  # every field the C side printed has a ctypes twin and the other way round


def test_argument_checks_from_c_need_no_gpu(report):
    got = {l[0]: l[1:] for l in report if l[0] in ("null_encode", "null_decode", "too_large", "strerror", "version")}
    assert got["null_encode"] == ["-1"] and got["null_decode"] == ["-1"]  # HIPRESS_ERR_NULL
    assert got["too_large"] == ["-2"]  # HIPRESS_ERR_SIZE
    assert " ".join(got["strerror"]) == "a required pointer is NULL"
    assert int(got["version"][0]) >= 100
