"""Variant builds for A/B measurements: `python -m hipress_amd.build --define ... --output x.so`
compiles the same sources with tuning constants of csrc/common.h overridden, leaves the in-tree
library alone, and HIPRESS_AMD_LIB makes the binding load the variant.  Host side only."""
import hashlib
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "hipress_amd", "libhipress_amd.so")


def _sha(path):
    return hashlib.sha256(open(path, "rb").read()).hexdigest()


def test_variant_build_exports_the_whole_abi_and_leaves_the_library_alone(tmp_path):
    before = _sha(LIB)
    out = str(tmp_path / "variant.so")
    r = subprocess.run([sys.executable, "-m", "hipress_amd.build", "--define", "HP_CACHE_TAIL_ONE_MIB=0", "--define",
                        "HP_CACHE_TAIL_MANY_MIB=0", "--define", "HP_SECOND_PASS_REVERSED=0", "--output", out],
                       cwd=ROOT, capture_output=True, text=True, timeout=900)
    assert r.returncode == 0, r.stderr[-2000:]
    assert os.path.exists(out) and _sha(LIB) == before
    assert _sha(out) != before  # the constants reach the kernels
    code = ("from hipress_amd import _lib; L = _lib.lib(); assert _lib.LIB_PATH == %r; "
            "assert all(hasattr(L, n) for n in _lib.SIGNATURES); print(L.hipress_version())" % out)
    r = subprocess.run([sys.executable, "-c", code], cwd=ROOT, env=dict(os.environ, HIPRESS_AMD_LIB=out),
                       capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr[-2000:]
    assert int(r.stdout.strip()) >= 100


def test_defines_without_an_output_path_are_refused():
    r = subprocess.run([sys.executable, "-m", "hipress_amd.build", "--define", "HP_CACHE_TAIL_ONE_MIB=0"], cwd=ROOT,
                       capture_output=True, text=True, timeout=60)
    assert r.returncode != 0 and "--output" in r.stderr
