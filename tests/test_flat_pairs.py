"""The 64-bit flat pair positions of the sparse merge (hipress_amd/csrc/flat_pairs.h), checked on
the host: the header is plain C++, so the very lines the kernel runs are compiled with g++ and
exercised with pair counts no GPU test could allocate (sixteen peers of 2^31 - 1 pairs)."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_flat_pair_positions_beyond_32_bits(tmp_path):
    exe = str(tmp_path / "flat_pairs_check")
    subprocess.check_call(["g++", "-std=c++17", "-O1", "-Wall", "-Werror", "-I", os.path.join(ROOT, "hipress_amd", "csrc"),
                           os.path.join(ROOT, "tests", "csrc", "flat_pairs_check.cpp"), "-o", exe])
    r = subprocess.run([exe], capture_output=True, text=True)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "flat pair positions ok" in r.stdout


def test_the_merge_kernel_uses_the_checked_header():
    src = open(os.path.join(ROOT, "hipress_amd", "csrc", "sparse.hip")).read()
    assert '#include "flat_pairs.h"' in src
    assert src.count("flat_advance(pcnt") == 3 and "flat_total(pcnt" in src
