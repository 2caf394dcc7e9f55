"""Builds hipress_amd/libhipress_amd.so for gfx950 with hipcc.

Usage: python -m hipress_amd.build   (cross-compiles without a GPU)
       python -m hipress_amd.build --define NAME=VALUE ... --output other.so
The second form builds a variant library with tuning constants of csrc/common.h overridden
(for A/B measurements: load it with the environment variable HIPRESS_AMD_LIB=other.so); its
objects go to a directory of their own next to the output, the in-tree library is untouched.
"""
import argparse
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libhipress_amd.so")
LATENCY_EXE = os.path.join(HERE, "hipress_latency")  # C-level latency probe (csrc/latency_main.cpp)
SOURCES = ["api.hip", "dense.hip", "sparse.hip", "merge.hip", "compll.hip"]
FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-ffp-contract=off",  # bit-exact residuals: a*b+c is never fused
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall",
    "-Wno-unused-function",
]


def build(verbose=False, defines=(), output=None):
    """Compiles the library (and, for the in-tree library, the C-level latency probe).
    defines: "NAME=VALUE" strings passed as -D; output: path of a variant library."""
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    lib = os.path.abspath(output) if output else LIB
    objdir = CSRC
    if output:
        objdir = lib + ".objs"
        os.makedirs(objdir, exist_ok=True)
    objs = []
    procs = []
    for src in SOURCES:
        obj = os.path.join(objdir, src.replace(".hip", ".o"))
        cmd = [hipcc, *FLAGS, *["-D" + d for d in defines], "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        objs.append(obj)
    failed = False
    for src, p in procs:
        out, _ = p.communicate()
        out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l and l.strip())
        if p.returncode != 0:
            failed = True
            sys.stderr.write(f"--- {src} failed ---\n{out}\n")
        elif verbose and out:
            print(out)
    if failed:
        raise RuntimeError("hipcc failed")
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", lib, *objs]
    subprocess.check_call(cmd)
    if output:
        return lib
    # a plain C++ program over the C ABI; no device code of its own
    subprocess.check_call([hipcc, "--offload-arch=gfx950", "-O2", "-std=c++17", os.path.join(CSRC, "latency_main.cpp"), "-o", LATENCY_EXE,
                           "-L" + HERE, "-lhipress_amd", "-Wl,-rpath,$ORIGIN"])
    return LIB


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--define", action="append", default=[], metavar="NAME=VALUE")
    ap.add_argument("--output", default=None, help="write a variant library here instead of the in-tree one")
    a = ap.parse_args()
    if a.define and not a.output:
        ap.error("--define needs --output: the in-tree library is always built with the defaults")
    print(build(verbose=True, defines=a.define, output=a.output))
