"""Generates HIP from every operator program under programs/ and builds
hipress_amd/libhipress_compll_gen.so for gfx950 (cross-compiles without a GPU).

Usage: python -m hipress_amd.compll.build
"""
import glob
import os
import subprocess
import sys

from . import compile_text

HERE = os.path.dirname(os.path.abspath(__file__))
PROGRAMS = os.path.join(HERE, "programs")
GENERATED = os.path.join(HERE, "_generated")
CSRC = os.path.join(os.path.dirname(HERE), "csrc")
LIB = os.path.join(os.path.dirname(HERE), "libhipress_compll_gen.so")
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wall", "-I", CSRC]


def programs():
    return sorted(glob.glob(os.path.join(PROGRAMS, "*.pse")))


def manifests():
    """name -> manifest entry of every operator of every shipped program."""
    out = {}
    for path in programs():
        with open(path) as f:
            for m in compile_text(f.read())[1]:
                out[m["name"]] = m
    return out


def build(verbose=False):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    os.makedirs(GENERATED, exist_ok=True)
    objs, procs = [], []
    for path in programs():
        stem = os.path.splitext(os.path.basename(path))[0]
        with open(path) as f:
            source, _ = compile_text(f.read())
        hip = os.path.join(GENERATED, stem + ".hip")
        with open(hip, "w") as f:
            f.write(source)
        obj = os.path.join(GENERATED, stem + ".o")
        cmd = [hipcc, *FLAGS, "-c", hip, "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((stem, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        objs.append(obj)
    failed = False
    for stem, p in procs:
        out, _ = p.communicate()
        out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l and l.strip())
        if p.returncode != 0:
            failed = True
            sys.stderr.write(f"--- {stem} failed ---\n{out}\n")
        elif out:
            sys.stderr.write(f"--- {stem} ---\n{out}\n")
    if failed:
        raise RuntimeError("hipcc failed on generated code")
    subprocess.check_call([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs])
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
