"""Generates HIP from every operator program under programs/ and builds
hipress_amd/libhipress_compll_gen.so for gfx950 (cross-compiles without a GPU).

Usage: python -m hipress_amd.compll.build
A program of one's own: python -m hipress_amd.compll my.pse --library my_ops.so, then
hipress_amd.compll.runtime.Operators("my_ops.so").
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


def build_library(paths, output, workdir=None, verbose=False):
    """Generates HIP from the operator programs `paths`, compiles it for gfx950 and links
    `output` (a shared library with one C entry point per operator); the operators'
    parameter lists go to `output + ".json"`, which runtime.Operators reads to bind them."""
    import json

    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    output = os.path.abspath(output)
    workdir = workdir or output + ".build"
    os.makedirs(workdir, exist_ok=True)
    objs, procs, manifest = [], [], {}
    for path in paths:
        stem = os.path.splitext(os.path.basename(path))[0]
        with open(path) as f:
            source, man = compile_text(f.read())
        for m in man:
            if m["name"] in manifest:
                raise RuntimeError(f"operator {m['name']!r} is defined twice ({path})")
            manifest[m["name"]] = m
        hip = os.path.join(workdir, stem + ".hip")
        with open(hip, "w") as f:
            f.write(source)
        obj = os.path.join(workdir, stem + ".o")
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
    subprocess.check_call([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", output, *objs])
    with open(output + ".json", "w") as f:
        json.dump(manifest, f, indent=1)
    return output


def build(verbose=False):
    """The shipped programs -> hipress_amd/libhipress_compll_gen.so."""
    return build_library(programs(), LIB, workdir=GENERATED, verbose=verbose)


# The two programs the reference checkout ships for its own generator.  Where that checkout is
# present they are compiled as they are, read in place, into a library of their own (kept out
# of version control like every built file), so that a GPU test can run the operators a user of
# the reference would bring.
REFERENCE_PROGRAMS = "/root/reference/src/CompLL/GCGen/pse"
REFERENCE_LIB = os.path.join(GENERATED, "reference_programs", "libreference_programs.so")


def build_reference_programs(verbose=False):
    """-> the library's path, or None when the reference checkout is not on this machine."""
    paths = sorted(glob.glob(os.path.join(REFERENCE_PROGRAMS, "*.pse")))
    if not paths:
        return None
    os.makedirs(os.path.dirname(REFERENCE_LIB), exist_ok=True)
    return build_library(paths, REFERENCE_LIB, verbose=verbose)


if __name__ == "__main__":
    print(build(verbose=True))
    print(build_reference_programs(verbose=True) or "no reference checkout here: its programs are not built")
