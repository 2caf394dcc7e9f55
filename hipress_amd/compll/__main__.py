"""python -m hipress_amd.compll program.pse [-o out.hip] [--manifest out.json] [--library out.so]

The counterpart of the reference's `python3 GCGen.py pse/X.pse -b`
(/root/reference/README.md:228-234): the operator program goes in, GPU code comes out.
-o writes the HIP source (default: stdout), --library also compiles it for gfx950 into a
shared library that hipress_amd.compll.runtime.Operators loads.  The reference's -b flag is
accepted (the body is what is generated here); its -w / -r / -f flags, which write framework
wrapper and registration files, have nothing to generate here: the library's entry points are
plain C and the Python binding is made at load time from the manifest."""
import argparse
import json
import sys

from . import CompileError, compile_text


def main(argv=None):
    ap = argparse.ArgumentParser(description="CompLL operator language -> HIP for gfx950")
    ap.add_argument("program")
    ap.add_argument("-o", "--output", default=None, help="HIP source (default: stdout, unless --library is given)")
    ap.add_argument("--manifest", default=None, help="write the operators' parameter lists as JSON")
    ap.add_argument("--library", default=None, metavar="OUT.so",
                    help="compile the generated source with hipcc into this shared library (+ OUT.so.json)")
    ap.add_argument("-b", "--body", action="store_true", help="accepted for familiarity: the body is always generated")
    ap.add_argument("-w", "--wrapper", action="store_true", help=argparse.SUPPRESS)
    ap.add_argument("-r", "--register", action="store_true", help=argparse.SUPPRESS)
    ap.add_argument("-f", "--framework", default=None, help=argparse.SUPPRESS)
    args = ap.parse_args(argv)
    if args.wrapper or args.register or args.framework:
        sys.stderr.write("no wrapper or registration files are generated: build the operators with --library OUT.so and "
                         "bind them with hipress_amd.compll.runtime.Operators('OUT.so')\n")
        return 2
    try:
        with open(args.program) as f:
            source, manifest = compile_text(f.read())
    except CompileError as e:
        sys.stderr.write(f"{args.program}: {e}\n")
        return 1
    if args.output:
        with open(args.output, "w") as f:
            f.write(source)
    elif not args.library:
        sys.stdout.write(source)
    if args.manifest:
        with open(args.manifest, "w") as f:
            json.dump(manifest, f, indent=1)
    if args.library:
        from .build import build_library

        try:
            print(build_library([args.program], args.library))
        except RuntimeError as e:
            sys.stderr.write(f"{args.program}: {e}\n")
            return 1
    return 0


if __name__ == "__main__":
    sys.exit(main())
