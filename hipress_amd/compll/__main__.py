"""python -m hipress_amd.compll program.pse [-o out.hip] [--manifest out.json]"""
import argparse
import json
import sys

from . import CompileError, compile_text


def main(argv=None):
    ap = argparse.ArgumentParser(description="CompLL operator language -> HIP for gfx950")
    ap.add_argument("program")
    ap.add_argument("-o", "--output", default=None, help="HIP source (default: stdout)")
    ap.add_argument("--manifest", default=None, help="write the operators' parameter lists as JSON")
    args = ap.parse_args(argv)
    try:
        with open(args.program) as f:
            source, manifest = compile_text(f.read())
    except CompileError as e:
        sys.stderr.write(f"{args.program}: {e}\n")
        return 1
    if args.output:
        with open(args.output, "w") as f:
            f.write(source)
    else:
        sys.stdout.write(source)
    if args.manifest:
        with open(args.manifest, "w") as f:
            json.dump(manifest, f, indent=1)
    return 0


if __name__ == "__main__":
    sys.exit(main())
