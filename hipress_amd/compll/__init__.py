"""CompLL operator language -> HIP for gfx950.

    from hipress_amd import compll
    source, manifest = compll.compile_text(open("op.pse").read())

`python -m hipress_amd.compll prog.pse -o prog.hip` does the same from the shell.
"""
from . import backend, frontend
from .frontend import CompileError, parse


def compile_text(text):
    """-> (HIP source, manifest) for every operator of the program."""
    return backend.generate(parse(text))


__all__ = ["CompileError", "parse", "compile_text"]
