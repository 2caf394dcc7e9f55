"""The CompLL operator language front end and back end (hipress_amd/compll), on the CPU:
tokens, syntax tree, the host/device classification of scalars, the launch plan and
the error messages.  The generated library is only checked for its symbols here."""
import ctypes
import os

import pytest

from hipress_amd import compll
from hipress_amd.compll import backend, frontend as F
from hipress_amd.compll.build import LIB, manifests, programs


def test_tokens_and_comments():
    toks = F.tokenize("a<<2 // note\n /* block\n */ x -> uint<b>* [&] 1.5e-3 >= 7")
    assert [t.text for t in toks[:-1]] == ["a", "<<", "2", "x", "->", "uint", "<", "b", ">", "*", "[&]", "1.5e-3", ">=", "7"]
    assert toks[3].line == 3 and toks[11].kind == "float" and toks[13].kind == "int"
    with pytest.raises(F.CompileError, match="line 2"):
        F.tokenize("ok\n $")


def test_precedence_and_tree():
    prog = F.parse("void f(float* v, uint8* out, uint8 b){ int k = 1 + 2 * 3 << 1; uint8 t = v.size % (1<<b); }")
    fn = prog.functions[0]
    assert [p.name for p in fn.params] == ["v", "out", "b"] and fn.params[0].type.pointer
    k = fn.body[0].value  # ((1 + (2*3)) << 1)
    assert isinstance(k, F.Binary) and k.op == "<<" and k.lhs.op == "+" and k.lhs.rhs.op == "*"
    t = fn.body[1].value
    assert t.op == "%" and isinstance(t.lhs, F.SizeOf) and t.rhs.op == "<<"


def test_uint_width_expression_stops_at_the_closing_bracket():
    prog = F.parse("void f(float* v, uint8* out, uint8 b){ lambda_func q = [&](int i) -> uint<b+1> { return i > 3; } }")
    lam = prog.functions[0].body[0]
    assert isinstance(lam, F.Lambda) and lam.ret.base == "uint" and lam.ret.bits.op == "+"
    assert lam.body[0].value.op == ">"


def test_param_block_is_accepted():
    prog = F.parse("param P { uint8 bitwidth; } void f(float* v, uint8* o){ }")
    assert prog.param_blocks["P"][0].name == "bitwidth"


PROGRAM = """
void Enc(float* g, uint8* out, uint8 b) {
    lambda_func hi = [&](float x, float y) -> float { if (x > y) { return x; } return y; }
    lambda_func lo = [&](float x, float y) -> float { if (x < y) { return x; } return y; }
    float top = reduce(g, -1, hi);
    float bottom = reduce(g, 1, lo);
    float step = (top - bottom) / ((1 << b) - 1);
    uint8 rest = g.size % (1 << b);
    lambda_func q = [&](int i) -> uint<b> { return floor((g[i] - bottom) / step + random<float>(0, 1)); }
    uint<b>* codes = map(range(g.size), q);
    out = concat(b, rest, bottom, top, codes);
}
"""


def test_plan_classifies_scalars_and_fuses_reductions():
    g = backend.FunctionGen(F.parse(PROGRAM).functions[0])
    cls = {n: s.cls for n, s in g.scalars.items()}
    assert cls == {"b": "host", "top": "dev", "bottom": "dev", "step": "dev", "rest": "host"}
    # both folds in one sweep; the scalars and header fields that follow are computed by the
    # reduce's last kernel, so the operator is two sweeps and no launch of one thread
    assert g.launch_kinds() == ["reduce", "map_packed"]
    assert [s.kind for s in g.stages] == ["reduce", "serial", "map_packed"]
    assert len(g.stages[0].folds) == 2 and g.needs_uniform
    src, man = compll.compile_text(PROGRAM)
    assert 'extern "C" int Enc(float* g, int32_t g_size, uint8_t* out, int32_t out_size, uint8_t b, const float* uniform, ' \
           "uint64_t seed, void* workspace, int64_t workspace_bytes, void* stream)" in src  # uniform NULL: drawn from seed
    assert "cl::put<float>(a.v_out + 2, (float)d.v_bottom);" in src  # header offsets 0, 1, 2, 6; codes behind byte 10
    assert "(a.v_out + 10)" in src
    assert man[0]["params"] == [{"name": "g", "kind": "float*"}, {"name": "out", "kind": "uint8*"}, {"name": "b", "kind": "uint8"}]


@pytest.mark.parametrize("body,message", [
    ("float m = reduce(g, 0, nothing);", "unknown lambda"),
    ("uint<2>* c = map(range(g.size), f); ", "never stored"),
    ("b = 3;", "cannot be assigned"),
    ("float r = random<float>(0, 1);", "inside a lambda"),
    ("float x = y + 1;", "unknown scalar"),
    ("float x; float z = x * 2;", "before it has a value"),
    ("out = concat(c, b);", "unknown"),
    ("lambda_func h = [&](float x) -> float { return x; } float m = reduce(g, 0, h);", r"\(float, float\) -> float"),
    ("float s = 1.5 << 2;", "needs integers"),
    ("float* w; ", "defined by map"),
    ("lambda_func m = [&](int i) -> float { return g[i]; } float* w = map(range(g.size), m); w = map(range(g.size), m);", "defined once"),
])
def test_errors_name_the_problem(body, message):
    text = "void Op(float* g, uint8* out, uint8 b) { lambda_func f = [&](int i) -> uint<2> { return i; } " + body + " }"
    with pytest.raises(F.CompileError, match=message):
        compll.compile_text(text)


def test_syntax_errors_carry_the_line():
    with pytest.raises(F.CompileError, match="line 3"):
        F.parse("void f(float* g, uint8* o) {\n float x = 1;\n float = 2;\n}")
    with pytest.raises(F.CompileError, match="no function"):
        F.parse("// nothing here")


def test_shipped_programs_compile_and_the_library_exports_them():
    assert programs(), "no operator programs shipped"
    man = manifests()
    assert {"MinMaxQuantEncode", "MinMaxQuantDecode", "ThresholdTernaryEncode", "ThresholdTernaryDecode",
            "MeanAndSpread", "SignMeanEncode", "SignMeanDecode", "ThresholdFeedbackEncode"} <= set(man)
    assert man["ThresholdFeedbackEncode"]["launches"] == ["map_fused"]  # codes and residual in one sweep
    assert man["MinMaxQuantEncode"]["launches"] == ["reduce", "map_packed"]
    assert man["MinMaxQuantDecode"]["launches"] == ["map_float"]  # the header is read at the start of the sweep
    assert man["MeanAndSpread"]["launches"] == ["reduce"]  # three folds, one sweep
    assert man["SignMeanEncode"]["launches"] == ["reduce", "map_packed"]  # the mapped magnitudes are folded, never stored
    assert os.path.exists(LIB), "generated library not built: python -m hipress_amd.compll.build"
    lib = ctypes.CDLL(LIB)
    for name in man:
        assert hasattr(lib, name) and hasattr(lib, name + "_workspace_bytes")
    ws = lib.MinMaxQuantEncode_workspace_bytes
    ws.argtypes, ws.restype = [ctypes.c_int64], ctypes.c_int64
    assert ws(0) >= 256 and ws(1 << 20) >= 256 + 4 * 2 * 256 and ws(-1) < 0


def test_command_line_writes_source_and_manifest(tmp_path):
    import json
    import subprocess
    import sys

    prog = tmp_path / "op.pse"
    prog.write_text(PROGRAM)
    out, man = tmp_path / "op.hip", tmp_path / "op.json"
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, "-m", "hipress_amd.compll", str(prog), "-o", str(out), "--manifest", str(man)],
                       cwd=root, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    assert 'extern "C" int Enc(' in out.read_text()
    assert json.loads(man.read_text())[0]["name"] == "Enc"
    prog.write_text("void Broken(float* g, uint8* o) {\n float x = ;\n}")
    r = subprocess.run([sys.executable, "-m", "hipress_amd.compll", str(prog)], cwd=root, capture_output=True, text=True)
    assert r.returncode == 1 and "line 2" in r.stderr


def test_lambda_bodies_translate_control_flow_and_helpers():
    text = """
void Op(float* g, uint8* out, float t) {
    lambda_func clip = [&](float x) -> float { if (x > t) { return t; } else if (x < -t) { return -t; } return x; }
    lambda_func level = [&](int i) -> uint<4> {
        float v = clip(g[i]) / t;
        int q = 0;
        if (v >= 0.5) { q = 15; } else { q = 7; }
        return q;
    }
    uint<4>* codes = map(range(g.size), level);
    out = concat(t, codes);
}
"""
    src, man = compll.compile_text(text)
    assert "fn_clip(a, d, s[0])" in src          # g[i] arrives as a streamed operand; the helper is an ordinary call
    assert "} else {" in src and "q = 15;" in src
    assert man[0]["launches"] == ["map_packed"]


def test_a_block_that_reads_its_own_output_keeps_its_launch():
    text = """
void Op(uint8* packed, float* g) {
    float k;
    uint<2>* codes;
    extract(packed, k, codes);
    k = k * 2;
    lambda_func f = [&](int i) -> float { return codes[i] * k; }
    g = map(range(g.size), f);
}
"""
    _, man = compll.compile_text(text)
    assert man[0]["launches"] == ["serial", "map_float"]  # k = k * 2 must run exactly once


FEEDBACK = """
void Op(float* g, float* r, uint8* out, float t) {
    lambda_func level = [&](int i) -> uint<2> { return r[%s] + g[i] >= t; }
    lambda_func carry = [&](int i) -> float { return r[i] + g[i]; }
    uint<2>* codes = map(range(g.size), level);
    %s
}
"""


def test_maps_share_a_sweep_only_when_that_is_what_the_program_says():
    stored_first = "out = concat(t, codes); r = map(range(g.size), carry);"
    assert compll.compile_text(FEEDBACK % ("i", stored_first))[1][0]["launches"] == ["map_fused"]
    # the codes read a neighbour of the element being rewritten: two sweeps, in program order
    assert compll.compile_text(FEEDBACK % ("i + 1", stored_first))[1][0]["launches"] == ["serial", "map_packed", "map_float"]
    # the residual may not change between the map that reads it and the concat that runs it
    with pytest.raises(F.CompileError, match="changes before the codes"):
        compll.compile_text(FEEDBACK % ("i", "r = map(range(g.size), carry); out = concat(t, codes);"))
    with pytest.raises(F.CompileError, match="only once"):
        compll.compile_text("void Op(float* g, uint8* o, uint8 b) { int k = b + 1; k = 2; }")


REFERENCE_PSE = "/root/reference/src/CompLL/GCGen/pse"


@pytest.mark.skipif(not os.path.isdir(REFERENCE_PSE), reason="the reference checkout is not on this machine")
def test_the_reference_checkout_s_own_programs_compile_unmodified(tmp_path):
    """A user of the reference's generator brings programs written for it.  The two it ships
    (TernGradEncode.pse, TernGradDecode.pse: read here where they lie, never copied) go through
    this compiler as they are - commented-out `param` block, `else` branches, `uint<bitwidth>`,
    `concat` / `extract`, `.size`, `random<float>` - give the same launch plan as the restated
    program the GPU tests run, and the HIP they turn into compiles for gfx950."""
    import subprocess

    from hipress_amd import build as hb

    plans = {}
    for name in ("TernGradEncode", "TernGradDecode"):
        text = open(os.path.join(REFERENCE_PSE, name + ".pse")).read()
        source, manifest = compll.compile_text(text)
        assert [m["name"] for m in manifest] == [name]
        plans[name] = manifest[0]
        assert f'extern "C" int {name}(' in source and f'extern "C" int64_t {name}_workspace_bytes(' in source
        src = tmp_path / (name + ".hip")
        src.write_text(source)
        r = subprocess.run([os.environ.get("HIPCC", "/opt/rocm/bin/hipcc"), *hb.FLAGS, "-I", os.path.join(os.path.dirname(hb.CSRC), "csrc"),
                            "--cuda-device-only", "-c", str(src), "-o", os.devnull], capture_output=True, text=True, timeout=600)
        assert r.returncode == 0, r.stderr[-3000:]
    ours = manifests()
    assert plans["TernGradEncode"]["launches"] == ours["MinMaxQuantEncode"]["launches"] == ["reduce", "map_packed"]
    assert plans["TernGradDecode"]["launches"] == ours["MinMaxQuantDecode"]["launches"] == ["map_float"]
    # same operator surface as the reference registers: (gradient, compressed, bitwidth) / (compressed, gradient)
    assert [p["name"] for p in plans["TernGradEncode"]["params"]][:3] == ["gradient", "compressed", "bitwidth"]
    assert [p["name"] for p in plans["TernGradDecode"]["params"]][:2] == ["compressed", "gradient"]


def test_a_program_of_one_s_own_becomes_a_loadable_library(tmp_path):
    """The whole way a user of the reference's generator goes: program in, library out
    (`python -m hipress_amd.compll prog.pse -b --library ops.so`), operators bound from the
    manifest the build leaves beside it.  No GPU call is made."""
    import json
    import subprocess
    import sys

    from hipress_amd.compll import runtime

    prog = tmp_path / "clip.pse"
    prog.write_text("""
void ClipScale(float* gradient, float* clipped, float bound) {
    lambda_func keep = [&](int index) -> float {
        float a = gradient[index];
        if (a > bound) { return bound; }
        if (a < 0 - bound) { return 0 - bound; }
        return a;
    }
    clipped = map(range(gradient.size), keep);
}
""")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    lib = tmp_path / "clip_ops.so"
    r = subprocess.run([sys.executable, "-m", "hipress_amd.compll", str(prog), "-b", "--library", str(lib)], cwd=root,
                       capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-3000:]
    assert lib.exists() and json.loads((tmp_path / "clip_ops.so.json").read_text())["ClipScale"]["launches"] == ["map_float"]
    ops = runtime.Operators(str(lib))
    assert callable(ops.ClipScale) and [p["name"] for p in ops.manifest["ClipScale"]["params"]] == ["gradient", "clipped", "bound"]
    with pytest.raises(TypeError):
        ops.ClipScale(1, 2, 3, 4)  # argument checks come before anything touches a GPU
    # the reference's wrapper / registration flags have nothing to generate here and say so
    r = subprocess.run([sys.executable, "-m", "hipress_amd.compll", str(prog), "-w", "-r", "-f", "mxnet"], cwd=root,
                       capture_output=True, text=True)
    assert r.returncode == 2 and "Operators" in r.stderr
