"""Back end for the CompLL operator language: syntax tree -> HIP source for gfx950.

Where the reference's generator turns every primitive into a Thrust call on whole
vectors, with host round trips for each scalar in between
(/root/reference/src/CompLL/GCGen/unit.py:217-403 for the emitted operator,
/root/reference/src/CompLL/GCGen/output/TernGradEncode/TernGradEncode_body.h:99-126
for what it looks like), this one plans a short sequence of launches over the
primitive kernels of hipress_amd/csrc/compll_prims.h:

* every scalar is classified as host-known (function of the arguments and sizes)
  or device-known (function of a reduce result or an extracted header field);
  host-known ones are evaluated in the entry function and travel in `Args`,
  device-known ones are evaluated by a one-thread kernel and stay in `Dev`;
* neighbouring `reduce` statements over the same vector share one sweep;
* a packed vector that only feeds `concat` is produced in place behind the header;
* `random<float>(lo, hi)` reads an explicit uniform[0,1) input tensor, or, when the caller passes
  NULL for it, is drawn in the kernel from the caller's seed and the element's index.

The emitted entry point mirrors the reference's body signature (vectors in the
order of declaration, each followed by its length, then the scalar parameters),
followed by the uniform tensor if the operator draws random numbers, a workspace
and the stream; it returns 0 or one of the negative codes of include/hipress_amd.h.
"""
from dataclasses import dataclass, field
from typing import Dict, List, Optional

from . import frontend as F
from .frontend import CompileError

_SCALAR_C = {"float": "float", "int": "int", "int32": "int", "uint8": "uint8_t", "uint16": "uint16_t", "uint32": "uint32_t"}
_SCALAR_BYTES = {"float": 4, "int": 4, "int32": 4, "uint8": 1, "uint16": 2, "uint32": 4}
_CALLS = {"floor": "floorf", "ceil": "ceilf", "abs": "fabsf", "fabs": "fabsf", "sqrt": "sqrtf", "exp": "expf", "log": "logf"}


def _rerunnable(lines) -> bool:
    """Whether a block of serial statements gives the same result when it is run again on
    its own output (no statement reads a device scalar that the block assigns at or after
    that statement): such a block may be run by every workgroup of the sweep that follows."""
    import re

    targets = [re.match(r"d\.v_(\w+) = ", ln) for ln in lines]
    names = [m.group(1) if m else None for m in targets]
    for i, ln in enumerate(lines):
        rhs = ln[targets[i].end():] if targets[i] else ln
        later = {n for n in names[i:] if n}
        if any(re.search(r"\bd\.v_%s\b" % re.escape(n), rhs) for n in later):
            return False
    return True


def _local(name: str) -> str:
    """A lambda's parameter or local variable as it is spelt in the generated source: prefixed,
    so that a program's own names (`a`, `d`, `s`, `i` ...) never meet the generator's."""
    return "l_" + name


def _unparen(code: str) -> str:
    """Drops one pair of parentheses that encloses the whole expression."""
    if code.startswith("(") and code.endswith(")"):
        depth = 0
        for k, ch in enumerate(code):
            depth += ch == "("
            depth -= ch == ")"
            if depth == 0 and k != len(code) - 1:
                return code
        return code[1:-1]
    return code


@dataclass
class Scalar:
    name: str
    base: str                  # key of _SCALAR_C; "uint" scalars are stored as uint32
    cls: Optional[str] = None  # "host" | "dev"; None until first assigned
    is_param: bool = False

    @property
    def ctype(self):
        return _SCALAR_C.get(self.base, "uint32_t")

    def ref(self):
        return f"{'a' if self.cls == 'host' else 'd'}.v_{self.name}"


@dataclass
class Vector:
    name: str
    elem: str                    # "float" | "bytes" | "packed"
    is_param: bool = False
    ptr: Optional[str] = None    # C expression of the base pointer (None: not placed yet)
    size: Optional[str] = None   # C expression of the element count
    size_cls: str = "host"
    bits: Optional[str] = None   # packed: C expression of the code width
    bits_cls: str = "host"
    pending_map: Optional[tuple] = None  # packed vector defined by map, waiting for its place: (count, lambda)
    bits_ast: Optional[F.Expr] = None    # code width not resolvable at the declaration (it is extracted later)
    virtual: Optional[tuple] = None      # float vector that is a map never stored: (count Value, lambda name)


@dataclass
class Value:
    code: str
    kind: str  # "float" | "int"
    cls: str   # "host" | "dev"


@dataclass
class Stage:
    kind: str  # serial | reduce | map_float | map_packed
    lines: List[str] = field(default_factory=list)
    vec: Optional[Vector] = None
    folds: List[tuple] = field(default_factory=list)  # (target scalar, init code, lambda name)
    fn: str = ""
    count: Optional[Value] = None
    bound: str = ""       # host expression bounding the launch
    dest: str = ""
    cap: str = ""
    bits: Optional[Value] = None
    float_map: Optional["Stage"] = None  # map_fused: the float map that shares the sweep of this packed map


class FunctionGen:
    def __init__(self, fn: F.Function):
        self.fn = fn
        self.ns = f"gen_{fn.name}"
        self.scalars: Dict[str, Scalar] = {}
        self.vectors: Dict[str, Vector] = {}
        self.lambdas: Dict[str, F.Lambda] = {}
        self.lambda_code: Dict[str, str] = {}
        self.lambda_order: List[str] = []
        self.host_lines: List[str] = []
        self.checks: List[str] = []
        self.stages: List[Stage] = []
        self.needs_uniform = False
        self.streams = None        # while a mapped lambda is compiled: pointer expressions it reads at its own index
        self.map_streams: Dict[str, list] = {}
        self.struct_id = 0
        self.max_folds = 0
        self.reduced: List[Vector] = []
        self._declare_params()
        for st in fn.body:
            self.statement(st)
        for v in self.vectors.values():
            if v.pending_map:
                raise CompileError(f"packed vector {v.name!r} is computed but never stored with concat", fn.line)
        self._fuse_maps()

    def _fuse_maps(self):
        """A packed map directly followed by a float map over the same range becomes one
        sweep when element i of either result depends on the vector being written only
        through element i (so computing both from the values loaded first is what running
        them one after the other would give)."""
        k = 0
        while k + 1 < len(self.stages):
            p, f = self.stages[k], self.stages[k + 1]
            if p.kind == "map_packed" and f.kind == "map_float" and p.count.code == f.count.code and p.count.cls == "host":
                written = f.vec.name
                ok = True
                for fn in (p.fn, f.fn):
                    _, vectors, elsewhere = self.uses(fn)
                    if written in elsewhere:
                        ok = False
                _, fvec, _ = self.uses(f.fn)
                if p.vec.name in fvec:  # the float map reads the codes themselves
                    ok = False
                if ok:
                    p.kind, p.float_map = "map_fused", f
                    del self.stages[k + 1]
                    self.checks.append(f"if ((long long)({p.count.code}) > (long long){f.vec.size}) return -2;")
            k += 1

    # ---------------------------------------------------------------- symbols
    def _declare_params(self):
        for p in self.fn.params:
            t = p.type
            if t.pointer:
                if t.base == "float":
                    v = Vector(p.name, "float", True)
                elif t.base == "uint8":
                    v = Vector(p.name, "bytes", True)
                else:
                    raise CompileError(f"vector parameter {p.name!r} must be float* or uint8*", t.line)
                v.ptr, v.size = f"a.v_{p.name}", f"a.v_{p.name}_size"
                self.vectors[p.name] = v
            else:
                if t.base not in _SCALAR_C:
                    raise CompileError(f"scalar parameter {p.name!r} has unsupported type {t.base}", t.line)
                self.scalars[p.name] = Scalar(p.name, t.base, "host", True)

    def scalar(self, name, line) -> Scalar:
        if name not in self.scalars:
            raise CompileError(f"unknown scalar {name!r}", line)
        return self.scalars[name]

    def vector(self, name, line) -> Vector:
        if name not in self.vectors:
            raise CompileError(f"unknown vector {name!r}", line)
        return self.vectors[name]

    # ---------------------------------------------------------------- expressions
    def expr(self, e: F.Expr, scope: Optional[dict] = None, index_name: Optional[str] = None) -> Value:
        """scope: names local to a lambda -> kind.  index_name: the element index of a map lambda."""
        scope = scope or {}
        if isinstance(e, F.Num):
            if e.is_float:
                return Value(e.text + "f", "float", "host")
            return Value(e.text, "int", "host")
        if isinstance(e, F.Name):
            if e.id in scope:
                return Value(_local(e.id), scope[e.id], "host")
            s = self.scalar(e.id, e.line)
            if s.cls is None:
                raise CompileError(f"{e.id!r} is used before it has a value", e.line)
            return Value(s.ref(), "float" if s.base == "float" else "int", s.cls)
        if isinstance(e, F.Unary):
            v = self.expr(e.arg, scope, index_name)
            return Value(f"({e.op}{v.code})", "int" if e.op == "!" else v.kind, v.cls)
        if isinstance(e, F.Binary):
            l, r = self.expr(e.lhs, scope, index_name), self.expr(e.rhs, scope, index_name)
            cls = "dev" if "dev" in (l.cls, r.cls) else "host"
            if e.op in ("<<", ">>", "%", "&", "|", "^"):
                if "float" in (l.kind, r.kind):
                    raise CompileError(f"operator {e.op} needs integers", e.line)
                return Value(f"({l.code} {e.op} {r.code})", "int", cls)
            if e.op in ("==", "!=", "<", ">", "<=", ">=", "&&", "||"):
                return Value(f"({l.code} {e.op} {r.code})", "int", cls)
            kind = "float" if "float" in (l.kind, r.kind) else "int"
            return Value(f"({l.code} {e.op} {r.code})", kind, cls)
        if isinstance(e, F.SizeOf):
            v = self.vector(e.vec, e.line)
            if v.size is None:
                raise CompileError(f"{e.vec}.size is not known here", e.line)
            return Value(f"({v.size})", "int", v.size_cls)
        if isinstance(e, F.Index):
            v = self.vector(e.vec, e.line)
            if v.virtual:  # an element of a mapped vector that is never stored is a call of its lambda
                i = self.expr(e.index, scope, index_name)
                if i.kind != "int":
                    raise CompileError("a vector index must be an integer", e.line)
                self.compile_lambda(v.virtual[1])
                return Value(f"fn_{v.virtual[1]}(a, d, {i.code})", "float", "dev")
            if v.ptr is None:
                raise CompileError(f"vector {e.vec!r} has no storage yet (it is waiting for concat)", e.line)
            i = self.expr(e.index, scope, index_name)
            if i.kind != "int":
                raise CompileError("a vector index must be an integer", e.line)
            if v.elem == "float":
                if self.streams is not None and isinstance(e.index, F.Name) and e.index.id == index_name:
                    return Value(f"s[{self._stream(v.ptr)}]", "float", "dev")
                return Value(f"{v.ptr}[{i.code}]", "float", "dev")
            if v.elem == "bytes":
                return Value(f"(int){v.ptr}[{i.code}]", "int", "dev")
            return Value(f"cl::get_code({v.ptr}, {i.code}, (int)({v.bits}))", "int", "dev")
        if isinstance(e, F.Random):
            if index_name is None:
                raise CompileError("random<...>() may only be drawn inside a lambda that is mapped over a range", e.line)
            if e.type.base != "float":
                raise CompileError("only random<float> is supported", e.line)
            lo, hi = self.expr(e.lo, scope, index_name), self.expr(e.hi, scope, index_name)
            self.needs_uniform = True
            if self.streams is not None:
                return Value(f"cl::uniform_from(s[{self._stream('a.uniform')}], (float)({lo.code}), (float)({hi.code}))", "float", "dev")
            return Value(f"cl::uniform_draw(a.uniform, a.ukey, {_local(index_name)}, (float)({lo.code}), (float)({hi.code}))", "float", "dev")
        if isinstance(e, F.Call):
            args = [self.expr(x, scope, index_name) for x in e.args]
            cls = "dev" if any(x.cls == "dev" for x in args) else "host"
            if e.fn in _CALLS:
                if len(args) != 1:
                    raise CompileError(f"{e.fn} takes one argument", e.line)
                return Value(f"{_CALLS[e.fn]}((float)({args[0].code}))", "float", cls)
            if e.fn in self.lambdas:
                lam = self.lambdas[e.fn]
                self.compile_lambda(e.fn)
                if len(args) != len(lam.params):
                    raise CompileError(f"{e.fn} takes {len(lam.params)} argument(s)", e.line)
                return Value(f"fn_{e.fn}(a, d, {', '.join(x.code for x in args)})", self.lambda_kind(lam), "dev")
            raise CompileError(f"unknown function {e.fn!r}", e.line)
        raise CompileError("expression not allowed here", getattr(e, "line", None))

    # ---------------------------------------------------------------- lambdas
    def lambda_kind(self, lam: F.Lambda) -> str:
        if lam.ret.base == "float":
            return "float"
        if lam.ret.base != "uint":
            return "int"
        # uint<bits>: the raw value is converted (saturating) where it is packed
        for st in self._returns(lam.body):
            scope = self._lambda_scope(lam)
            self._collect_locals(lam.body, scope)
            return self.expr(st.value, scope, lam.params[0].name if lam.params else None).kind
        raise CompileError(f"lambda {lam.name!r} returns nothing", lam.line)

    def _returns(self, body):
        for st in body:
            if isinstance(st, F.Return):
                yield st
            elif isinstance(st, F.If):
                yield from self._returns(st.then)
                yield from self._returns(st.otherwise)

    @staticmethod
    def _kind_of(t: F.Type) -> str:
        return "float" if t.base == "float" else "int"

    def _lambda_scope(self, lam):
        return {p.name: self._kind_of(p.type) for p in lam.params}

    def _collect_locals(self, body, scope):
        for st in body:
            if isinstance(st, F.Declare):
                scope[st.name] = self._kind_of(st.type)
            elif isinstance(st, F.If):
                self._collect_locals(st.then, scope)
                self._collect_locals(st.otherwise, scope)

    def compile_lambda(self, name: str):
        if name in self.lambda_code:
            return
        lam = self.lambdas[name]
        for p in lam.params:
            if p.type.pointer:
                raise CompileError(f"lambda {name!r}: vector parameters are not supported", lam.line)
        self.lambda_code[name] = ""  # guards against recursion
        kind = self.lambda_kind(lam)
        ret = {"float": "float", "int": "long long"}[kind]
        index_name = lam.params[0].name if len(lam.params) == 1 and self._kind_of(lam.params[0].type) == "int" else None
        params = ", ".join(("float " if self._kind_of(p.type) == "float" else "long long ") + _local(p.name) for p in lam.params)
        scope = self._lambda_scope(lam)
        lines = [f"static __device__ __forceinline__ {ret} fn_{name}(const Args& a, const Dev& d, {params}) {{"]
        lines += self.lambda_body(lam.body, scope, index_name, ret, 1)
        lines.append(f"    return ({ret})0;")
        lines.append("}")
        self.lambda_code[name] = "\n".join(lines)
        self.lambda_order.append(name)

    def uses(self, name: str, _seen=None):
        """What a lambda reads from the operator's scope, found on the syntax tree:
        (scalars, vectors, vectors read anywhere but at the lambda's own index).  Helpers it
        calls and mapped vectors it indexes are followed; what they read counts as read at
        other indices."""
        _seen = _seen or set()
        if name in _seen:
            return set(), set(), set()
        _seen = _seen | {name}
        lam = self.lambdas[name]
        local = {p.name for p in lam.params}
        own = lam.params[0].name if len(lam.params) == 1 and self._kind_of(lam.params[0].type) == "int" else None
        if own and self._assigns(lam.body, own):
            own = None
        scalars, vectors, elsewhere = set(), set(), set()

        def follow(fn):
            s2, v2, _ = self.uses(fn, _seen)
            scalars.update(s2)
            vectors.update(v2)
            elsewhere.update(v2)

        def ex(e):
            if isinstance(e, F.Name):
                if e.id not in local:
                    scalars.add(e.id)
            elif isinstance(e, F.Unary):
                ex(e.arg)
            elif isinstance(e, F.Binary):
                ex(e.lhs)
                ex(e.rhs)
            elif isinstance(e, F.Index):
                ex(e.index)
                vec = self.vectors.get(e.vec)
                if vec is not None and vec.virtual:
                    follow(vec.virtual[1])
                else:
                    vectors.add(e.vec)
                    if not (own and isinstance(e.index, F.Name) and e.index.id == own):
                        elsewhere.add(e.vec)
            elif isinstance(e, F.Call):
                for x in e.args:
                    ex(x)
                if e.fn in self.lambdas:
                    follow(e.fn)
            elif isinstance(e, F.Random):
                ex(e.lo)
                ex(e.hi)

        def body(stmts):
            for st in stmts:
                if isinstance(st, F.Declare):
                    if st.value is not None:
                        ex(st.value)
                    local.add(st.name)
                elif isinstance(st, F.Assign):
                    ex(st.value)
                elif isinstance(st, F.If):
                    ex(st.cond)
                    body(st.then)
                    body(st.otherwise)
                elif isinstance(st, F.Return):
                    ex(st.value)

        body(lam.body)
        return scalars, vectors, elsewhere

    def _guard_pending(self, line, scalar=None, vector=None):
        """A packed vector computed by map is produced where concat places it.  Nothing its
        lambda reads may change in between, or the codes would be computed from the new values."""
        for v in self.vectors.values():
            if not v.pending_map:
                continue
            scalars, vectors, _ = self.uses(v.pending_map[1])
            if (scalar and scalar in scalars) or (vector and vector in vectors):
                what = scalar or vector
                raise CompileError(f"{what!r} changes before the codes {v.name!r} computed from it are stored; "
                                   f"put the concat of {v.name!r} first", line)

    def _stream(self, ptr: str) -> int:
        if ptr not in self.streams:
            self.streams.append(ptr)
        return self.streams.index(ptr)

    def _assigns(self, body, name) -> bool:
        for st in body:
            if isinstance(st, F.Assign) and st.name == name:
                return True
            if isinstance(st, F.If) and (self._assigns(st.then, name) or self._assigns(st.otherwise, name)):
                return True
        return False

    def compile_map_lambda(self, name: str):
        """The lambda as the function of a map over a range: float vectors it reads at its
        own index (and its random draws) arrive as values the kernel has loaded as whole
        rows, instead of being indexed element by element."""
        if name in self.map_streams:
            return
        lam = self.lambdas[name]
        kind = self.lambda_kind(lam)
        ret = {"float": "float", "int": "long long"}[kind]
        index_name = lam.params[0].name
        self.streams = None if self._assigns(lam.body, index_name) else []
        lines = [f"static __device__ __forceinline__ {ret} mfn_{name}(const Args& a, const Dev& d, long long {_local(index_name)}, const float* s) {{"]
        lines += self.lambda_body(lam.body, self._lambda_scope(lam), index_name, ret, 1)
        lines.append(f"    return ({ret})0;")
        lines.append("}")
        self.map_streams[name] = self.streams or []
        self.streams = None
        self.lambda_code["map:" + name] = "\n".join(lines)
        self.lambda_order.append("map:" + name)

    def lambda_body(self, body, scope, index_name, ret, depth):
        pad = "    " * depth
        out = []
        for st in body:
            if isinstance(st, F.Declare):
                if st.type.pointer:
                    raise CompileError("vectors cannot be declared inside a lambda", st.line)
                ctype = "float" if st.type.base == "float" else "long long"
                if st.value is None:
                    out.append(f"{pad}{ctype} {_local(st.name)} = 0;")
                else:
                    if not isinstance(st.value, F.Expr) or isinstance(st.value, (F.Reduce, F.Map, F.Concat)):
                        raise CompileError("vector primitives cannot be used inside a lambda", st.line)
                    v = self.expr(st.value, scope, index_name)
                    out.append(f"{pad}{ctype} {_local(st.name)} = ({ctype})({v.code});")
                scope[st.name] = "float" if ctype == "float" else "int"
            elif isinstance(st, F.Assign):
                if st.name not in scope:
                    raise CompileError(f"a lambda may only assign its own variables ({st.name!r})", st.line)
                v = self.expr(st.value, scope, index_name)
                out.append(f"{pad}{_local(st.name)} = {v.code};")
            elif isinstance(st, F.If):
                c = self.expr(st.cond, scope, index_name)
                out.append(f"{pad}if ({_unparen(c.code)}) {{")
                out += self.lambda_body(st.then, dict(scope), index_name, ret, depth + 1)
                if st.otherwise:
                    out.append(f"{pad}}} else {{")
                    out += self.lambda_body(st.otherwise, dict(scope), index_name, ret, depth + 1)
                out.append(f"{pad}}}")
            elif isinstance(st, F.Return):
                v = self.expr(st.value, scope, index_name)
                out.append(f"{pad}return ({ret})({v.code});")
            else:
                raise CompileError("statement not allowed inside a lambda", st.line)
        return out

    # ---------------------------------------------------------------- statements
    def serial(self) -> Stage:
        if not self.stages or self.stages[-1].kind != "serial":
            self.stages.append(Stage("serial"))
        return self.stages[-1]

    def assign_scalar(self, s: Scalar, value: F.Expr, line):
        if isinstance(value, F.Reduce):
            return self.reduce(s, value)
        if isinstance(value, (F.Map, F.Concat)):
            raise CompileError(f"{s.name!r} is a scalar; map and concat produce vectors", line)
        v = self.expr(value)
        if s.is_param:
            raise CompileError(f"parameter {s.name!r} cannot be assigned", line)
        if s.cls is not None and s.cls != v.cls and not (s.cls == "dev" and v.cls == "host"):
            raise CompileError(f"{s.name!r} cannot change from a host value to a device value", line)
        if s.cls == "host":
            # host-known scalars are all evaluated before the first launch, so a second value
            # would also be seen by the launches that should see the first
            raise CompileError(f"{s.name!r} is known on the host and can be assigned only once", line)
        self._guard_pending(line, scalar=s.name)
        s.cls = s.cls or v.cls
        if s.cls == "host":
            self.host_lines.append(f"a.v_{s.name} = ({s.ctype})({v.code});")
        else:
            self.serial().lines.append(f"d.v_{s.name} = ({s.ctype})({v.code});")

    def reduce(self, target: Scalar, r: F.Reduce):
        vec = self.vector(r.vec, r.line)
        if vec.elem != "float" or (vec.ptr is None and not vec.virtual):
            raise CompileError("reduce works on float vectors", r.line)
        if vec.virtual:
            if vec.virtual[0].cls != "host":
                raise CompileError("a mapped vector that is reduced needs a host-known length", r.line)
            self.compile_map_lambda(vec.virtual[1])
        if target.base != "float":
            raise CompileError("the result of reduce is a float", r.line)
        if r.fn not in self.lambdas:
            raise CompileError(f"unknown lambda {r.fn!r}", r.line)
        lam = self.lambdas[r.fn]
        if len(lam.params) != 2 or any(self._kind_of(p.type) != "float" for p in lam.params) or lam.ret.base != "float":
            raise CompileError(f"reduce needs a (float, float) -> float lambda, {r.fn!r} is not one", r.line)
        self.compile_lambda(r.fn)
        init = self.expr(r.init)
        if target.cls == "host":
            raise CompileError(f"{target.name!r} already holds a host value", r.line)
        target.cls = "dev"
        last = self.stages[-1] if self.stages else None
        if last and last.kind == "reduce" and last.vec is vec and init.cls == "host":
            last.folds.append((target, init.code, r.fn))
        else:
            st = Stage("reduce", vec=vec)
            st.folds.append((target, init.code, r.fn))
            self.stages.append(st)
            if vec not in self.reduced:
                self.reduced.append(vec)
        self.max_folds = max(self.max_folds, len(self.stages[-1].folds))

    def map_check(self, m: F.Map, want_ret):
        if m.fn not in self.lambdas:
            raise CompileError(f"unknown lambda {m.fn!r}", m.line)
        lam = self.lambdas[m.fn]
        if len(lam.params) != 1 or self._kind_of(lam.params[0].type) != "int":
            raise CompileError(f"map over a range needs a lambda of one integer, {m.fn!r} is not one", m.line)
        if want_ret == "float" and lam.ret.base != "float":
            raise CompileError(f"{m.fn!r} must return float here", m.line)
        if want_ret == "packed" and lam.ret.base != "uint":
            raise CompileError(f"{m.fn!r} must return uint<bits> here", m.line)
        count = self.expr(m.count)
        if count.kind != "int":
            raise CompileError("range() needs an integer", m.line)
        return lam, count

    def assign_vector(self, v: Vector, value, line):
        if isinstance(value, F.Map):
            if v.elem == "float":
                if not v.is_param:
                    raise CompileError("a local float vector is defined once, where it is declared", line)
                _, count = self.map_check(value, "float")
                self._guard_pending(line, vector=v.name)
                self.compile_map_lambda(value.fn)
                st = Stage("map_float", vec=v, fn=value.fn, count=count)
                st.bound = count.code if count.cls == "host" else v.size
                self.stages.append(st)
            elif v.elem == "packed":
                _, count = self.map_check(value, "packed")
                v.pending_map = (count, value.fn)
                v.size, v.size_cls = count.code, count.cls
            else:
                raise CompileError("map cannot fill a byte vector; use concat", line)
        elif isinstance(value, F.Concat):
            self.concat(v, value)
        else:
            raise CompileError(f"{v.name!r} is a vector; it can only be assigned map(...) or concat(...)", line)

    def concat(self, dest: Vector, c: F.Concat):
        if dest.elem != "bytes" or not dest.is_param:
            raise CompileError("concat writes into a uint8* parameter", c.line)
        off, writes = 0, []
        for k, name in enumerate(c.parts):
            if name in self.scalars:
                s = self.scalar(name, c.line)
                if s.cls is None:
                    raise CompileError(f"{name!r} has no value yet", c.line)
                writes.append(f"cl::put<{s.ctype}>({dest.ptr} + {off}, ({s.ctype}){s.ref()});")
                off += _SCALAR_BYTES.get(s.base, 4)
            else:
                vec = self.vector(name, c.line)
                if k != len(c.parts) - 1:
                    raise CompileError("a vector can only be the last part of concat", c.line)
                # the header fields are all known by now: they are written before the codes,
                # in the serial block that is open (or a new one), not in a launch of their own
                self.serial().lines += writes
                writes = []
                if vec.elem != "packed" or not vec.pending_map:
                    raise CompileError(f"{name!r} must be a uint<bits> vector just computed by map", c.line)
                count, fn = vec.pending_map
                vec.pending_map = None
                self.compile_map_lambda(fn)
                vec.ptr = f"({dest.ptr} + {off})"
                st = Stage("map_packed", vec=vec, fn=fn, count=count)
                st.dest, st.cap = vec.ptr, f"((long long){dest.size} - {off})"
                st.bits = Value(vec.bits, "int", vec.bits_cls)
                if count.cls != "host":
                    raise CompileError("a packed vector needs a host-known length", c.line)
                st.bound = count.code
                if vec.bits_cls == "host":
                    self.checks.append(f"if (!({vec.bits} == 1 || {vec.bits} == 2 || {vec.bits} == 4 || {vec.bits} == 8)) return -4;")
                    self.checks.append(f"if ((long long){off} + ((long long)({count.code}) * ({vec.bits}) + 7) / 8 > (long long){dest.size}) return -2;")
                self.stages.append(st)
        if writes:
            self.serial().lines += writes
        if off:
            self.checks.append(f"if ((long long){dest.size} < {off}) return -2;")

    def extract(self, st: F.Extract):
        src = self.vector(st.source, st.line)
        if src.elem != "bytes":
            raise CompileError("extract reads from a uint8* vector", st.line)
        off, lines = 0, []
        for k, name in enumerate(st.targets):
            if name in self.scalars:
                s = self.scalar(name, st.line)
                if s.is_param or s.cls == "host":
                    raise CompileError(f"{name!r} cannot receive an extracted value", st.line)
                s.cls = "dev"
                size = _SCALAR_BYTES.get(s.base, 4)
                lines.append(f"d.v_{name} = ((long long){src.size} >= {off + size}) ? cl::get<{s.ctype}>({src.ptr} + {off}) : ({s.ctype})0;")
                off += size
            else:
                vec = self.vector(name, st.line)
                if k != len(st.targets) - 1:
                    raise CompileError("a vector can only be the last target of extract", st.line)
                if vec.elem != "packed":
                    raise CompileError(f"{name!r} must be declared uint<bits>*", st.line)
                if vec.bits is None:
                    bits = self.expr(vec.bits_ast)
                    vec.bits, vec.bits_cls = bits.code, bits.cls
                vec.ptr = f"({src.ptr} + {off})"
                # bits outside {1,2,4,8} leave the vector empty
                b = vec.bits
                vec.size = (f"(((long long){src.size} > {off} && cl::valid_bits((int)({b}))) ? "
                            f"((long long){src.size} - {off}) * 8 / (long long)({b}) : 0ll)")
                vec.size_cls = "dev" if vec.bits_cls == "dev" else src.size_cls
        self.serial().lines += lines

    def declare(self, st: F.Declare):
        t = st.type
        if st.name in self.scalars or st.name in self.vectors or st.name in self.lambdas:
            raise CompileError(f"{st.name!r} is declared twice", st.line)
        if t.pointer:
            if t.base == "uint":
                try:
                    bits = self.expr(t.bits)
                    v = Vector(st.name, "packed", bits=bits.code, bits_cls=bits.cls)
                except CompileError:
                    if st.value is not None:
                        raise
                    v = Vector(st.name, "packed", bits_ast=t.bits)  # the width comes out of an extract
            elif t.base == "float":
                if not isinstance(st.value, F.Map):
                    raise CompileError("a local float vector must be defined by map(...)", st.line)
                _, count = self.map_check(st.value, "float")
                v = Vector(st.name, "float", size=count.code, size_cls=count.cls, virtual=(count, st.value.fn))
                self.vectors[st.name] = v
                return
            else:
                raise CompileError("local vectors must be float* or uint<bits>*", st.line)
            self.vectors[st.name] = v
            if st.value is not None:
                self.assign_vector(v, st.value, st.line)
            return
        base = t.base
        if base == "uint":
            base = "uint32"
        if base not in _SCALAR_C:
            raise CompileError(f"unsupported scalar type {t.base}", st.line)
        s = Scalar(st.name, base)
        self.scalars[st.name] = s
        if st.value is not None:
            self.assign_scalar(s, st.value, st.line)

    def statement(self, st):
        if isinstance(st, F.Lambda):
            if st.name in self.lambdas or st.name in self.scalars or st.name in self.vectors:
                raise CompileError(f"{st.name!r} is declared twice", st.line)
            self.lambdas[st.name] = st
        elif isinstance(st, F.Declare):
            self.declare(st)
        elif isinstance(st, F.Assign):
            if st.name in self.vectors:
                self.assign_vector(self.vectors[st.name], st.value, st.line)
            else:
                self.assign_scalar(self.scalar(st.name, st.line), st.value, st.line)
        elif isinstance(st, F.Extract):
            self.extract(st)
        else:
            raise CompileError("only declarations, assignments, lambdas and extract are allowed at function level", st.line)

    # ---------------------------------------------------------------- emission
    def launch_kinds(self):
        """The launches of the operator in order; a serial block right after a reduce
        runs inside the reduce's last kernel and is not a launch of its own."""
        out = []
        last = len(self.stages) - 1
        for k, st in enumerate(self.stages):
            if st.kind == "serial":
                if not st.lines or (k and self.stages[k - 1].kind == "reduce"):
                    continue
                if k == last - 1 and self.stages[last].kind in ("map_float", "map_packed", "map_fused") and _rerunnable(st.lines):
                    continue  # runs at the start of the last sweep
            out.append(st.kind)
        return out

    def signature(self):
        """[(c type, name)] of the entry point, and the manifest entry."""
        sig, man = [], []
        for p in self.fn.params:
            if p.type.pointer:
                ct = "float*" if p.type.base == "float" else "uint8_t*"
                sig += [(ct, p.name), ("int32_t", p.name + "_size")]
                man.append({"name": p.name, "kind": "float*" if p.type.base == "float" else "uint8*"})
        for p in self.fn.params:
            if not p.type.pointer:
                sig.append((_SCALAR_C[p.type.base], p.name))
                man.append({"name": p.name, "kind": p.type.base})
        if self.needs_uniform:
            sig += [("const float*", "uniform"), ("uint64_t", "seed")]
        sig += [("void*", "workspace"), ("int64_t", "workspace_bytes"), ("void*", "stream")]
        return sig, man

    def emit(self) -> str:
        name, o = self.fn.name, []
        o.append(f"namespace {self.ns} {{")
        o.append("struct Args {")
        for v in self.vectors.values():
            if v.is_param:
                o.append(f"    {'float' if v.elem == 'float' else 'uint8_t'}* v_{v.name};")
                o.append(f"    long long v_{v.name}_size;")
        for s in self.scalars.values():
            if s.cls == "host":
                o.append(f"    {s.ctype} v_{s.name};")
        o.append("    const float* uniform;")
        o.append("    unsigned ukey;")
        o.append("};")
        o.append("struct Dev {")
        dev = [s for s in self.scalars.values() if s.cls == "dev"]
        for s in dev:
            o.append(f"    {s.ctype} v_{s.name};")
        if not dev:
            o.append("    int unused;")
        o.append("};")
        for ln in self.lambda_order:
            o.append(self.lambda_code[ln])
        launches = []
        fused = set()  # serial blocks that run at the end of the reduce before them
        for k, st in enumerate(self.stages):
            if st.kind == "reduce" and k + 1 < len(self.stages) and self.stages[k + 1].kind == "serial" and self.stages[k + 1].lines:
                fused.add(k + 1)
        # a serial block right before the last sweep of the operator runs at the start of that
        # sweep, in every workgroup, if running it again changes nothing
        before = {}
        last = len(self.stages) - 1
        if last >= 1 and self.stages[last].kind in ("map_float", "map_packed", "map_fused") and self.stages[last - 1].kind == "serial" \
                and self.stages[last - 1].lines and (last - 1) not in fused and _rerunnable(self.stages[last - 1].lines):
            before[last] = last - 1
        order = sorted(range(len(self.stages)), key=lambda k: (k - 1.5) if k in fused else k)  # a fused block is emitted first
        for k in order:
            st = self.stages[k]
            if st.kind == "serial":
                if not st.lines:
                    continue
                o.append(f"struct Serial{k} {{")
                o.append("    static __device__ void run(const Args& a, Dev& d) {")
                o += ["        " + ln for ln in st.lines]
                o.append("    }")
                o.append("};")
                if k not in fused and k not in before.values():
                    launches.append(f"hipLaunchKernelGGL((cl::serial_kernel<Args, Dev, Serial{k}>), dim3(1), dim3(64), 0, st, a, d);")
            elif st.kind == "reduce":
                K = len(st.folds)
                o.append(f"struct Folds{k} {{")
                o.append(f"    static constexpr int K = {K};")
                o.append("    static __device__ __forceinline__ float init(const Args& a, const Dev& d, int k) {")
                for i, (_, init, _) in enumerate(st.folds):
                    o.append(f"        if (k == {i}) return (float)({init});")
                o.append("        return 0.f;")
                o.append("    }")
                o.append("    static __device__ __forceinline__ float apply(const Args& a, const Dev& d, int k, float x, float y) {")
                for i, (_, _, fn) in enumerate(st.folds):
                    o.append(f"        if (k == {i}) return fn_{fn}(a, d, x, y);")
                o.append("        return x;")
                o.append("    }")
                o.append("    static __device__ __forceinline__ void store(Dev& d, int k, float v) {")
                for i, (t, _, _) in enumerate(st.folds):
                    o.append(f"        if (k == {i}) d.v_{t.name} = v;")
                o.append("    }")
                o.append("};")
                n = st.vec.size
                o.append(f"struct Source{k} {{  // what is folded: a stored vector, or a mapped one computed on the way")
                o.append(f"    static __device__ __forceinline__ long long count(const Args& a, const Dev& d) {{ return (long long)({n}); }}")
                if st.vec.virtual:
                    fn = st.vec.virtual[1]
                    streams = self.map_streams[fn]
                    call = f"mfn_{fn}(a, d, i, s)"
                else:
                    streams, call = [st.vec.ptr], "s[0]"
                o.append(f"    static constexpr int NS = {len(streams)};")
                o.append(f"    static constexpr int UNIFORM = {streams.index('a.uniform') if 'a.uniform' in streams else -1};  // the stream that may come without a vector")
                o.append("    static __device__ __forceinline__ const float* stream(const Args& a, int k) {")
                for i, ptr in enumerate(streams):
                    o.append(f"        if (k == {i}) return {ptr};")
                o.append("        return nullptr;")
                o.append("    }")
                o.append(f"    static __device__ __forceinline__ float call(const Args& a, const Dev& d, long long i, const float* s) {{ return {call}; }}")
                o.append("};")
                if st.vec.virtual:
                    for ptr in streams:
                        if ptr != "a.uniform":
                            self.checks.append(f"if ((long long)({n}) > (long long){ptr}_size) return -2;")
                launches.append(f"{{ const long long n = {n}; const unsigned tiles = (unsigned)(n > 0 ? (n + cl::kTile - 1) / cl::kTile : 0);")
                launches.append(f"  if (tiles) hipLaunchKernelGGL((cl::reduce_tiles_kernel<Args, Dev, Folds{k}, Source{k}>), dim3(tiles), dim3(cl::kBlock), 0, st, a, d, partial);")
                after = f"Serial{k + 1}" if k + 1 in fused else "cl::Nothing"
                launches.append(f"  hipLaunchKernelGGL((cl::reduce_final_kernel<Args, Dev, Folds{k}, {after}>), dim3(1), dim3(cl::kFinalBlock), 0, st, a, d, partial, tiles); }}")
            else:
                o.append(f"struct Map{k} {{")
                o.append(f"    static __device__ __forceinline__ long long count(const Args& a, const Dev& d) {{ return (long long)({st.count.code}); }}")
                streams = list(self.map_streams[st.fn])
                if st.kind == "map_fused":
                    for ptr in self.map_streams[st.float_map.fn]:
                        if ptr not in streams:
                            streams.append(ptr)
                o.append(f"    static constexpr int NS = {len(streams)};  // float vectors read at the index itself")
                o.append(f"    static constexpr int UNIFORM = {streams.index('a.uniform') if 'a.uniform' in streams else -1};  // the stream that may come without a vector")
                o.append("    static __device__ __forceinline__ const float* stream(const Args& a, int k) {")
                for i, ptr in enumerate(streams):
                    o.append(f"        if (k == {i}) return {ptr};")
                o.append("        return nullptr;")
                o.append("    }")
                if st.kind in ("map_packed", "map_fused"):
                    o.append(f"    static __device__ __forceinline__ int bits(const Args& a, const Dev& d) {{ return (int)({st.bits.code}); }}")
                    lam = self.lambdas[st.fn]
                    ret = {"float": "float", "int": "long long"}[self.lambda_kind(lam)]
                else:
                    ret = "float"
                if st.kind == "map_fused":  # each lambda sees its own operands in its own order
                    for label, fn, r in (("call_codes", st.fn, ret), ("call_values", st.float_map.fn, "float")):
                        own = self.map_streams[fn]
                        picks = ", ".join(f"s[{streams.index(ptr)}]" for ptr in own) or "0.f"
                        o.append(f"    static __device__ __forceinline__ {r} {label}(const Args& a, const Dev& d, long long i, const float* s) {{")
                        o.append(f"        const float mine[{max(len(own), 1)}] = {{{picks}}};")
                        o.append(f"        return mfn_{fn}(a, d, i, mine);")
                        o.append("    }")
                else:
                    o.append(f"    static __device__ __forceinline__ {ret} call(const Args& a, const Dev& d, long long i, const float* s) {{ return mfn_{st.fn}(a, d, i, s); }}")
                o.append("};")
                for ptr in streams:  # a streamed vector must cover the range
                    if ptr != "a.uniform" and st.count.cls == "host":
                        self.checks.append(f"if ((long long)({st.count.code}) > (long long){ptr}_size) return -2;")
                launches.append(f"{{ long long bound = (long long)({st.bound}); if (bound < 0) bound = 0;")
                launches.append("  const unsigned tiles = (unsigned)((bound + cl::kTile - 1) / cl::kTile);")
                pre = f"Serial{before[k]}" if k in before else "cl::Nothing"
                if st.kind == "map_fused":
                    launches.append(f"  if (tiles) hipLaunchKernelGGL((cl::map_fused_kernel<Args, Dev, Map{k}, {pre}>), dim3(tiles), dim3(cl::kBlock), 0, st, a, d, {st.dest}, {st.cap}, {st.float_map.vec.ptr});")
                elif st.kind == "map_packed":
                    launches.append(f"  if (tiles) hipLaunchKernelGGL((cl::map_packed_kernel<Args, Dev, Map{k}, {pre}>), dim3(tiles), dim3(cl::kBlock), 0, st, a, d, {st.dest}, {st.cap});")
                else:
                    launches.append(f"  if (tiles) hipLaunchKernelGGL((cl::map_float_kernel<Args, Dev, Map{k}, {pre}>), dim3(tiles), dim3(cl::kBlock), 0, st, a, d, {st.vec.ptr}, (long long){st.vec.size});")
                if k in before:  # an empty range launches no sweep; the block still has to run
                    launches.append(f"  else hipLaunchKernelGGL((cl::serial_kernel<Args, Dev, {pre}>), dim3(1), dim3(64), 0, st, a, d);")
                launches.append("}")
        o.append(f"}}  // namespace {self.ns}")
        o.append("")
        sig, _ = self.signature()
        K = max(self.max_folds, 1)
        o.append(f'extern "C" int64_t {name}_workspace_bytes(int64_t max_elements) {{')
        o.append("    if (max_elements < 0) return -2;")
        o.append(f"    return 256 + 4 * {K} * ((max_elements + cl::kTile - 1) / cl::kTile + 1);")
        o.append("}")
        o.append("")
        o.append(f"// {name}: vectors with their lengths in elements, then the scalar parameters" +
                 (", then `uniform`: one uniform[0,1) float per element of the longest mapped range, or NULL: the values are then drawn in the kernels from `seed`" if self.needs_uniform else "") +
                 f"; workspace of at least {name}_workspace_bytes(longest float vector) bytes, 16-byte aligned;")
        o.append("// returns 0, -1 null pointer, -2 a buffer too small, -3 misaligned workspace, -4 bad parameter, -5 HIP error, -6 workspace.")
        o.append(f'extern "C" int {name}({", ".join(t + " " + n for t, n in sig)}) {{')
        o.append(f"    using namespace {self.ns};")
        o.append("    Args a;")
        for v in self.vectors.values():
            if v.is_param:
                o.append(f"    if ({v.name}_size < 0) return -2;")
                o.append(f"    if ({v.name}_size > 0 && !{v.name}) return -1;")
                o.append(f"    a.v_{v.name} = {v.name};")
                o.append(f"    a.v_{v.name}_size = {v.name}_size;")
        for s in self.scalars.values():
            if s.is_param:
                o.append(f"    a.v_{s.name} = {s.name};")
        if self.needs_uniform:
            o.append("    a.uniform = uniform;")
            o.append("    a.ukey = hp::tensor_key(hp::uniform_key(seed), 0u);")
        else:
            o.append("    a.uniform = nullptr;")
            o.append("    a.ukey = 0u;")
        o += ["    " + ln for ln in self.host_lines]
        o += ["    " + ln for ln in self.checks]
        biggest = " , ".join(f"(long long){v.size}" for v in self.reduced) or "0ll"
        o.append(f"    long long reduced = 0; for (long long x : {{{biggest}}}) reduced = x > reduced ? x : reduced;")
        o.append(f"    if (!workspace || workspace_bytes < {name}_workspace_bytes(reduced)) return -6;")
        o.append("    if (reinterpret_cast<uintptr_t>(workspace) & 15u) return -3;")
        o.append("    Dev* d = static_cast<Dev*>(workspace);")
        o.append("    float* partial = reinterpret_cast<float*>(static_cast<char*>(workspace) + 256);")
        o.append("    (void)partial;")
        o.append("    hipStream_t st = static_cast<hipStream_t>(stream);")
        o += ["    " + ln for ln in launches]
        o.append("    return hipGetLastError() == hipSuccess ? 0 : -5;")
        o.append("}")
        return "\n".join(o)


def generate(program: F.Program):
    """-> (HIP source text, manifest).  The manifest lists, per operator, its parameters
    in call order so that a host language can bind the entry points."""
    parts = ["// Generated by hipress_amd.compll from an operator program; do not edit.",
             '#include "compll_prims.h"', "#include <initializer_list>", ""]
    manifest = []
    for fn in program.functions:
        g = FunctionGen(fn)
        parts.append(g.emit())
        parts.append("")
        _, man = g.signature()
        manifest.append({"name": fn.name, "params": man, "uniform": g.needs_uniform,
                         "launches": g.launch_kinds()})
    return "\n".join(parts), manifest
