"""Front end for the CompLL operator language: text -> syntax tree.

The language is the one the reference's generator reads
(/root/reference/src/CompLL/GCGen/parser.py:3-8 for the token classes,
/root/reference/src/CompLL/GCGen/tree.py:48-660 for the constructs): optional
`param` blocks, `void` functions over typed vectors and scalars, `lambda_func`
definitions with C-like bodies, and the vector primitives `reduce`, `map` over
`range`, `concat`, `extract`, `random<T>(lo, hi)` and `.size`.  This is a
recursive-descent parser with ordinary C operator precedence; it builds plain
dataclasses and knows nothing about code generation.
"""
from dataclasses import dataclass, field
from typing import List, Optional


class CompileError(Exception):
    def __init__(self, msg, line=None):
        super().__init__(f"line {line}: {msg}" if line else msg)
        self.line = line


# ---------------------------------------------------------------- tokens
@dataclass
class Token:
    kind: str  # name | int | float | op | end
    text: str
    line: int


_OPS3 = ["[&]"]
_OPS2 = ["<<", ">>", "->", "==", "!=", "<=", ">=", "&&", "||"]
_OPS1 = list("+-*/%[](){};,=<>&|^!.")


def tokenize(text: str) -> List[Token]:
    out, i, line, n = [], 0, 1, len(text)
    while i < n:
        c = text[i]
        if c == "\n":
            line += 1
            i += 1
        elif c.isspace():
            i += 1
        elif text.startswith("//", i):
            while i < n and text[i] != "\n":
                i += 1
        elif text.startswith("/*", i):
            j = text.find("*/", i + 2)
            if j < 0:
                raise CompileError("comment never closed", line)
            line += text.count("\n", i, j)
            i = j + 2
        elif c.isalpha() or c == "_":
            j = i
            while j < n and (text[j].isalnum() or text[j] == "_"):
                j += 1
            out.append(Token("name", text[i:j], line))
            i = j
        elif c.isdigit():
            j = i
            while j < n and text[j].isdigit():
                j += 1
            kind = "int"
            if j < n and text[j] == "." and j + 1 < n and text[j + 1].isdigit():
                kind = "float"
                j += 1
                while j < n and text[j].isdigit():
                    j += 1
            if j < n and text[j] in "eE" and (j + 1 < n and (text[j + 1].isdigit() or text[j + 1] in "+-")):
                kind = "float"
                j += 2
                while j < n and text[j].isdigit():
                    j += 1
            out.append(Token(kind, text[i:j], line))
            i = j
        else:
            for group in (_OPS3, _OPS2, _OPS1):
                op = next((o for o in group if text.startswith(o, i)), None)
                if op:
                    break
            if not op:
                raise CompileError(f"unexpected character {c!r}", line)
            out.append(Token("op", op, line))
            i += len(op)
    out.append(Token("end", "", line))
    return out


# ---------------------------------------------------------------- tree
@dataclass
class Type:
    base: str                      # float | int | uint8 | uint16 | uint32 | int32 | uint
    bits: Optional["Expr"] = None  # uint<bits>
    pointer: bool = False
    line: int = 0


@dataclass
class Expr:
    line: int = 0


@dataclass
class Num(Expr):
    text: str = "0"
    is_float: bool = False


@dataclass
class Name(Expr):
    id: str = ""


@dataclass
class Unary(Expr):
    op: str = ""
    arg: Expr = None


@dataclass
class Binary(Expr):
    op: str = ""
    lhs: Expr = None
    rhs: Expr = None


@dataclass
class Index(Expr):
    vec: str = ""
    index: Expr = None


@dataclass
class SizeOf(Expr):
    vec: str = ""


@dataclass
class Call(Expr):
    fn: str = ""
    args: List[Expr] = field(default_factory=list)


@dataclass
class Random(Expr):
    type: Type = None
    lo: Expr = None
    hi: Expr = None


@dataclass
class Reduce(Expr):
    vec: str = ""
    init: Expr = None
    fn: str = ""


@dataclass
class Map(Expr):
    count: Expr = None  # map(range(count), fn)
    fn: str = ""


@dataclass
class Concat(Expr):
    parts: List[str] = field(default_factory=list)


@dataclass
class Stmt:
    line: int = 0


@dataclass
class Declare(Stmt):
    type: Type = None
    name: str = ""
    value: Optional[Expr] = None


@dataclass
class Assign(Stmt):
    name: str = ""
    value: Expr = None


@dataclass
class Extract(Stmt):
    source: str = ""
    targets: List[str] = field(default_factory=list)


@dataclass
class If(Stmt):
    cond: Expr = None
    then: List[Stmt] = field(default_factory=list)
    otherwise: List[Stmt] = field(default_factory=list)


@dataclass
class Return(Stmt):
    value: Expr = None


@dataclass
class Param:
    type: Type
    name: str


@dataclass
class Lambda(Stmt):
    name: str = ""
    params: List[Param] = field(default_factory=list)
    ret: Type = None
    body: List[Stmt] = field(default_factory=list)


@dataclass
class Function:
    name: str
    params: List[Param]
    body: List[Stmt]
    line: int = 0


@dataclass
class Program:
    functions: List[Function]
    param_blocks: dict  # name -> [Param]; accepted for compatibility, not used by the back end


_TYPES = {"float", "int", "int32", "uint8", "uint16", "uint32", "uint"}
_BINARY_LEVELS = [["||"], ["&&"], ["|"], ["^"], ["&"], ["==", "!="], ["<", ">", "<=", ">="], ["<<", ">>"], ["+", "-"],
                  ["*", "/", "%"]]


class Parser:
    def __init__(self, text: str):
        self.toks = tokenize(text)
        self.i = 0

    # -- token helpers
    @property
    def tok(self) -> Token:
        return self.toks[self.i]

    def peek(self, k=1) -> Token:
        return self.toks[min(self.i + k, len(self.toks) - 1)]

    def at(self, text) -> bool:
        return self.tok.text == text and self.tok.kind in ("op", "name")

    def take(self, text=None, kind=None) -> Token:
        t = self.tok
        if (text is not None and t.text != text) or (kind is not None and t.kind != kind):
            want = text if text is not None else kind
            raise CompileError(f"expected {want!r}, found {t.text!r}", t.line)
        self.i += 1
        return t

    def maybe(self, text) -> bool:
        if self.at(text):
            self.i += 1
            return True
        return False

    # -- grammar
    def program(self) -> Program:
        funcs, blocks = [], {}
        while self.tok.kind != "end":
            if self.at("param"):
                name, fields = self.param_block()
                blocks[name] = fields
            else:
                funcs.append(self.function())
        if not funcs:
            raise CompileError("no function in the program", self.tok.line)
        return Program(funcs, blocks)

    def param_block(self):
        self.take("param")
        name = self.take(kind="name").text
        self.take("{")
        fields = []
        while not self.at("}"):
            t = self.type()
            fields.append(Param(t, self.take(kind="name").text))
            self.take(";")
        self.take("}")
        return name, fields

    def is_type_start(self) -> bool:
        return self.tok.kind == "name" and self.tok.text in _TYPES

    def type(self) -> Type:
        t = self.take(kind="name")
        if t.text not in _TYPES:
            raise CompileError(f"unknown type {t.text!r}", t.line)
        ty = Type(t.text, line=t.line)
        if t.text == "uint":
            self.take("<")
            ty.bits = self.expr(stop_at_gt=True)
            self.take(">")
        if self.maybe("*"):
            ty.pointer = True
        return ty

    def params(self) -> List[Param]:
        self.take("(")
        ps = []
        while not self.at(")"):
            ty = self.type()
            ps.append(Param(ty, self.take(kind="name").text))
            if not self.maybe(","):
                break
        self.take(")")
        return ps

    def function(self) -> Function:
        line = self.take("void").line
        name = self.take(kind="name").text
        return Function(name, self.params(), self.block(), line)

    def block(self) -> List[Stmt]:
        self.take("{")
        body = []
        while not self.at("}"):
            body.append(self.statement())
        self.take("}")
        return body

    def statement(self) -> Stmt:
        t = self.tok
        if self.at("lambda_func"):
            return self.lambda_func()
        if self.at("if"):
            self.take("if")
            self.take("(")
            cond = self.expr()
            self.take(")")
            then = self.block()
            other = []
            if self.maybe("else"):
                other = [self.statement()] if self.at("if") else self.block()
            return If(t.line, cond, then, other)
        if self.at("return"):
            self.take("return")
            v = self.expr()
            self.take(";")
            return Return(t.line, v)
        if self.at("extract"):
            self.take("extract")
            self.take("(")
            names = [self.take(kind="name").text]
            while self.maybe(","):
                names.append(self.take(kind="name").text)
            self.take(")")
            self.take(";")
            if len(names) < 2:
                raise CompileError("extract needs a source and at least one target", t.line)
            return Extract(t.line, names[0], names[1:])
        if self.is_type_start():
            ty = self.type()
            name = self.take(kind="name").text
            value = self.rhs() if self.maybe("=") else None
            self.take(";")
            return Declare(t.line, ty, name, value)
        if t.kind == "name" and self.peek().text == "=":
            name = self.take(kind="name").text
            self.take("=")
            value = self.rhs()
            self.take(";")
            return Assign(t.line, name, value)
        raise CompileError(f"statement cannot start with {t.text!r}", t.line)

    def lambda_func(self) -> Lambda:
        line = self.take("lambda_func").line
        name = self.take(kind="name").text
        self.take("=")
        self.take("[&]")
        ps = self.params()
        self.take("->")
        ret = self.type()
        body = self.block()
        self.maybe(";")
        return Lambda(line, name, ps, ret, body)

    def rhs(self) -> Expr:
        t = self.tok
        if self.at("reduce") and self.peek().text == "(":
            self.take("reduce")
            self.take("(")
            vec = self.take(kind="name").text
            self.take(",")
            init = self.expr()
            self.take(",")
            fn = self.take(kind="name").text
            self.take(")")
            return Reduce(t.line, vec, init, fn)
        if self.at("map") and self.peek().text == "(":
            self.take("map")
            self.take("(")
            self.take("range")
            self.take("(")
            count = self.expr()
            self.take(")")
            self.take(",")
            fn = self.take(kind="name").text
            self.take(")")
            return Map(t.line, count, fn)
        if self.at("concat") and self.peek().text == "(":
            self.take("concat")
            self.take("(")
            parts = [self.take(kind="name").text]
            while self.maybe(","):
                parts.append(self.take(kind="name").text)
            self.take(")")
            return Concat(t.line, parts)
        return self.expr()

    def expr(self, level=0, stop_at_gt=False) -> Expr:
        if level == len(_BINARY_LEVELS):
            return self.unary()
        lhs = self.expr(level + 1, stop_at_gt)
        while self.tok.kind == "op" and self.tok.text in _BINARY_LEVELS[level]:
            if stop_at_gt and self.tok.text in (">", ">>", ">="):
                break  # the '>' that closes uint<...>
            op = self.take()
            rhs = self.expr(level + 1, stop_at_gt)
            lhs = Binary(op.line, op.text, lhs, rhs)
        return lhs

    def unary(self) -> Expr:
        t = self.tok
        if t.kind == "op" and t.text in ("-", "!", "+"):
            self.take()
            return Unary(t.line, t.text, self.unary())
        return self.postfix()

    def postfix(self) -> Expr:
        t = self.tok
        if t.kind in ("int", "float"):
            self.take()
            return Num(t.line, t.text, t.kind == "float")
        if self.maybe("("):
            e = self.expr()
            self.take(")")
            return e
        if t.kind != "name":
            raise CompileError(f"expression cannot start with {t.text!r}", t.line)
        self.take()
        if t.text == "random" and self.at("<"):
            self.take("<")
            ty = self.type()
            self.take(">")
            self.take("(")
            lo = self.expr()
            self.take(",")
            hi = self.expr()
            self.take(")")
            return Random(t.line, ty, lo, hi)
        if self.maybe("("):
            args = []
            while not self.at(")"):
                args.append(self.expr())
                if not self.maybe(","):
                    break
            self.take(")")
            return Call(t.line, t.text, args)
        if self.maybe("["):
            idx = self.expr()
            self.take("]")
            return Index(t.line, t.text, idx)
        if self.at(".") and self.peek().text == "size":
            self.take(".")
            self.take("size")
            return SizeOf(t.line, t.text)
        return Name(t.line, t.text)


def parse(text: str) -> Program:
    return Parser(text).program()
