"""Reader and printer of LLH graphs in MLIR's generic op syntax, the wire format between the reference's importer
and its compiler (llcompiler/compiler/compiler.py:133-135 hands the printed module to the C++ side, which parses
it at src/Support/File.cpp:60-76) and the language of its lit tests (test/Conversion/LLHToHLO/llh_to_hlo.mlir,
test/RunnerTest/abs.mlir):

    func.func @main(%arg0: tensor<?x3x?x?xf32>) -> tensor<?x4x?x?xf32> attributes {entrance} {
      %0 = "llh.constant"() <{value = 2 : i64}> : () -> i64
      %1 = "llh.dim"(%arg0, %0) : (tensor<?x3x?x?xf32>, i64) -> i64
      %2 = "llh.conv"(%arg0, %w) <{dilation = array<i64: 1, 1>, ...}> : (...) -> tensor<?x4x?x?xf32>
      return %2 : tensor<?x4x?x?xf32>
    }

`parse_llh(text)` builds a Graph: tensor ops become graph ops (result shapes are inferred again, the printed
result types are only checked for rank); the scalar side of the dialect (i64 constants, llh.dim, arithmetic on
i64, llh.torch_symbolic_int) becomes symbolic extents; the ops of the symbol system that carry no computation
(symbolic_int, symbol_bind, encoding_bind, symbol_relation...) are skipped.  A function without results returns
the operands of its llh.print ops, which is how the reference's runner tests observe values.
`print_llh(graph)` writes a Graph in the same syntax (shape operands as attributes).
"""
import re

import torch

from .expr import Expr
from .graph import BINARY_OPS, COMPARE_KINDS, DTYPE_NAMES, UNARY_OPS, Graph, Value

_DTYPES = {v: k for k, v in DTYPE_NAMES.items()}
_DTYPES["index"] = torch.int64
_SKIPPED = ("symbolic_int", "symbol_bind", "symbolic_bind", "encoding_bind", "symbol_relation", "symbol_relations",
            "symbol_relation_map", "symbol_binary_relation", "symbolic_cast")


class LLHSyntaxError(ValueError):
    pass


class _Cursor:
    def __init__(self, text):
        self.s, self.i = text, 0

    def ws(self):
        while self.i < len(self.s) and self.s[self.i] in " \t\r\n":
            self.i += 1

    def eof(self):
        self.ws()
        return self.i >= len(self.s)

    def peek(self, lit):
        self.ws()
        return self.s.startswith(lit, self.i)

    def take(self, lit):
        if self.peek(lit):
            self.i += len(lit)
            return True
        return False

    def expect(self, lit):
        if not self.take(lit):
            raise LLHSyntaxError("expected %r at ...%s" % (lit, self.s[self.i:self.i + 40].replace("\n", " ")))

    def match(self, pattern):
        self.ws()
        m = re.compile(pattern).match(self.s, self.i)
        if m:
            self.i = m.end()
        return m

    def bracketed(self, open_, close):
        """The text between a bracket pair at the cursor, nesting respected, strings skipped."""
        self.expect(open_)
        depth, start = 1, self.i
        while self.i < len(self.s):
            c = self.s[self.i]
            if c == '"':
                self.i = self.s.index('"', self.i + 1)
            elif c == "-" and self.s.startswith("->", self.i):
                self.i += 1  # the '>' of an arrow closes nothing
            elif c == open_:
                depth += 1
            elif c == close:
                depth -= 1
                if depth == 0:
                    out = self.s[start:self.i]
                    self.i += 1
                    return out
            self.i += 1
        raise LLHSyntaxError("unbalanced %s" % open_)


def _strip_comments(text):
    out = []
    for line in text.splitlines():
        i, in_str = 0, False
        while i < len(line):
            if line[i] == '"':
                in_str = not in_str
            elif not in_str and line.startswith("//", i):
                line = line[:i]
                break
            i += 1
        out.append(line)
    return "\n".join(out)


def _split_top(text, sep=","):
    parts, depth, cur, in_str = [], 0, [], False
    for c in text:
        if c == '"':
            in_str = not in_str
        if not in_str:
            if c in "<([{":
                depth += 1
            elif c in ">)]}":
                depth -= 1
            elif c == sep and depth == 0:
                parts.append("".join(cur).strip())
                cur = []
                continue
        cur.append(c)
    tail = "".join(cur).strip()
    if tail:
        parts.append(tail)
    return parts


# ------------------------------------------------------------------------------------------ types
class _Type:
    def __init__(self, kind, shape=(), dtype=None, symbols=None, ranked=True):
        self.kind, self.shape, self.dtype, self.symbols, self.ranked = kind, tuple(shape), dtype, symbols, ranked


def _parse_type(text):
    text = text.strip()
    if text in _DTYPES:
        return _Type("scalar", dtype=_DTYPES[text])
    if text in ("()", "none"):
        return _Type("none")
    m = re.match(r"tensor<(.*)>$", text, re.S)
    if not m:
        raise LLHSyntaxError("type %r" % text)
    parts = _split_top(m.group(1))
    symbols = None
    if len(parts) > 1:  # tensor<?x3xf32, #llh.encoding<shapes = @s0, @c3>>
        symbols = re.findall(r"@([A-Za-z_][\w]*)", parts[1])
    toks = parts[0].strip().split("x")
    dtype = _DTYPES.get(toks[-1].strip())
    if dtype is None:
        raise LLHSyntaxError("element type in %r" % text)
    if toks[0].strip() == "*":  # tensor<*xf32>: rank and extents are whatever shape inference says
        return _Type("tensor", (), dtype, None, ranked=False)
    dims = []
    for t in toks[:-1]:
        t = t.strip()
        dims.append(None if t == "?" else int(t))
    return _Type("tensor", dims, dtype, symbols)


def _type_list(text):
    text = text.strip()
    if text.startswith("("):
        text = text[1:text.rindex(")")]
    return [_parse_type(t) for t in _split_top(text)] if text.strip() else []


# ------------------------------------------------------------------------------------------ attributes
def _number(tok):
    tok = tok.strip()
    if tok in ("true", "false"):
        return tok == "true"
    if re.fullmatch(r"[-+]?\d+", tok):
        return int(tok)
    if re.fullmatch(r"0x[0-9a-fA-F]+", tok):
        return int(tok, 16)
    return float(tok)


def _parse_attr(text):
    text = text.strip()
    if text.startswith('"'):
        return text[1:text.rindex('"')]
    if text.startswith("@"):
        return text[1:]
    if text.startswith("array<"):
        body = text[6:text.rindex(">")]
        body = body.split(":", 1)[1] if ":" in body else ""
        return tuple(_number(t) for t in body.split(",") if t.strip())
    if text.startswith("dense<"):
        c = _Cursor(text[5:])
        body = c.bracketed("<", ">")
        c.expect(":")
        ty = _parse_type(text[5 + c.i:])
        body = body.strip()
        if body.startswith("["):
            vals = [_number(t) for t in re.sub(r"[\[\]]", " ", body).replace(",", " ").split()]
            return ("dense", vals, ty)
        return ("dense", _number(body), ty)
    if text.startswith("#"):  # #llh.Layout<NCHW>, #llh.Compare<EQ>, #llh.encoding<...>
        m = re.match(r"#[\w.]+<(.*)>$", text, re.S)
        return m.group(1).strip() if m else text
    if ":" in text:  # 3 : i64, 1.000000e-05 : f64
        val, ty = text.rsplit(":", 1)
        v = _number(val)
        t = _parse_type(ty)
        return float(v) if t.dtype is not None and t.dtype.is_floating_point else v
    if text in ("unit",):
        return True
    return _number(text)


def _parse_attr_dict(text):
    out = {}
    for item in _split_top(text):
        if "=" in item:
            k, v = item.split("=", 1)
            out[k.strip()] = _parse_attr(v)
        else:
            out[item.strip()] = True
    return out


# ------------------------------------------------------------------------------------------ reader
class _Reader:
    def __init__(self):
        self.g = Graph()
        self.env = {}        # SSA name -> Value | int | float | Expr
        self.printed = []
        self.n_sym = 0

    def fresh_symbol(self):
        self.n_sym += 1
        return "d%d" % self.n_sym

    def operand(self, name):
        try:
            return self.env[name]
        except KeyError:
            raise LLHSyntaxError("use of undefined value %%%s" % name)

    def tensor(self, name):
        v = self.operand(name)
        if not isinstance(v, Value):
            raise LLHSyntaxError("%%%s is not a tensor" % name)
        return v

    def scalar(self, name):
        v = self.operand(name)
        if isinstance(v, Value):
            if v.const is None:
                raise LLHSyntaxError("%%%s is not a scalar" % name)
            return v.const
        return v

    def add_argument(self, name, ty):
        if ty.kind == "scalar":
            sym = name if name.startswith("s") else self.fresh_symbol()
            self.g.add_symbol_arg(sym)
            self.env[name] = Expr.sym(sym)
            return
        shape = []
        for k, d in enumerate(ty.shape):
            if d is not None:
                shape.append(d)
            elif ty.symbols and k < len(ty.symbols) and ty.symbols[k] and not re.fullmatch(r"c\d+", ty.symbols[k]):
                shape.append(Expr.sym(ty.symbols[k]))
            else:
                shape.append(Expr.sym(self.fresh_symbol()))
        self.env[name] = self.g.add_input(tuple(shape), ty.dtype, name=name)

    def constant(self, attrs, rtype):
        v = attrs["value"]
        if rtype.kind == "scalar":
            return v[1] if isinstance(v, tuple) else v
        if isinstance(v, tuple):
            _, val, ty = v
            shape, dtype = tuple(ty.shape), ty.dtype
        else:
            val, shape, dtype = v, tuple(rtype.shape), rtype.dtype
        n = 1
        for d in shape:
            n *= d
        if isinstance(val, list) and len(val) == 1:
            val = val[0]
        const = val if (n == 1 and not isinstance(val, list)) else None
        return self.g.add_op("constant", [], {"value": val}, shapes=[shape], dtypes=[dtype], const=const)

    def emit(self, name, operands, attrs, rtypes):
        g = self.g
        rt = rtypes[0] if rtypes else _Type("none")
        if name in _SKIPPED:
            return None
        if name == "constant":
            return self.constant(attrs, rt)
        if name == "torch_symbolic_int":
            return Expr.sym(attrs["sym_name"])
        if name == "dim":
            t = self.tensor(operands[0])
            k = int(self.scalar(operands[1]))
            return t.shape[k % t.rank]
        if rt.kind == "scalar" and name in ("add", "sub", "mul", "div"):
            a, b = (self.scalar(o) for o in operands)
            if name == "div" and not isinstance(b, Expr) and b == 0:
                raise NotImplementedError("llh.div of scalars by the constant 0")
            return {"add": lambda: a + b, "sub": lambda: a - b, "mul": lambda: a * b, "div": lambda: a // b}[name]()
        if name == "scalar_cast":
            # an i64 (or float) scalar as a one-element tensor (LLHOps.td:120-127): a constant when the scalar is a
            # number, else a value that every binding of the symbols fills in
            v = self.scalar(operands[0])
            shape = tuple(rt.shape) if len(rt.shape) else (1,)
            if isinstance(v, Expr):
                return g.add_op("scalar_cast", [], {"value": v}, shapes=[shape], dtypes=[rt.dtype], const=v)
            return g.add_op("constant", [], {"value": v}, shapes=[shape], dtypes=[rt.dtype], const=v)
        if name == "print":
            self.printed.append(self.tensor(operands[0]))
            return None
        if name == "weight":
            shape = tuple(rt.shape) if len(rt.shape) else (1,)  # tensor<f32> is refined to tensor<1xf32>
            return g.add_op("weight", [], {"weight_file": attrs["weight_file"]}, shapes=[shape], dtypes=[rt.dtype])
        if name in UNARY_OPS or name in BINARY_OPS or name in ("where", "matmul", "batch_matmul", "softmax", "identity", "gather"):
            ins = [self.tensor(o) for o in operands]
            return g.add_op(name, ins, {"axis": ins[0].rank - 1} if name == "softmax" else {})
        if name == "compare":
            kind = str(attrs["kind"]).split("<")[-1].strip(">")
            if kind not in COMPARE_KINDS:
                raise LLHSyntaxError("compare kind %r" % kind)
            return g.add_op("compare", [self.tensor(o) for o in operands], {"kind": kind})
        if name == "convert_to":
            return g.add_op("convert_to", [self.tensor(operands[0])], {"dtype": rt.dtype})
        if name in ("conv", "conv_bias"):
            layout = str(attrs.get("layout", "NCHW")).split("<")[-1].strip(">")
            if layout not in ("NCHW", "NHWC"):
                raise NotImplementedError("llh.conv layout %s (NCHW and NHWC are implemented)" % layout)
            wl = str(attrs.get("weight_layout", layout)).split("<")[-1].strip(">")
            if wl not in ({"NCHW": ("NCHW", "FCHW"), "NHWC": ("NHWC", "FHWC")}[layout]):
                raise NotImplementedError("llh.conv weight_layout %s with layout %s" % (wl, layout))
            a = {k: tuple(attrs[k]) for k in ("dilation", "kernel_shape", "pad", "stride")}
            a["group"] = int(attrs.get("group", 1))
            a["layout"] = layout
            return g.add_op(name, [self.tensor(o) for o in operands], a)
        if name == "max_pool":
            a = {k: tuple(attrs[k]) for k in ("dilation", "kernel_shape", "pad", "stride")}
            a.update({"ceil_mode": bool(attrs.get("ceil_mode", False)), "layout": "NCHW"})
            return g.add_op("max_pool", [self.tensor(operands[0])], a)
        if name == "adaptive_average_pool":
            return g.add_op(name, [self.tensor(operands[0])], {"out_size": tuple(attrs["out_size"])})
        if name == "batch_norm_inference":
            return g.add_op(name, [self.tensor(o) for o in operands],
                            {"epsilon": float(attrs["epsilon"]), "momentum": float(attrs.get("momentum", 0.1)),
                             "feature_index": int(attrs.get("feature_index", 1))})
        if name == "layer_norm":
            ins = [self.tensor(o) for o in operands]
            return g.add_op(name, ins, {"epsilon": float(attrs["epsilon"]), "axis": int(attrs.get("axis", -1)),
                                        "has_scale": len(ins) > 1, "has_bias": len(ins) > 2})
        if name in ("reduce_sum", "reduce_max", "reduce_min"):
            return g.add_op(name, [self.tensor(operands[0])], {"axis": tuple(attrs["axis"])})
        if name == "transpose":
            return g.add_op(name, [self.tensor(operands[0])], {"perms": tuple(attrs["perms"])})
        if name in ("reshape", "broadcast_to"):
            x = self.tensor(operands[0])
            shape = tuple(self.scalar(o) for o in operands[1:]) if len(operands) > 1 else tuple(attrs["shape"])
            a = {"shape": shape}
            if name == "broadcast_to":
                a["cast_dims"] = tuple(attrs.get("cast_dims", range(len(shape))))
                if "noexpand_dims" in attrs:
                    a["noexpand_dims"] = tuple(attrs["noexpand_dims"])
                return g.add_op(name, [x], a)
            return g.add_op(name, [x], a, shapes=[_resolve(x, shape)], dtypes=[x.dtype])
        if name == "stride_slice":
            x = self.tensor(operands[0])
            if len(operands) > 1:
                seg = attrs.get("operandSegmentSizes", (1, x.rank, x.rank, x.rank))
                vals = [self.scalar(o) for o in operands[1:]]
                st, en, sp = vals[:seg[1]], vals[seg[1]:seg[1] + seg[2]], vals[seg[1] + seg[2]:]
            else:
                st, en, sp = attrs["start"], attrs["end"], attrs["stride"]
            return g.add_op(name, [x], {"start": tuple(st), "end": tuple(en), "stride": tuple(sp)})
        if name == "extract":
            idx = self.scalar(operands[1]) if len(operands) > 1 else attrs["index"]
            if isinstance(idx, Expr):
                raise NotImplementedError("llh.extract with a symbolic index")
            return g.add_op(name, [self.tensor(operands[0])], {"index": int(idx)})
        if name == "flatten":
            x = self.tensor(operands[0])
            if not rt.ranked:
                raise NotImplementedError("llh.flatten with an unranked result type")
            return g.add_op("reshape", [x], {"shape": tuple(rt.shape)}, shapes=[_resolve(x, tuple(-1 if d is None else d for d in rt.shape))],
                            dtypes=[x.dtype])
        raise NotImplementedError("llh.%s has no reader" % name)

    def statement(self, c):
        results = []
        if c.peek("%"):
            while True:
                m = c.match(r"%([\w.$-]+)(?::\d+)?")
                results.append(m.group(1))
                if not c.take(","):
                    break
            c.expect("=")
        m = c.match(r"(?:arith|index)\.constant\s*(?:\{[^}]*\}\s*)?(-?\d+)(?:\s*:\s*(?:i64|i32|index))?")
        if m:  # the scalar side also appears in MLIR's custom syntax: %c3 = arith.constant 3 : i64
            if results:
                self.env[results[0]] = int(m.group(1))
            return
        m = c.match(r'"([\w.]+)"')
        if not m:
            raise LLHSyntaxError("operation expected at ...%s" % c.s[c.i:c.i + 40].replace("\n", " "))
        full = m.group(1)
        operands = re.findall(r"%([\w.$-]+)", c.bracketed("(", ")"))
        attrs = {}
        if c.peek("<{"):
            c.expect("<")
            attrs.update(_parse_attr_dict(c.bracketed("{", "}")))
            c.expect(">")
        if c.peek("{"):
            attrs.update(_parse_attr_dict(c.bracketed("{", "}")))
        c.expect(":")
        c.bracketed("(", ")")
        c.expect("->")
        if c.peek("("):
            rtypes = _type_list("(" + c.bracketed("(", ")") + ")")
        elif c.peek("tensor"):
            c.match("tensor")
            rtypes = [_parse_type("tensor<" + c.bracketed("<", ">") + ">")]
        else:
            rtypes = [_parse_type(c.match(r"[\w]+").group(0))]
        if not full.startswith("llh."):
            raise NotImplementedError("operation %s (only the llh dialect is read)" % full)
        value = self.emit(full[4:], operands, attrs, rtypes)
        if results:
            # (a printed tensor<f32> for a one-element result is what the importer writes; the reference's
            # legalisation refines it to tensor<1xf32>, Operationlegalization.cpp:152-193)
            scalar_as_1 = isinstance(value, Value) and rtypes and len(rtypes[0].shape) == 0 and tuple(value.shape) == (1,)
            if isinstance(value, Value) and rtypes and rtypes[0].kind == "tensor" and rtypes[0].ranked and not scalar_as_1 and \
                    len(rtypes[0].shape) != value.rank:
                raise LLHSyntaxError("%%%s: printed type has rank %d, inferred rank %d" % (results[0], len(rtypes[0].shape), value.rank))
            self.env[results[0]] = value


def _resolve(x, shape):
    from .infer import resolve_reshape
    return resolve_reshape(x.shape, shape)


def parse_llh(text, func=None, ssa=None):
    """Parses the (first, or named) func.func of `text` into a Graph.  `ssa`, if given, is a dict that is filled with what every
    SSA name of the function stands for (a graph Value, an int, or a symbolic extent)."""
    text = _strip_comments(text)
    pat = r"func\.func\s+(?:private\s+|public\s+)?@(%s)\s*\(" % (re.escape(func) if func else r"[\w.$-]+")
    m = re.search(pat, text)
    if not m:
        raise LLHSyntaxError("no func.func%s found" % (" @" + func if func else ""))
    c = _Cursor(text)
    c.i = m.end() - 1
    r = _Reader()
    for arg in _split_top(c.bracketed("(", ")")):
        am = re.match(r"%([\w.$-]+)\s*:\s*(.*?)(\s*\{.*\})?$", arg, re.S)
        if not am:
            raise LLHSyntaxError("argument %r" % arg)
        ty = _parse_type(am.group(2))
        if am.group(3) and ty.kind == "tensor" and not ty.symbols:
            # {func.input_symbol_0 = "s0", ...}: which symbol every extent of the argument is (fx_translate.py:197-224)
            bound = dict((int(k), v) for k, v in re.findall(r'func\.input_symbol_(\d+)\s*=\s*"([^"]+)"', am.group(3)))
            if bound:
                ty.symbols = [bound.get(k, "") for k in range(len(ty.shape))]
        r.add_argument(am.group(1), ty)
    if c.take("->"):
        if c.peek("("):
            c.bracketed("(", ")")
        elif c.peek("tensor<"):
            c.match("tensor")
            c.bracketed("<", ">")
        else:
            c.match(r"[\w]+")
    if c.take("attributes"):
        c.bracketed("{", "}")
    body = _Cursor(c.bracketed("{", "}"))
    returned = None
    while not body.eof():
        if body.match(r"(func\.)?return\b"):
            names = []
            while body.peek("%"):
                names.append(body.match(r"%([\w.$-]+)").group(1))
                if not body.take(","):
                    break
            if body.take(":"):
                rest = body.s[body.i:]
                body.i = len(body.s) if "\n" not in rest else body.i + rest.index("\n")
            returned = [r.operand(n) for n in names]
            break
        r.statement(body)
    outs = returned if returned else r.printed
    if ssa is not None:
        ssa.update(r.env)
    r.g.set_outputs(list(outs))
    r.g.single_output = len(outs) == 1
    return r.g


# ------------------------------------------------------------------------------------------ printer
def _dim_str(d):
    return "?" if isinstance(d, Expr) else str(d)


def _type_str(v):
    return "tensor<%s%s>" % ("".join(_dim_str(d) + "x" for d in v.shape), DTYPE_NAMES[v.dtype])


def _attr_text(key, v, result):
    if key == "dtype":
        return None  # carried by the result type
    if isinstance(v, bool):
        return "true" if v else "false"
    if isinstance(v, str):
        if key == "kind":
            return "#llh.Compare<%s>" % v
        if key in ("layout", "weight_layout"):
            return "#llh.Layout<%s>" % v
        return '"%s"' % v
    if isinstance(v, (tuple, list)):
        if any(isinstance(x, Expr) for x in v):
            raise NotImplementedError("symbolic extents in attribute %s cannot be printed as constants" % key)
        return "array<i64: %s>" % ", ".join(str(int(x)) for x in v)
    if isinstance(v, float):
        return "%r : f64" % v
    if isinstance(v, int):
        return "%d : i64" % v
    raise NotImplementedError("attribute %s = %r" % (key, v))


_SCALAR_OP_NAMES = {"add": "add", "sub": "sub", "mul": "mul", "floordiv": "div"}


def _print_scalar(e, g, lines, counter):
    """Writes the i64 arithmetic that computes the symbolic value `e` (llh.dim of the argument that carries a
    symbol, llh.torch_symbolic_int for a symbol passed as an int argument, llh.constant, scalar add/sub/mul/div)
    and returns the SSA name of the result."""
    counter[0] += 1
    name = "e%d" % counter[0]
    if isinstance(e, int):
        lines.append('  %%%s = "llh.constant"() <{value = %d : i64}> : () -> i64' % (name, e))
    elif e.kind == "sym" and e.args[0] in g.symbol_sources:
        i, k = g.symbol_sources[e.args[0]]
        c = _print_scalar(k, g, lines, counter)
        lines.append('  %%%s = "llh.dim"(%%%s, %%%s) : (%s, i64) -> i64' % (name, g.inputs[i].name, c, _type_str(g.inputs[i])))
    elif e.kind == "sym":
        lines.append('  %%%s = "llh.torch_symbolic_int"() <{sym_name = "%s"}> : () -> i64' % (name, e.args[0]))
    elif e.kind in _SCALAR_OP_NAMES:
        a, b = (_print_scalar(x, g, lines, counter) for x in e.args)
        lines.append('  %%%s = "llh.%s"(%%%s, %%%s) : (i64, i64) -> i64' % (name, _SCALAR_OP_NAMES[e.kind], a, b))
    else:
        raise NotImplementedError("scalar expression %r has no spelling in llh scalar ops" % (e,))
    return name


def print_llh(g):
    """The graph in generic op syntax; `parse_llh(print_llh(g))` gives an equivalent graph when every attribute is
    static (symbolic reshape / broadcast targets are printed as llh.dim arithmetic only for plain symbols)."""
    lines = []
    counter = [0]
    args = ["%%%s: %s" % (v.name, _type_str(v)) for v in g.inputs]
    outs = [o for o in g.outputs if isinstance(o, Value)]
    lines.append("func.func @main(%s) -> (%s) attributes {entrance} {" % (", ".join(args), ", ".join(_type_str(o) for o in outs)))
    for op in g.ops:
        r = op.results[0]
        if op.name == "scalar_cast":
            src = _print_scalar(op.attrs["value"], g, lines, counter)
            lines.append('  %%%s = "llh.scalar_cast"(%%%s) : (i64) -> %s' % (r.name, src, _type_str(r)))
            continue
        if op.name == "constant":
            val = op.attrs["value"]
            body = "[%s]" % ", ".join(repr(x) for x in val) if isinstance(val, list) else repr(float(val) if r.dtype.is_floating_point else int(val))
            attrs = "value = dense<%s> : %s" % (body, _type_str(r))
        else:
            items = []
            for k in sorted(op.attrs):
                if k in ("has_scale", "has_bias") or (op.name == "softmax" and k == "axis"):
                    continue
                t = _attr_text(k, op.attrs[k], r)
                if t is not None:
                    items.append("%s = %s" % (k, t))
            attrs = ", ".join(items)
        lines.append('  %%%s = "llh.%s"(%s)%s : (%s) -> %s' % (
            r.name, op.name, ", ".join("%" + o.name for o in op.operands), " <{%s}>" % attrs if attrs else "",
            ", ".join(_type_str(o) for o in op.operands), _type_str(r)))
    lines.append("  return %s : %s" % (", ".join("%" + o.name for o in outs), ", ".join(_type_str(o) for o in outs)))
    lines.append("}")
    return "\n".join(lines) + "\n"
