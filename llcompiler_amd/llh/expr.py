"""Symbolic extents: small integer expression trees over named symbols ("s0", "s1", ...).

This is the host-side stand-in for the reference's symbol system (SymEngine expressions attached
to tensor dims, src/Dialect/LLH/SymbolInfer/): every dynamic dim of a graph value is an `Expr`,
and the executor evaluates it with the symbol values bound at call time.  The node kinds are the
ones the reference's run-time evaluator handles (llcompiler/executor/out_put_call.py:21-48: Add,
Mul, FloorDiv, Pow, Symbol, Number) plus CeilDiv (the affine maps of
src/Dialect/LLH/IR/LLHinfersymbolShape.cpp:281-288), Sub, Max and Min.

A symbol may also be a scalar OPERAND of a tensor op (`x / x.shape[0]`, `scores / sqrt(d)`): the reference casts
the i64 value to a one-element tensor with llh.scalar_cast (include/llcompiler/Dialect/LLH/IR/LLHOps.td:120-127,
lowered to a fill at src/Conversion/LLHToLinalg/LLHToLinalg.cpp:67-88) after computing it with scalar arithmetic
(src/Conversion/LLHToArith/LLHToArith.cpp:112-144).  For that use the trees also carry real-valued nodes:
TrueDiv, Sqrt, Float, Neg and Pow with any exponent; `is_float` tells the two kinds of tree apart and `evaluate`
returns a Python float for them.
"""
import math
from functools import reduce as _reduce

_NUM = (int, float)


class Expr:
    __slots__ = ("kind", "args")

    def __init__(self, kind, args):
        self.kind, self.args = kind, tuple(args)

    # ---- construction ----
    @staticmethod
    def sym(name):
        return Expr("sym", (name,))

    def _bin(self, kind, other, swap=False):
        a, b = (other, self) if swap else (self, other)
        return simplify(Expr(kind, (a, b)))

    def __add__(self, o): return self._bin("add", o)
    def __radd__(self, o): return self._bin("add", o, True)
    def __sub__(self, o): return self._bin("sub", o)
    def __rsub__(self, o): return self._bin("sub", o, True)
    def __mul__(self, o): return self._bin("mul", o)
    def __rmul__(self, o): return self._bin("mul", o, True)
    def __floordiv__(self, o): return self._bin("floordiv", o)
    def __rfloordiv__(self, o): return self._bin("floordiv", o, True)
    def __truediv__(self, o): return self._bin("truediv", o)
    def __rtruediv__(self, o): return self._bin("truediv", o, True)
    def __pow__(self, o): return self._bin("pow", o)
    def __rpow__(self, o): return self._bin("pow", o, True)
    def __neg__(self): return simplify(Expr("neg", (self,)))

    def __eq__(self, other):
        if isinstance(other, Expr):
            return self.kind == other.kind and self.args == other.args
        return False

    def __hash__(self):
        return hash((self.kind, self.args))

    def __repr__(self):
        if self.kind == "sym":
            return self.args[0]
        op = {"add": "+", "sub": "-", "mul": "*", "floordiv": "//", "truediv": "/"}.get(self.kind)
        if op:
            return "(%r %s %r)" % (self.args[0], op, self.args[1])
        return "%s(%s)" % (self.kind, ", ".join(repr(a) for a in self.args))

    def symbols(self):
        if self.kind == "sym":
            return {self.args[0]}
        out = set()
        for a in self.args:
            if isinstance(a, Expr):
                out |= a.symbols()
        return out


def ceildiv(a, b):
    if isinstance(a, int) and isinstance(b, int):
        return -(-a // b)
    return simplify(Expr("ceildiv", (a, b)))


def emax(a, b):
    if isinstance(a, int) and isinstance(b, int):
        return max(a, b)
    return a if a == b else Expr("max", (a, b))


def sqrt(a):
    """torch._sym_sqrt of a symbolic value."""
    return math.sqrt(a) if isinstance(a, _NUM) else Expr("sqrt", (a,))


def to_float(a):
    """torch.sym_float of a symbolic value."""
    return float(a) if isinstance(a, _NUM) else Expr("float", (a,))


def is_float(e):
    """Whether the value of `e` is a real number rather than an integer."""
    if isinstance(e, float):
        return True
    if not isinstance(e, Expr) or e.kind == "sym":
        return False
    if e.kind in ("truediv", "sqrt", "float"):
        return True
    if e.kind == "pow" and not (isinstance(e.args[1], int) and e.args[1] >= 0):
        return True
    return any(is_float(a) for a in e.args)


def _affine(e, scale, terms, order):
    """Adds scale * e to the integer-affine form (terms: atom -> coefficient, terms[None]: the constant); returns
    False when e holds a float constant (real-valued trees are left as they are written)."""
    if isinstance(e, int):
        terms[None] = terms.get(None, 0) + scale * e
        return True
    if not isinstance(e, Expr):
        return False
    if e.kind in ("add", "sub"):
        return _affine(e.args[0], scale, terms, order) and _affine(e.args[1], scale if e.kind == "add" else -scale, terms, order)
    if e.kind == "mul" and isinstance(e.args[0], int):
        return _affine(e.args[1], scale * e.args[0], terms, order)
    if e.kind == "mul" and isinstance(e.args[1], int):
        return _affine(e.args[0], scale * e.args[1], terms, order)
    if e not in terms:
        order.append(e)
    terms[e] = terms.get(e, 0) + scale
    return True


def _normal_sum(e):
    """An integer sum / difference / multiple in one canonical form: atoms in order of first appearance, each with
    its collected coefficient, then the collected constant.  (H + 2) - 3 + 1 becomes H, so that the extent of a
    padded stride-1 window equals the extent it was computed from, structurally.)"""
    terms, order = {}, []
    if is_float(e) or not _affine(e, 1, terms, order):
        return e
    out = None
    for atom in order:
        c = terms[atom]
        if c == 0:
            continue
        t = atom if c == 1 else Expr("mul", (c, atom))
        out = t if out is None else Expr("add", (out, t))
    c = terms.get(None, 0)
    if out is None:
        return c
    if c > 0:
        return Expr("add", (out, c))
    if c < 0:
        return Expr("sub", (out, -c))
    return out


def simplify(e):
    if not isinstance(e, Expr) or e.kind == "sym":
        return e
    a = [simplify(x) for x in e.args]
    if all(isinstance(x, _NUM) for x in a):
        return evaluate(Expr(e.kind, a), {})
    k = e.kind
    if k in ("add", "sub") or (k == "mul" and (isinstance(a[0], int) or isinstance(a[1], int))):
        return _normal_sum(Expr(k, a))
    if k == "add":
        if a[0] == 0: return a[1]
        if a[1] == 0: return a[0]
    if k == "sub" and a[1] == 0:
        return a[0]
    if k == "sub" and a[0] == a[1]:
        return 0
    if k == "mul":
        if a[0] == 1: return a[1]
        if a[1] == 1: return a[0]
        if a[0] == 0 or a[1] == 0: return 0
    if k in ("floordiv", "ceildiv") and a[1] == 1:
        return a[0]
    return Expr(k, a)


def evaluate(e, env):
    """Value of `e` with symbols bound by `env` (name -> int): an int for extents, a float for the real-valued
    trees of scalar operands."""
    if isinstance(e, _NUM):
        return e
    k, a = e.kind, e.args
    if k == "sym":
        try:
            return int(env[a[0]])
        except KeyError:
            raise KeyError("symbol %s is not bound by any input of this call" % a[0])
    x = evaluate(a[0], env)
    if k == "sqrt": return math.sqrt(x)
    if k == "float": return float(x)
    if k == "neg": return -x
    y = evaluate(a[1], env)
    if k == "pow": return x ** y
    if k == "truediv": return x / y
    if k == "add": return x + y
    if k == "sub": return x - y
    if k == "mul": return x * y
    if k == "floordiv": return x // y
    if k == "ceildiv": return -(-x // y)
    if k == "max": return max(x, y)
    if k == "min": return min(x, y)
    raise NotImplementedError(k)


def product(dims):
    return _reduce(lambda x, y: x * y, dims, 1)


def from_sympy(expr):
    """Converts the sympy expression behind a torch SymInt (the same node kinds as
    llcompiler/executor/out_put_call.py:21-48)."""
    import sympy
    if isinstance(expr, (int,)):
        return expr
    if isinstance(expr, sympy.Integer):
        return int(expr)
    if isinstance(expr, sympy.Symbol):
        return Expr.sym(expr.name)
    name = type(expr).__name__
    if isinstance(expr, sympy.Add):
        return _reduce(lambda x, y: x + y, [from_sympy(a) for a in expr.args])
    if isinstance(expr, sympy.Mul):
        return _reduce(lambda x, y: x * y, [from_sympy(a) for a in expr.args])
    if name in ("FloorDiv", "CleanDiv", "PythonFloorDiv", "IntTrueDiv"):
        return from_sympy(expr.args[0]) // from_sympy(expr.args[1])
    if name == "CeilDiv":
        return ceildiv(from_sympy(expr.args[0]), from_sympy(expr.args[1]))
    if isinstance(expr, sympy.Pow) and isinstance(expr.args[1], sympy.Integer) and int(expr.args[1]) >= 0:
        return simplify(Expr("pow", (from_sympy(expr.args[0]), int(expr.args[1]))))
    if name == "Max":
        return _reduce(emax, [from_sympy(a) for a in expr.args])
    raise NotImplementedError("symbolic extent %r (%s)" % (expr, name))
