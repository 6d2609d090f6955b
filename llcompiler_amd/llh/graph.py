"""The LLH graph: op names, attributes and shape rules of the reference's `llh` dialect
(include/llcompiler/Dialect/LLH/IR/LLHOps.td), held as a small Python IR instead of MLIR.

A Graph is what the importer produces from an FX graph and what the planner lowers to kernel
calls.  Dynamic dims are `Expr`s over named symbols; `Graph.dump()` prints the reference's generic
op syntax (`%3 = "llh.add"(%1, %2) : (tensor<?x10xf32>, ...) -> ...`) so that pass-level tests can
check op sequences the way the reference's FileCheck tests do.
"""
import torch

from .expr import Expr, ceildiv, product  # noqa: F401

DTYPE_NAMES = {torch.float32: "f32", torch.bfloat16: "bf16", torch.float16: "f16", torch.int64: "i64",
               torch.int32: "i32", torch.bool: "i1", torch.int8: "i8", torch.float64: "f64"}

UNARY_OPS = ("abs", "sqrt", "exp", "relu", "rsqrt", "neg", "gelu", "tanh", "erf", "sigmoid", "log", "recip")
BINARY_OPS = ("add", "sub", "mul", "div", "max", "min", "pow")
ELEMENTWISE_OPS = UNARY_OPS + BINARY_OPS + ("compare", "where", "convert_to")
VIEW_OPS = ("reshape", "transpose", "broadcast_to", "stride_slice", "extract", "flatten", "identity")
COMPARE_KINDS = ("EQ", "GE", "LE", "GT", "LT", "NE")  # LLHEnums.td:111-116


class Value:
    __slots__ = ("name", "shape", "dtype", "producer", "users", "const")

    def __init__(self, name, shape, dtype, producer=None, const=None):
        self.name, self.shape, self.dtype, self.producer = name, tuple(shape), dtype, producer
        self.users = []
        self.const = const  # python scalar for llh.constant of one element, else None

    @property
    def rank(self):
        return len(self.shape)

    def is_static(self):
        return all(isinstance(d, int) for d in self.shape)

    def type_str(self):
        dims = "x".join("?" if isinstance(d, Expr) else str(d) for d in self.shape)
        return "tensor<%s%s%s>" % (dims, "x" if self.shape else "", DTYPE_NAMES.get(self.dtype, str(self.dtype)))

    def __repr__(self):
        return "%%%s: %s" % (self.name, self.type_str())


class Op:
    __slots__ = ("name", "operands", "attrs", "results")

    def __init__(self, name, operands, attrs, results):
        self.name, self.operands, self.attrs, self.results = name, list(operands), dict(attrs), list(results)

    @property
    def result(self):
        return self.results[0]

    def __repr__(self):
        attrs = ""
        if self.attrs:
            attrs = " <{%s}>" % ", ".join("%s = %s" % (k, _attr_str(v)) for k, v in sorted(self.attrs.items()))
        return '%s = "llh.%s"(%s)%s : (%s) -> %s' % (
            ", ".join("%" + r.name for r in self.results), self.name, ", ".join("%" + o.name for o in self.operands), attrs,
            ", ".join(o.type_str() for o in self.operands), ", ".join(r.type_str() for r in self.results))


def _attr_str(v):
    if isinstance(v, (list, tuple)):
        return "array<i64: %s>" % ", ".join(str(x) for x in v)
    if isinstance(v, torch.dtype):
        return DTYPE_NAMES.get(v, str(v))
    return repr(v)


class Graph:
    """func @main {entrance}: inputs (tensors and leading int symbols), ops in topological order, outputs."""

    def __init__(self):
        self.inputs = []          # Values, in call order (tensor placeholders)
        self.symbol_args = []     # names of symbols passed as leading python ints (symbol_int_arg_nums)
        self.arg_kinds = []       # per positional call argument: ("tensor", index) | ("symbol", name) | ("none", None)
        self.ops = []
        self.outputs = []         # Values, Exprs/ints (symbolic int results) or None
        self.symbol_sources = {}  # symbol name -> (input index, dim): llh.torch_symbolic_int -> llh.dim(arg, k)
        self.single_output = False
        self.prepared = set()     # ops that compute derived weights (batch norm folded into filters): run per instance, not per call
        self._n = 0

    # ---- construction ----
    def _fresh(self, prefix="v"):
        self._n += 1
        return "%s%d" % (prefix, self._n)

    def add_input(self, shape, dtype, name=None):
        v = Value(name or self._fresh("arg"), shape, dtype)
        self.inputs.append(v)
        self.arg_kinds.append(("tensor", len(self.inputs) - 1))
        # func.input_symbol_k attributes (llcompiler/importer/fx_translate.py:197-215): the first input
        # dim that is exactly a symbol is where that symbol's run-time value is read
        for k, d in enumerate(v.shape):
            if isinstance(d, Expr) and d.kind == "sym" and d.args[0] not in self.symbol_sources:
                self.symbol_sources[d.args[0]] = (len(self.inputs) - 1, k)
        return v

    def add_symbol_arg(self, name):
        self.symbol_args.append(name)
        self.arg_kinds.append(("symbol", name))

    def add_op(self, name, operands, attrs=None, shapes=None, dtypes=None, const=None):
        from .infer import infer
        attrs = attrs or {}
        if shapes is None:
            shapes, inferred_dtypes = infer(name, operands, attrs)
            dtypes = dtypes or inferred_dtypes
        results = [Value(self._fresh(), s, d) for s, d in zip(shapes, dtypes)]
        op = Op(name, operands, attrs, results)
        for r in results:
            r.producer = op
        if const is not None:
            results[0].const = const
        for o in operands:
            o.users.append(op)
        self.ops.append(op)
        return results[0] if len(results) == 1 else results

    def constant(self, value, dtype=torch.float32):
        """Scalar constants are tensor<1xT>, as in the reference (llcompiler/importer/fx_translate.py:274-282)."""
        return self.add_op("constant", [], {"value": value}, shapes=[(1,)], dtypes=[dtype], const=value)

    def set_outputs(self, values):
        self.outputs = list(values)

    # ---- rewriting helpers ----
    def replace_all_uses(self, old, new):
        for op in list(old.users):
            op.operands = [new if o is old else o for o in op.operands]
            new.users.append(op)
        old.users = []
        self.outputs = [new if o is old else o for o in self.outputs]

    def erase(self, op):
        for o in op.operands:
            if op in o.users:
                o.users.remove(op)
        self.ops.remove(op)

    def dead_code_eliminate(self):
        live = set(id(o) for o in self.outputs if isinstance(o, Value))
        changed = True
        while changed:
            changed = False
            for op in reversed(list(self.ops)):
                if not any(r.users or id(r) in live for r in op.results):
                    self.erase(op)
                    changed = True

    def symbols(self):
        out = set()
        for v in self.inputs:
            for d in v.shape:
                if isinstance(d, Expr):
                    out |= d.symbols()
        return out | set(self.symbol_args)

    def dump(self):
        lines = ["func.func @main(%s) attributes {entrance, symbol_int_arg_nums = %d}" % (
            ", ".join(repr(v) for v in self.inputs), len(self.symbol_args))]
        lines += ["  " + repr(op) for op in self.ops]
        lines.append("  return %s" % ", ".join("%" + o.name if isinstance(o, Value) else repr(o) for o in self.outputs))
        return "\n".join(lines)

    def op_names(self):
        return [op.name for op in self.ops]
