"""LLH graph -> kernel plan.

This is the "LLH -> HIP kernel call" lowering that stands where the reference lowers LLH to
StableHLO/linalg/loops (src/Conversion/LLHToHLO, src/Pipeline/TransformPipeline.cpp:134-226).  The
fusion decisions mirror what the reference's pipeline gets from linalg-fuse-elementwise-ops
(include/llcompiler/TransformLibrary/linalg_include.mlir:50-53): elementwise consumers are fused
into their producers; here additionally into the epilogue of the contraction kernels.

A plan is a list of Steps over graph Values:
  view      reshape / transpose / broadcast_to / stride_slice / extract: descriptor changes only
  ew        one fused elementwise chain (a register program for llc_hip_elementwise)
  matmul / batch_matmul / conv      with epilogue {alpha, bias, residual, act}
  softmax, layer_norm, reduce, max_pool, avg_pool, gather, constant, weight (a .npy file, llh.weight)
"""
import torch

from ..llh.expr import Expr
from ..llh.graph import BINARY_OPS, ELEMENTWISE_OPS, UNARY_OPS, VIEW_OPS, Value

MAX_INPUTS, MAX_REGS, MAX_INSTS = 6, 4, 24
_CMP = {"EQ": "eq", "GE": "ge", "LE": "le", "GT": "gt", "LT": "lt", "NE": "ne"}


class Step:
    __slots__ = ("kind", "inputs", "output", "attrs")

    def __init__(self, kind, inputs, output, attrs=None):
        self.kind, self.inputs, self.output, self.attrs = kind, list(inputs), output, attrs or {}

    def __repr__(self):
        extra = ""
        if self.attrs.get("prepared"):
            extra = " (prepared)"
        if self.kind == "ew":
            extra += " [%s]" % " ".join(i[0] for i in self.attrs["insts"])
        elif self.kind in ("matmul", "batch_matmul", "conv"):
            e = self.attrs["epilogue"]
            parts = [k for k in ("bias", "residual") if e.get(k) is not None]
            if isinstance(e.get("alpha", 1.0), Expr):
                parts.append("alpha=%r" % (e["alpha"],))
            elif e.get("alpha", 1.0) != 1.0:
                parts.append("alpha=%g" % e["alpha"])
            if e.get("act"):
                parts.append(e["act"])
            extra = " {%s}" % ",".join(parts) if parts else ""
        elif self.kind == "view":
            extra += " " + self.attrs["op"]
        return "%s%s(%s) -> %%%s" % (self.kind, extra, ", ".join("%" + v.name for v in self.inputs), self.output.name)


def _strip_views(v):
    """Root of a reshape / broadcast_to chain."""
    chain = []
    while v.producer is not None and v.producer.name in ("reshape", "broadcast_to"):
        chain.append(v.producer)
        v = v.producer.operands[0]
    return v, chain


def _scalar_const(v):
    root, _ = _strip_views(v)
    return root.const if root.const is not None else None


def _numel_static_one(v):
    return all(isinstance(d, int) and d == 1 for d in v.shape)


def _same_extent(a, b):
    return a == b or str(a) == str(b)


class Planner:
    def __init__(self, graph):
        self.g = graph
        self.outputs = set(id(o) for o in graph.outputs if isinstance(o, Value))
        self.absorbed = set()   # ids of ops folded into another step
        self.steps = []

    # ------------------------------------------------------------------ contraction epilogues
    def _is_bias(self, other, out, channel_dim):  # noqa: C901
        """`other` broadcasts a rank-1 tensor of out.shape[channel_dim] along channel_dim."""
        root, chain = _strip_views(other)
        n = out.shape[channel_dim]
        nontrivial = [d for d in root.shape if not (isinstance(d, int) and d == 1)]
        if len(nontrivial) != 1 or nontrivial[0] != n or root.const is not None:
            return None
        # the rank-aligned view must put that extent on channel_dim
        aligned = chain[0].results[0].shape if chain and chain[0].name == "broadcast_to" else other.shape
        for op in chain:
            if op.name == "broadcast_to":
                aligned = op.operands[0].shape
        if len(aligned) != out.rank:
            if len(aligned) < out.rank and channel_dim == out.rank - 1 and len(root.shape) == 1:
                return root
            return None
        for d in range(out.rank):
            is_one = isinstance(aligned[d], int) and aligned[d] == 1
            if d == channel_dim and is_one and not (isinstance(n, int) and n == 1):
                return None
            if d != channel_dim and not is_one:
                return None
        return root

    def match_epilogue(self, op):
        channel_dim = 1 if op.name in ("conv", "conv_bias") and op.attrs.get("layout", "NCHW") == "NCHW" else op.results[0].rank - 1
        epi = {"alpha": 1.0, "bias": None, "residual": None, "act": None}
        if op.name == "conv_bias":
            epi["bias"] = op.operands[2]
        v = op.results[0]
        absorbed, reshaped, last = [], False, op
        while len(v.users) == 1 and id(v) not in self.outputs:
            u = v.users[0]
            if id(u) in self.absorbed:
                break  # already the epilogue of an earlier contraction (e.g. the other branch of a residual add)
            if u.name == "reshape" and epi["act"] is None:
                # a reshape of the contiguous result keeps the linear element order
                nxt = u.results[0]
                if len(nxt.users) == 1 and nxt.users[0].name in ("add", "mul", "div", "relu", "gelu") and id(nxt) not in self.outputs:
                    absorbed.append(u)
                    reshaped = True
                    v = nxt
                    continue
                break
            if u.name in ("mul", "div") and epi["bias"] is None and epi["residual"] is None and epi["act"] is None:
                other = u.operands[1] if u.operands[0] is v else u.operands[0]
                c = _scalar_const(other)
                if c is None or (u.name == "div" and u.operands[0] is not v) or tuple(u.results[0].shape) != tuple(v.shape):
                    break
                c = c if isinstance(c, Expr) else float(c)  # (a symbol-valued scale stays an expression)
                epi["alpha"] = epi["alpha"] * c if u.name == "mul" else epi["alpha"] / c
                absorbed.append(u)
                v = u.results[0]
                continue
            if u.name == "add" and epi["act"] is None and tuple(u.results[0].shape) == tuple(v.shape):
                other = u.operands[1] if u.operands[0] is v else u.operands[0]
                if other is v:
                    break
                bias = None
                if epi["bias"] is None and epi["residual"] is None and not reshaped:
                    bias = self._is_bias(other, v, channel_dim)
                if bias is None and epi["bias"] is None and epi["residual"] is None and reshaped and \
                        op.name == "batch_matmul" and v.rank == 4 and other.rank == 4 and _strip_views(other)[0] is other and \
                        other.dtype == v.dtype and _scalar_const(other) is None and \
                        _same_extent(other.shape[0], v.shape[0]) and _same_extent(other.shape[3], v.shape[3]) and \
                        all(isinstance(other.shape[d], int) and other.shape[d] == 1 for d in (1, 2)):
                    # [B0,1,1,N] added to [B0,B1,M,N] (attention mask): one bias row per outer batch
                    bias = other
                    epi["bias_rows"] = True
                if bias is not None:
                    epi["bias"] = bias
                elif epi["residual"] is None and tuple(other.shape) == tuple(v.shape) and other.dtype == v.dtype and \
                        _scalar_const(other) is None and _strip_views(other)[0] is other:
                    epi["residual"] = other
                else:
                    break
                absorbed.append(u)
                v = u.results[0]
                continue
            if u.name in ("relu", "gelu") and epi["act"] is None:
                epi["act"] = u.name
                absorbed.append(u)
                v = u.results[0]
                continue
            break
        return epi, absorbed, v

    # ------------------------------------------------------------------ elementwise groups
    def _ew_class(self, op):
        dts = [o.dtype for o in op.operands] + [op.results[0].dtype]
        if any(dt.is_floating_point for dt in dts):
            return "float"
        return "int"

    def build_program(self, ops):
        """Register program for a topologically ordered list of elementwise ops whose last op is the output."""
        prog, inputs = self._build_program(ops, None)
        if not inputs:
            # every operand is a one-element constant (a constant expression in LLH text): the kernel wants at
            # least one tensor to read, so the first constant stays a tensor operand
            first = next(o for op in ops for o in op.operands if o.producer is None or o.producer not in ops)
            prog, inputs = self._build_program(ops, id(first))
        return prog, inputs

    def _build_program(self, ops, keep_as_input):
        produced = {id(op.results[0]): i for i, op in enumerate(ops)}
        last_use = {}
        for i, op in enumerate(ops):
            for o in op.operands:
                if id(o) in produced:
                    last_use[id(o)] = i
        inputs, in_index = [], {}
        reg_of, free = {}, list(range(MAX_REGS))
        insts = []
        integer = all(self._ew_class(op) == "int" for op in ops)

        def operand(o):
            if id(o) in produced:
                return "r%d" % reg_of[id(o)]
            c = _scalar_const(o) if id(o) != keep_as_input else None
            if isinstance(c, Expr):
                return c  # a symbol-valued immediate: the engine puts in the number per binding
            if c is not None:
                return float(c) if not isinstance(c, bool) else float(int(c))
            if id(o) not in in_index:
                if len(inputs) >= MAX_INPUTS:
                    raise OverflowError("inputs")
                in_index[id(o)] = len(inputs)
                inputs.append(o)
            return "in%d" % in_index[id(o)]

        for i, op in enumerate(ops):
            srcs = [operand(o) for o in op.operands]
            # registers whose last use is this instruction can be overwritten by its result
            for o in op.operands:
                if id(o) in produced and last_use.get(id(o)) == i and reg_of[id(o)] not in free:
                    free.append(reg_of[id(o)])
            imms = [s for s in srcs if not isinstance(s, str)]
            while len(imms) > 1:
                # one immediate per instruction: park extra constants in registers first
                if not free:
                    raise OverflowError("registers")
                k = max(j for j, s in enumerate(srcs) if not isinstance(s, str))
                r = free.pop(0)
                insts.append(("mov", "r%d" % r, srcs[k]))
                srcs[k] = "r%d" % r
                imms = [s for s in srcs if not isinstance(s, str)]
                free.append(r)  # only needed by this instruction
            if not free:
                raise OverflowError("registers")
            free.sort()
            dst = free.pop(0)
            reg_of[id(op.results[0])] = dst
            if op.name == "compare":
                insts.append((_CMP[op.attrs["kind"]], "r%d" % dst, *srcs))
            elif op.name == "convert_to":
                insts.append(("mov", "r%d" % dst, *srcs))
            else:
                insts.append((op.name, "r%d" % dst, *srcs))
            if len(insts) > MAX_INSTS:
                raise OverflowError("instructions")
        return {"insts": insts, "result": "r%d" % reg_of[id(ops[-1].results[0])], "integer": integer}, inputs

    def group_elementwise(self, ops):
        """Greedy producer->consumer fusion.  Returns {id(last op): [ops of the group]}; member ops other
        than the last are marked absorbed."""
        group = {}   # id(op) -> list of ops (the group that op currently terminates)
        for op in ops:
            if op.name not in ELEMENTWISE_OPS or id(op) in self.absorbed:
                continue
            members = []
            out_shape = tuple(op.results[0].shape)
            cls = self._ew_class(op)
            for o in op.operands:
                p = o.producer
                if p is None or id(p) not in group or id(o) in self.outputs or len(o.users) != 1:
                    continue
                if tuple(o.shape) != out_shape or self._ew_class(p) != cls:
                    continue
                if (p in self.g.prepared) != (op in self.g.prepared):
                    continue  # derived weights are computed once per instance, the rest on every call
                cand = members + [m for m in group[id(p)] if m not in members]
                try:
                    self.build_program(cand + [op])
                except OverflowError:
                    continue
                members = cand
            for m in members:
                group.pop(id(m), None)
                self.absorbed.add(id(m))
            group[id(op)] = members + [op]
        return group

    # ------------------------------------------------------------------ driver
    def plan(self):
        g = self.g
        fused_at = {}   # id(last absorbed op) -> Step to emit there
        for op in g.ops:
            if op.name in ("matmul", "batch_matmul", "conv", "conv_bias"):
                epi, absorbed, out = self.match_epilogue(op)
                kind = "conv" if op.name.startswith("conv") else op.name
                attrs = {"epilogue": epi}
                if kind == "conv":
                    attrs.update({k: op.attrs[k] for k in ("dilation", "kernel_shape", "pad", "stride", "group")})
                    attrs["layout"] = op.attrs.get("layout", "NCHW")
                step = Step(kind, op.operands[:2], out, attrs)
                step.attrs["natural_shape"] = tuple(op.results[0].shape)
                self.absorbed.add(id(op))
                for a in absorbed:
                    self.absorbed.add(id(a))
                fused_at[id(absorbed[-1] if absorbed else op)] = step
        groups = self.group_elementwise(g.ops)
        for op in g.ops:
            if id(op) in fused_at:
                self.steps.append(fused_at[id(op)])
                continue
            if id(op) in self.absorbed:
                continue
            r = op.results[0]
            if op.name in ELEMENTWISE_OPS:
                prog, inputs = self.build_program(groups[id(op)])
                if all(m in g.prepared for m in groups[id(op)]):
                    prog["prepared"] = True
                self.steps.append(Step("ew", inputs, r, prog))
            elif op.name in VIEW_OPS:
                self.steps.append(Step("view", op.operands[:1], r, dict(op.attrs, op=op.name)))
                if op in g.prepared:
                    self.steps[-1].attrs["prepared"] = True
            elif op.name in ("constant", "scalar_cast"):
                self.steps.append(Step("constant", [], r, {"value": op.attrs["value"]}))
            elif op.name == "weight":
                self.steps.append(Step("weight", [], r, {"weight_file": op.attrs["weight_file"]}))
            elif op.name == "softmax":
                self.steps.append(Step("softmax", op.operands, r))
            elif op.name == "layer_norm":
                self.steps.append(Step("layer_norm", op.operands, r, dict(op.attrs)))
            elif op.name in ("reduce_sum", "reduce_max", "reduce_min"):
                self.steps.append(Step("reduce", op.operands, r, {"kind": op.name[7:], "axis": tuple(op.attrs["axis"])}))
            elif op.name == "max_pool":
                self.steps.append(Step("max_pool", op.operands, r, dict(op.attrs)))
            elif op.name == "adaptive_average_pool":
                if tuple(op.attrs["out_size"]) != (1, 1):
                    raise NotImplementedError("adaptive_average_pool to %s" % (op.attrs["out_size"],))
                self.steps.append(Step("avg_pool", op.operands, r))
            elif op.name == "gather":
                self.steps.append(Step("gather", op.operands, r))
            else:
                raise NotImplementedError("no kernel lowering for llh.%s" % op.name)
        return self.steps


def make_plan(graph):
    return Planner(graph).plan()
