"""LLH-level rewrites run before kernel planning.  Counterparts of the reference's
src/Dialect/LLH/Transforms passes and canonicalisers, on the Python graph:

  canonicalize           no-op reshape / broadcast / convert / identity folds, abs(abs x), reshape of a constant,
                         x*1, x/1, x+0, 0+x, x-0, c-c (LLHCanonicalize.cpp:378-455, LLHFolder.cpp:33-330).  x*0 is not
                         folded (the reference does): the product is NaN where x is NaN or infinite
  decompose_batch_norm   batch_norm_inference -> add, sqrt, reshape, broadcast_to x4, sub, mul, div, add
                         (DecomposeOps.cpp:110-148; op order pinned by test/Dialect/LLH/decompose_ops.mlir:10-20)
  fold_batch_norm        conv / conv_bias -> batch_norm_inference whose parameters are weights  ==>  conv_bias on
                         w * scale / sqrt(var + eps) and (b - mean) * scale / sqrt(var + eps) + bias: the same
                         affine map as the decomposition (DecomposeOps.cpp:139-144) applied to the filters instead
                         of to every output element; the folded filters are computed by ops marked as prepared
  fuse_softmax           reduce_max -> sub -> exp -> reduce_sum -> div  ==>  softmax
                         (the group ATen _softmax decomposes to, torch_compile_config.py:24)
"""
import torch

from .expr import Expr, is_float
from .graph import BINARY_OPS, Value


def _is_const(v, value=None):
    if not isinstance(v, Value) or v.const is None:
        return False
    if isinstance(v.const, Expr):
        return value is None
    return value is None or float(v.const) == float(value)


def _through_broadcast(v):
    """Looks through reshape / broadcast_to of a one-element constant."""
    while v.producer is not None and v.producer.name in ("reshape", "broadcast_to") and v.const is None:
        v = v.producer.operands[0]
    return v


def _splat(v):
    """The value every element of v has when v is a constant filled with one number (seen through reshape and
    broadcast_to), else None."""
    v = _through_broadcast(v)
    if isinstance(v.const, Expr):
        return None  # a symbol-valued scalar: known per binding only
    if v.const is not None:
        return float(v.const)
    if v.producer is not None and v.producer.name == "constant" and not isinstance(v.producer.attrs.get("value"), (list, tuple)):
        return float(v.producer.attrs["value"])
    return None


def _static(shape):
    return all(isinstance(d, int) for d in shape)


def canonicalize(g):
    changed = True
    while changed:
        changed = False
        for op in list(g.ops):
            r = op.results[0]
            rep = None
            if op.name == "identity":
                rep = op.operands[0]
            elif op.name == "convert_to" and op.attrs["dtype"] == op.operands[0].dtype:
                rep = op.operands[0]
            elif op.name == "convert_to" and op.operands[0].producer is not None and \
                    op.operands[0].producer.name == "scalar_cast" and \
                    (op.attrs["dtype"].is_floating_point or not is_float(op.operands[0].const)):
                # llh.convert_to of llh.scalar_cast (what the importer writes for a symbol-valued operand,
                # fx_translate.py:309-323): the cast produces the wanted element type directly
                src = op.operands[0].producer
                idx = g.ops.index(op)
                tail = g.ops[idx:]
                del g.ops[idx:]
                rep = g.add_op("scalar_cast", [], dict(src.attrs), shapes=[tuple(r.shape)], dtypes=[op.attrs["dtype"]],
                               const=src.attrs["value"])
                g.ops += tail
            elif op.name in ("reshape", "broadcast_to") and tuple(op.operands[0].shape) == tuple(r.shape):
                rep = op.operands[0]
            elif op.name == "reshape" and op.operands[0].producer is not None and op.operands[0].producer.name == "reshape":
                # reshape(reshape(x)) -> reshape(x)
                src = op.operands[0].producer.operands[0]
                op.operands[0].users.remove(op)
                op.operands[0] = src
                src.users.append(op)
                changed = True
                continue
            elif op.name == "broadcast_to" and op.operands[0].rank == r.rank and \
                    sorted(op.attrs.get("noexpand_dims", ())) == list(range(r.rank)):
                # the importer's hint that no dim expands (LLHCanonicalize.cpp: fold of broadcast_to, pinned by
                # test/Dialect/LLH/canonicalize.mlir fold_broadcast)
                rep = op.operands[0]
            elif op.name == "transpose" and tuple(op.attrs["perms"]) == tuple(range(r.rank)):
                rep = op.operands[0]
            elif op.name == "transpose" and op.operands[0].producer is not None and op.operands[0].producer.name == "transpose":
                # transpose(transpose(x, p), q) -> transpose(x, p o q): what the layout transform leaves between two
                # convolutions that follow each other cancels this way
                inner = op.operands[0].producer
                src = inner.operands[0]
                op.attrs = dict(op.attrs, perms=tuple(inner.attrs["perms"][q] for q in op.attrs["perms"]))
                op.operands[0].users.remove(op)
                op.operands[0] = src
                src.users.append(op)
                changed = True
                continue
            elif op.name == "abs" and op.operands[0].producer is not None and op.operands[0].producer.name == "abs":
                rep = op.operands[0]      # abs(abs(x)) (canonicalize.mlir fold_two_abs)
            elif op.name == "reshape" and _static(r.shape) and op.operands[0].producer is not None and \
                    op.operands[0].producer.name == "constant" and op.operands[0].const is None and \
                    not isinstance(op.operands[0].producer.attrs["value"], (list, tuple)):
                # reshape of a constant filled with one value is that constant in the new shape (fold_reshape)
                idx = g.ops.index(op)
                tail = g.ops[idx:]
                del g.ops[idx:]
                rep = g.add_op("constant", [], {"value": op.operands[0].producer.attrs["value"]}, shapes=[tuple(r.shape)], dtypes=[r.dtype])
                g.ops += tail
            elif op.name == "reshape" and _static(r.shape) and op.operands[0].producer is not None and \
                    op.operands[0].producer.name == "constant" and isinstance(op.operands[0].producer.attrs["value"], (list, tuple)):
                idx = g.ops.index(op)
                tail = g.ops[idx:]
                del g.ops[idx:]
                rep = g.add_op("constant", [], {"value": list(op.operands[0].producer.attrs["value"])}, shapes=[tuple(r.shape)], dtypes=[r.dtype])
                g.ops += tail
            elif op.name == "sub" and op.operands[0] is op.operands[1] and _static(r.shape) and r.dtype.is_floating_point and \
                    _splat(op.operands[0]) is not None:
                # c - c for a constant c (fold.mlir sub_same_fold; for a general x the difference is NaN where x is)
                idx = g.ops.index(op)
                tail = g.ops[idx:]
                del g.ops[idx:]
                rep = g.add_op("constant", [], {"value": 0.0}, shapes=[tuple(r.shape)], dtypes=[r.dtype])
                g.ops += tail
            elif op.name in ("add", "sub", "mul", "div") and r.dtype == torch.float32 and _static(r.shape) and \
                    all(o.producer is not None and o.producer.name == "constant" and tuple(o.shape) == tuple(r.shape)
                        for o in op.operands) and _splat(op.operands[0]) is not None and _splat(op.operands[1]) is not None and \
                    not (op.name == "div" and _splat(op.operands[1]) == 0.0):
                # two constants filled with one value each: the result is such a constant (fold.mlir mul_fold, div_fold),
                # computed in fp32 like the kernel would
                import numpy as np
                a, b = np.float32(_splat(op.operands[0])), np.float32(_splat(op.operands[1]))
                val = a + b if op.name == "add" else a - b if op.name == "sub" else a * b if op.name == "mul" else a / b
                idx = g.ops.index(op)
                tail = g.ops[idx:]
                del g.ops[idx:]
                rep = g.add_op("constant", [], {"value": float(val)}, shapes=[tuple(r.shape)], dtypes=[r.dtype])
                g.ops += tail
            elif op.name == "add" and _splat(op.operands[0]) == 0.0 and \
                    tuple(op.operands[1].shape) == tuple(r.shape) and op.operands[1].dtype == r.dtype:
                rep = op.operands[1]
            elif op.name in ("mul", "div") and _splat(op.operands[1]) == 1.0 and \
                    tuple(op.operands[0].shape) == tuple(r.shape) and op.operands[0].dtype == r.dtype:
                rep = op.operands[0]
            elif op.name == "mul" and _splat(op.operands[0]) == 1.0 and \
                    tuple(op.operands[1].shape) == tuple(r.shape) and op.operands[1].dtype == r.dtype:
                rep = op.operands[1]
            elif op.name in ("add", "sub") and _splat(op.operands[1]) == 0.0 and \
                    tuple(op.operands[0].shape) == tuple(r.shape) and op.operands[0].dtype == r.dtype:
                rep = op.operands[0]
            if rep is not None:
                g.replace_all_uses(r, rep)
                g.erase(op)
                changed = True
        g.dead_code_eliminate()
    return g


def decompose_batch_norm(g):
    """scale * (input - mean) / sqrt(var + eps) + bias with per-channel reshape + broadcast_to."""
    for op in list(g.ops):
        if op.name != "batch_norm_inference":
            continue
        x, scale, bias, mean, var = op.operands
        idx = g.ops.index(op)
        tail = g.ops[idx:]
        del g.ops[idx:]
        feature = op.attrs.get("feature_index", 1)
        eps = g.constant(op.attrs["epsilon"], var.dtype)
        fined = g.add_op("add", [var, eps])
        stddev = g.add_op("sqrt", [fined])
        aligned = tuple(x.shape[d] if d == feature else 1 for d in range(x.rank))

        def expand(v):
            r = g.add_op("reshape", [v], {"shape": aligned}, shapes=[aligned], dtypes=[v.dtype])
            return g.add_op("broadcast_to", [r], {"shape": tuple(x.shape), "cast_dims": tuple(range(x.rank))})

        m, s, b, sd = expand(mean), expand(scale), expand(bias), expand(stddev)
        res = g.add_op("sub", [x, m])
        res = g.add_op("mul", [res, s])
        res = g.add_op("div", [res, sd])
        res = g.add_op("add", [res, b])
        g.ops += [t for t in tail if t is not op]
        g.replace_all_uses(op.results[0], res)
        for o in op.operands:
            if op in o.users:
                o.users.remove(op)
    return g


def _weight_like(v, depth=0):
    """A graph input, an llh.weight / llh.constant, or a view of one: a value that does not depend on activations
    computed by the graph (parameters and buffers of the module)."""
    if v.producer is None:
        return True
    if v.producer.name in ("weight", "constant"):
        return True
    if v.producer.name in ("reshape", "broadcast_to", "transpose", "identity") and depth < 8:
        return _weight_like(v.producer.operands[0], depth + 1)
    return False


def fold_batch_norm(g):
    """Eval-mode batch norm behind a convolution becomes part of the convolution's filters and bias.

    batch_norm_inference(conv(x, w[, b]), scale, bias, mean, var) = conv_bias(x, w', b') with
        k = scale / sqrt(var + eps),  w'[f, ...] = w[f, ...] * k[f],  b' = (b - mean) * k + bias,
    which is DecomposeOps.cpp:139-144's scale * (y - mean) / sqrt(var + eps) + bias with the per-filter factor moved
    through the sum.  Done when the convolution's result has no other reader and the filters and all four
    batch-norm parameters are weights (graph inputs, llh.weight, constants): the ops that compute w' and b' are
    marked in `g.prepared`, which tells the planner and the engine to run them when a plan instance is made
    (and again when a parameter's address or version changes), not on every call."""
    prepared = getattr(g, "prepared", None)
    if prepared is None:
        prepared = g.prepared = set()
    outputs = set(id(o) for o in g.outputs if isinstance(o, Value))
    for op in list(g.ops):
        if op.name != "batch_norm_inference" or op not in g.ops:
            continue
        y, scale, bias, mean, var = op.operands
        conv = y.producer
        if conv is None or conv.name not in ("conv", "conv_bias") or len(y.users) != 1 or id(y) in outputs:
            continue
        feature = op.attrs.get("feature_index", 1) % y.rank
        if feature != (y.rank - 1 if conv.attrs.get("layout", "NCHW") == "NHWC" else 1):
            continue
        w = conv.operands[1]
        b = conv.operands[2] if conv.name == "conv_bias" else None
        params = [w, scale, bias, mean, var] + ([b] if b is not None else [])
        if not all(_weight_like(p) and p.is_static() for p in params):
            continue
        if any(p.dtype != w.dtype for p in params) or not w.dtype.is_floating_point:
            continue
        idx = g.ops.index(conv)
        tail = g.ops[idx:]
        del g.ops[idx:]
        first_new = len(g.ops)
        f = w.shape[0]
        eps = g.constant(op.attrs["epsilon"], var.dtype)
        k = g.add_op("div", [scale, g.add_op("sqrt", [g.add_op("add", [var, eps])])])
        per_filter = (f,) + (1,) * (w.rank - 1)
        kw = g.add_op("reshape", [k], {"shape": per_filter}, shapes=[per_filter], dtypes=[k.dtype])
        kw = g.add_op("broadcast_to", [kw], {"shape": tuple(w.shape), "cast_dims": tuple(range(w.rank))})
        w2 = g.add_op("mul", [w, kw])
        shifted = g.add_op("sub", [b, mean]) if b is not None else g.add_op("neg", [mean])
        b2 = g.add_op("add", [g.add_op("mul", [shifted, k]), bias])
        for new in g.ops[first_new:]:
            prepared.add(new)
        z = g.add_op("conv_bias", [conv.operands[0], w2, b2], dict(conv.attrs))
        g.ops += [t for t in tail if t is not conv and t is not op]
        g.replace_all_uses(op.results[0], z)
        for dead in (op, conv):
            for o in dead.operands:
                if dead in o.users:
                    o.users.remove(dead)
    return g


def _strip_keepdim(v, full_shape):
    """v is (reduce result) possibly followed by reshape (keepdim) and broadcast_to back to full_shape."""
    chain = []
    while v.producer is not None and v.producer.name in ("reshape", "broadcast_to"):
        chain.append(v.producer)
        v = v.producer.operands[0]
    return v, chain


def fuse_softmax(g):
    for op in list(g.ops):
        if op.name != "div" or op not in g.ops:
            continue
        e, denom = op.operands
        if e.producer is None or e.producer.name != "exp":
            continue
        s, _ = _strip_keepdim(denom, e.shape)
        if s.producer is None or s.producer.name != "reduce_sum" or s.producer.operands[0] is not e:
            continue
        rank = e.rank
        if tuple(a % rank for a in s.producer.attrs["axis"]) != (rank - 1,):
            continue
        sub = e.producer.operands[0].producer
        if sub is None or sub.name != "sub":
            continue
        x, mx = sub.operands
        m, _ = _strip_keepdim(mx, x.shape)
        if m.producer is None or m.producer.name != "reduce_max" or m.producer.operands[0] is not x:
            continue
        if tuple(a % rank for a in m.producer.attrs["axis"]) != (rank - 1,):
            continue
        if tuple(x.shape) != tuple(op.results[0].shape):
            continue
        # every intermediate must be private to the pattern
        if len(e.users) != 2 or len(sub.results[0].users) != 1 or len(x.users) < 2:
            continue
        idx = g.ops.index(op)
        tail = g.ops[idx:]
        del g.ops[idx:]
        y = g.add_op("softmax", [x], {"axis": rank - 1})
        g.ops += tail
        g.replace_all_uses(op.results[0], y)
        g.dead_code_eliminate()
    return g


LAYOUT_PERMS = {("NCHW", "NHWC"): (0, 2, 3, 1), ("NHWC", "NCHW"): (0, 3, 1, 2)}


def transform_layout(g, target="NCHW"):
    """Every convolution whose layout attribute differs from `target` becomes transpose(x), transpose(w) ->
    conv{layout = target} -> transpose back, with the permutations of the reference's pass
    (src/Dialect/LLH/Transforms/TransformLayout.cpp:141-198, perms :47-72; pinned by its
    test/Dialect/LLH/transform_layout.mlir: 0,2,3,1 on both operands, 0,3,1,2 on the result).  The weight moves
    with the same permutation (FCHW -> FHWC), as there."""
    if target not in ("NCHW", "NHWC"):
        raise ValueError("target layout %r (NCHW or NHWC)" % (target,))
    for op in list(g.ops):
        if op.name not in ("conv", "conv_bias"):
            continue
        layout = op.attrs.get("layout", "NCHW")
        if layout == target:
            continue
        to, back = LAYOUT_PERMS[(layout, target)], LAYOUT_PERMS[(target, layout)]
        idx = g.ops.index(op)
        tail = g.ops[idx:]
        del g.ops[idx:]
        x = g.add_op("transpose", [op.operands[0]], {"perms": to})
        w = g.add_op("transpose", [op.operands[1]], {"perms": to})
        attrs = dict(op.attrs, layout=target, weight_layout=target)
        y = g.add_op(op.name, [x, w] + list(op.operands[2:]), attrs)
        z = g.add_op("transpose", [y], {"perms": back})
        g.ops += tail
        g.replace_all_uses(op.results[0], z)
        g.erase(op)
    return g


def run_llh_pipeline(g, target_layout="NCHW"):
    """Order follows the reference's pipeline (src/Pipeline/TransformPipeline.cpp:103-128):
    legalise/remove-redundant, decompose, canonicalise, layout transform, canonicalise.  Batch norms that follow a
    convolution are folded into it before the decomposition sees them."""
    canonicalize(g)
    fold_batch_norm(g)
    decompose_batch_norm(g)
    fuse_softmax(g)
    canonicalize(g)
    transform_layout(g, target_layout)
    canonicalize(g)
    return g
