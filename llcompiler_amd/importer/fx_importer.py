"""FX graph (ATen / prims ops after AOT decomposition) -> LLH graph.

Counterpart of the reference's importer (llcompiler/importer/fx_translate.py:289-521 and
fx_op_translate/*.py): one translator per ATen/prims target, registered in
TORCH_FUNCTION_TRANSLATE, producing the same LLH ops and attributes (conv attrs as in conv.py:48-70,
negative reduce axes normalised and keepdim expressed as reduce + reshape as in
reduce_ops.py:56-82, scalars as tensor<1xT> constants as in fx_translate.py:274-282).
Differences, all on purpose: bf16/f16 are accepted; `where` passes on_false (the reference passes
on_true twice, where.py:48-49); gelu, softmax, layer_norm, embedding and the extra unary ops
are translated instead of being left to torch eager.
"""
import operator

import torch

from ..llh import expr as sym
from ..llh.expr import Expr, from_sympy
from ..llh.graph import Graph, Value

aten = torch.ops.aten
prims = torch.ops.prims

TORCH_FUNCTION_TRANSLATE = {}
_SUPPORT_CHECKS = {}


def TORCH_FUNCTION_TRANSLATE_REGISTER(*targets, check=None):
    def deco(fn):
        for t in targets:
            TORCH_FUNCTION_TRANSLATE[t] = fn
            if check is not None:
                _SUPPORT_CHECKS[t] = check
        return fn
    return deco


def dim_of(d):
    if isinstance(d, int):
        return d
    if isinstance(d, torch.SymInt):
        e = d.node.expr
        if e.is_number:
            return int(e)
        return from_sympy(e)
    raise TypeError("extent %r" % (d,))


def meta_shape(node_or_val):
    val = node_or_val.meta["val"] if isinstance(node_or_val, torch.fx.Node) else node_or_val
    return tuple(dim_of(d) for d in val.shape)


class Ctx:
    def __init__(self, graph):
        self.g = graph
        self.env = {}  # fx node -> Value | tuple of Values | None (symbolic ints)

    def val(self, a):
        return self.env[a] if isinstance(a, torch.fx.Node) else a

    def like(self, a):
        """The tensor value of `a` when it is one (the operand whose element type a scalar beside it takes)."""
        v = self.env.get(a) if isinstance(a, torch.fx.Node) else None
        return v if isinstance(v, Value) else None

    def tensor_or_const(self, a, like):
        """Python scalars become tensor<1xT> constants of the other operand's element type.  A symbolic scalar (an
        extent, or arithmetic on extents) becomes llh.scalar_cast of its value followed by llh.convert_to that
        type, as in the reference's importer (llcompiler/importer/fx_translate.py:309-323)."""
        if isinstance(a, torch.fx.Node):
            v = self.env[a]
            if isinstance(v, Value):
                return v
            if v is None:
                raise NotImplementedError("scalar operand %s has no value" % a)
            a = v
        dt = like.dtype if like is not None else torch.float32
        real = sym.is_float(a)
        if real and not dt.is_floating_point:
            dt = torch.float32
        if isinstance(a, Expr):
            own = torch.float32 if real else torch.int64
            c = self.g.add_op("scalar_cast", [], {"value": a}, shapes=[(1,)], dtypes=[own], const=a)
            return c if own == dt else self.g.add_op("convert_to", [c], {"dtype": dt})
        return self.g.constant(a, dt)


def _out_shape(node):
    return meta_shape(node)


def _out_dtype(node):
    return node.meta["val"].dtype


def _reshape_to(ctx, x, shape):
    if tuple(x.shape) == tuple(shape):
        return x
    return ctx.g.add_op("reshape", [x], {"shape": tuple(shape)}, shapes=[tuple(shape)], dtypes=[x.dtype])


# ---------------------------------------------------------------- contractions
@TORCH_FUNCTION_TRANSLATE_REGISTER(aten.mm.default)
def _mm(ctx, node):
    return ctx.g.add_op("matmul", [ctx.val(node.args[0]), ctx.val(node.args[1])])


@TORCH_FUNCTION_TRANSLATE_REGISTER(aten.addmm.default)
def _addmm(ctx, node):
    """beta * bias + alpha * (a @ b), kept whole: torch's own decomposition of addmm computes 16-bit operands in
    fp32 (a convert before and after every matmul), while the kernel takes them as they are and accumulates
    in fp32.  The add folds into the matmul's epilogue."""
    bias, a, b = (ctx.val(x) for x in node.args[:3])
    beta, alpha = node.kwargs.get("beta", 1), node.kwargs.get("alpha", 1)
    out = ctx.g.add_op("matmul", [a, b])
    if alpha != 1:
        out = ctx.g.add_op("mul", [out, ctx.g.constant(alpha, out.dtype)])
    if beta != 1:
        bias = ctx.g.add_op("mul", [bias, ctx.g.constant(beta, bias.dtype)])
    return ctx.g.add_op("add", [out, bias])


@TORCH_FUNCTION_TRANSLATE_REGISTER(aten.bmm.default)
def _bmm(ctx, node):
    return ctx.g.add_op("batch_matmul", [ctx.val(node.args[0]), ctx.val(node.args[1])])


def _conv_ok(node):
    a = node.args
    return (not a[6]) and len(a[3]) == 2 and all(int(p) == 0 for p in a[7])


@TORCH_FUNCTION_TRANSLATE_REGISTER(aten.convolution.default, check=_conv_ok)
def _conv(ctx, node):
    x, w, b, stride, padding, dilation, transposed, output_padding, groups = node.args
    xv, wv = ctx.val(x), ctx.val(w)
    attrs = {"dilation": tuple(dilation), "kernel_shape": tuple(wv.shape[-2:]),
             "pad": (padding[0], padding[1], padding[0], padding[1]), "stride": tuple(stride), "group": int(groups),
             "layout": "NCHW"}
    if b is None:
        return ctx.g.add_op("conv", [xv, wv], attrs)
    return ctx.g.add_op("conv_bias", [xv, wv, ctx.val(b)], attrs)


# ---------------------------------------------------------------- views
@TORCH_FUNCTION_TRANSLATE_REGISTER(aten.t.default)
def _t(ctx, node):
    x = ctx.val(node.args[0])
    if x.rank < 2:
        return x
    return ctx.g.add_op("transpose", [x], {"perms": (1, 0)})


@TORCH_FUNCTION_TRANSLATE_REGISTER(aten.permute.default)
def _permute(ctx, node):
    x = ctx.val(node.args[0])
    perms = tuple(p % x.rank for p in node.args[1])
    return ctx.g.add_op("transpose", [x], {"perms": perms})


@TORCH_FUNCTION_TRANSLATE_REGISTER(aten.transpose.int)
def _transpose_int(ctx, node):
    x = ctx.val(node.args[0])
    a, b = node.args[1] % x.rank, node.args[2] % x.rank
    perms = list(range(x.rank))
    perms[a], perms[b] = perms[b], perms[a]
    return ctx.g.add_op("transpose", [x], {"perms": tuple(perms)})


@TORCH_FUNCTION_TRANSLATE_REGISTER(aten.view.default, aten.reshape.default, aten._unsafe_view.default,
                                   aten.unsqueeze.default, aten.squeeze.dim, aten.squeeze.dims, aten.squeeze.default,
                                   prims.squeeze.default, aten.flatten.using_ints)
def _view(ctx, node):
    return _reshape_to(ctx, ctx.val(node.args[0]), _out_shape(node))


# (prims.inductor_force_stride_order asks for a memory layout, not for other values: layouts travel in the
# strides here; the reference rebuilds the shape from the strides, reshape_ops.py:110-140)
@TORCH_FUNCTION_TRANSLATE_REGISTER(aten.clone.default, aten.contiguous.default, aten.alias.default,
                                   aten.detach.default, aten.lift_fresh_copy.default, aten._to_copy.default,
                                   prims.convert_element_type.default, prims.clone.default)
def _identity_or_convert(ctx, node):
    x = ctx.val(node.args[0])
    dt = _out_dtype(node)
    if dt != x.dtype:
        return ctx.g.add_op("convert_to", [x], {"dtype": dt})
    return ctx.g.add_op("identity", [x])


def register_inductor_prims():
    """prims.inductor_force_stride_order only exists once torch._inductor has been imported (it defines the op): called
    at import time here and again by the backend before it translates a graph."""
    op = getattr(prims, "inductor_force_stride_order", None) if "inductor_force_stride_order" in dir(prims) else None
    if op is not None:
        TORCH_FUNCTION_TRANSLATE[op.default] = _identity_or_convert


register_inductor_prims()


@TORCH_FUNCTION_TRANSLATE_REGISTER(prims.broadcast_in_dim.default)
def _broadcast_in_dim(ctx, node):
    x = ctx.val(node.args[0])
    shape = _out_shape(node)
    dims = list(node.args[2])
    aligned = [1] * len(shape)
    for i, d in enumerate(dims):
        aligned[d] = x.shape[i]
    x = _reshape_to(ctx, x, aligned)
    if tuple(aligned) == tuple(shape):
        return x
    return ctx.g.add_op("broadcast_to", [x], {"shape": shape, "cast_dims": tuple(range(len(shape)))})


@TORCH_FUNCTION_TRANSLATE_REGISTER(aten.expand.default)
def _expand(ctx, node):
    x = ctx.val(node.args[0])
    shape = _out_shape(node)
    aligned = (1,) * (len(shape) - x.rank) + tuple(x.shape)
    x = _reshape_to(ctx, x, aligned)
    if tuple(aligned) == tuple(shape):
        return x
    return ctx.g.add_op("broadcast_to", [x], {"shape": shape, "cast_dims": tuple(range(len(shape)))})


@TORCH_FUNCTION_TRANSLATE_REGISTER(aten.select.int)
def _select(ctx, node):
    x = ctx.val(node.args[0])
    dim, index = node.args[1] % x.rank, node.args[2]
    if dim == 0:
        r = ctx.g.add_op("extract", [x], {"index": int(index)})
        # llh.extract of a vector gives tensor<1>, torch a 0-d tensor
        return r if x.rank > 1 else _reshape_to(ctx, r, _out_shape(node))
    if index < 0:
        index += x.shape[dim]
    start = [0] * x.rank
    end = list(x.shape)
    start[dim], end[dim] = index, index + 1
    s = ctx.g.add_op("stride_slice", [x], {"start": tuple(start), "end": tuple(end), "stride": (1,) * x.rank})
    return _reshape_to(ctx, s, _out_shape(node))


@TORCH_FUNCTION_TRANSLATE_REGISTER(aten.slice.Tensor)
def _slice(ctx, node):
    x = ctx.val(node.args[0])
    args = list(node.args) + [None] * (5 - len(node.args))
    dim = (args[1] or 0) % x.rank
    size = x.shape[dim]
    start = args[2] or 0
    end = size if args[3] is None else args[3]
    step = 1 if args[4] is None else args[4]
    if isinstance(start, torch.fx.Node):
        start = ctx.env[start]
    if isinstance(end, torch.fx.Node):
        end = ctx.env[end]
    if isinstance(size, int):
        if start < 0:
            start += size
        if isinstance(end, int):
            if end < 0:
                end += size
            end = min(end, size)
    st = [0] * x.rank
    en = list(x.shape)
    sp = [1] * x.rank
    st[dim], en[dim], sp[dim] = start, end, step
    if st[dim] == 0 and en[dim] == size and step == 1:
        return x
    return ctx.g.add_op("stride_slice", [x], {"start": tuple(st), "end": tuple(en), "stride": tuple(sp)},
                        shapes=[_out_shape(node)], dtypes=[x.dtype])


# ---------------------------------------------------------------- elementwise
def _binary(name):
    def tr(ctx, node):
        a, b = node.args[0], node.args[1]
        av = ctx.tensor_or_const(a, ctx.like(b))
        bv = ctx.tensor_or_const(b, av)
        if ctx.like(a) is None:
            av = ctx.tensor_or_const(a, bv)
        alpha = node.kwargs.get("alpha", 1)
        if alpha != 1:
            bv = ctx.g.add_op("mul", [bv, ctx.g.constant(alpha, bv.dtype)])
        out = ctx.g.add_op(name, [av, bv])
        dt = _out_dtype(node)
        if out.dtype != dt:
            out = ctx.g.add_op("convert_to", [out], {"dtype": dt})
        return out
    return tr


_SCALAR_OPERAND_TARGETS = set()  # translators that accept a symbol-valued scalar where a tensor or number may stand

for _name, _targets in {
    "add": (aten.add.Tensor, aten.add.Scalar, prims.add.default),
    "sub": (aten.sub.Tensor, aten.sub.Scalar, prims.sub.default),
    "mul": (aten.mul.Tensor, aten.mul.Scalar, prims.mul.default),
    "max": (aten.maximum.default, prims.maximum.default),
    "min": (aten.minimum.default, prims.minimum.default),
    "pow": (aten.pow.Tensor_Scalar, aten.pow.Tensor_Tensor, prims.pow.default),
}.items():
    TORCH_FUNCTION_TRANSLATE_REGISTER(*_targets)(_binary(_name))
    _SCALAR_OPERAND_TARGETS.update(_targets)
_SCALAR_OPERAND_TARGETS.update((aten.div.Tensor, aten.div.Scalar, prims.div.default, aten.rsub.Scalar, aten.rsub.Tensor))


def _div_ok(node):
    """True division only: the result is floating point.  prims.div of two integers truncates in torch and the
    elementwise kernel's integer division floors, so that form stays in eager."""
    return node.meta["val"].dtype.is_floating_point


@TORCH_FUNCTION_TRANSLATE_REGISTER(aten.div.Tensor, aten.div.Scalar, prims.div.default, check=_div_ok)
def _div(ctx, node):
    """llh.div on floating point operands.  Integer (or bool) operands of a true division are converted to the
    result type first: torch computes int / int in floating point, an integer llh.div would floor."""
    a, b = node.args[0], node.args[1]
    dt = _out_dtype(node)
    av = ctx.tensor_or_const(a, ctx.like(b))
    bv = ctx.tensor_or_const(b, av)
    if ctx.like(a) is None:
        av = ctx.tensor_or_const(a, bv)
    if av.dtype != dt:
        av = ctx.g.constant(a, dt) if not isinstance(a, torch.fx.Node) else ctx.g.add_op("convert_to", [av], {"dtype": dt})
    if bv.dtype != dt:
        bv = ctx.g.constant(b, dt) if not isinstance(b, torch.fx.Node) else ctx.g.add_op("convert_to", [bv], {"dtype": dt})

    return ctx.g.add_op("div", [av, bv])


@TORCH_FUNCTION_TRANSLATE_REGISTER(aten.rsub.Scalar, aten.rsub.Tensor)
def _rsub(ctx, node):
    a = ctx.val(node.args[0])
    b = ctx.tensor_or_const(node.args[1], a)
    return ctx.g.add_op("sub", [b, a])


def _unary(name):
    def tr(ctx, node):
        x = ctx.val(node.args[0])
        dt = _out_dtype(node)
        # torch promotes the integer operand of exp / sqrt / reciprocal ... to floating point: convert first, an
        # integer program would compute in int64
        if dt.is_floating_point and not x.dtype.is_floating_point:
            x = ctx.g.add_op("convert_to", [x], {"dtype": dt})
        return ctx.g.add_op(name, [x])
    return tr


for _name, _targets in {
    "relu": (aten.relu.default,), "abs": (aten.abs.default, prims.abs.default), "exp": (aten.exp.default, prims.exp.default),
    "sqrt": (aten.sqrt.default, prims.sqrt.default), "rsqrt": (aten.rsqrt.default, prims.rsqrt.default),
    "neg": (aten.neg.default, prims.neg.default), "tanh": (aten.tanh.default, prims.tanh.default),
    "erf": (aten.erf.default, prims.erf.default), "sigmoid": (aten.sigmoid.default,),
    "log": (aten.log.default, prims.log.default), "recip": (aten.reciprocal.default, prims.reciprocal.default),
}.items():
    TORCH_FUNCTION_TRANSLATE_REGISTER(*_targets)(_unary(_name))


@TORCH_FUNCTION_TRANSLATE_REGISTER(aten.gelu.default, check=lambda n: n.kwargs.get("approximate", "none") == "none")
def _gelu(ctx, node):
    return ctx.g.add_op("gelu", [ctx.val(node.args[0])])


def _compare(kind):
    def tr(ctx, node):
        a = ctx.val(node.args[0])
        b = ctx.tensor_or_const(node.args[1], a)
        return ctx.g.add_op("compare", [a, b], {"kind": kind})
    return tr


for _kind, _targets in {
    "EQ": (aten.eq.Tensor, aten.eq.Scalar, prims.eq.default), "NE": (aten.ne.Tensor, aten.ne.Scalar, prims.ne.default),
    "GE": (aten.ge.Tensor, aten.ge.Scalar, prims.ge.default), "GT": (aten.gt.Tensor, aten.gt.Scalar, prims.gt.default),
    "LE": (aten.le.Tensor, aten.le.Scalar, prims.le.default), "LT": (aten.lt.Tensor, aten.lt.Scalar, prims.lt.default),
}.items():
    TORCH_FUNCTION_TRANSLATE_REGISTER(*_targets)(_compare(_kind))
    _SCALAR_OPERAND_TARGETS.update(_targets)
_SCALAR_OPERAND_TARGETS.update((prims.where.default, aten.where.self))


@TORCH_FUNCTION_TRANSLATE_REGISTER(prims.where.default, aten.where.self)
def _where(ctx, node):
    pred = ctx.val(node.args[0])
    t, f = node.args[1], node.args[2]
    like = ctx.like(t) if ctx.like(t) is not None else ctx.like(f)
    tv = ctx.tensor_or_const(t, like)
    fv = ctx.tensor_or_const(f, tv)
    out = ctx.g.add_op("where", [pred, tv, fv])
    dt = _out_dtype(node)
    if out.dtype != dt:
        out = ctx.g.add_op("convert_to", [out], {"dtype": dt})
    return out


def _fill_value_ok(node):
    if node.target in (aten.full.default, aten.full_like.default):
        return isinstance(node.args[1], (int, float, bool))
    if node.target is aten.scalar_tensor.default:
        return isinstance(node.args[0], (int, float, bool))
    return True


@TORCH_FUNCTION_TRANSLATE_REGISTER(aten.scalar_tensor.default, aten.full.default, aten.full_like.default, aten.zeros_like.default,
                                   aten.ones_like.default, aten.zeros.default, aten.ones.default, check=_fill_value_ok)
def _full(ctx, node):
    """Tensors filled with one value (the reference's alloc translators, fx_op_translate/alloc_ops.py:46-103, make a
    constant and broadcast it the same way)."""
    if node.target is aten.scalar_tensor.default:
        value = node.args[0]
    elif node.target in (aten.full.default, aten.full_like.default):
        value = node.args[1]
    elif node.target in (aten.ones_like.default, aten.ones.default):
        value = 1
    else:
        value = 0
    dt = _out_dtype(node)
    c = ctx.g.constant(value, dt)
    shape = _out_shape(node)
    if len(shape) == 0:
        return _reshape_to(ctx, c, ())
    c = _reshape_to(ctx, c, (1,) * len(shape))
    if all(isinstance(d, int) and d == 1 for d in shape):
        return c
    return ctx.g.add_op("broadcast_to", [c], {"shape": shape, "cast_dims": tuple(range(len(shape)))})


@TORCH_FUNCTION_TRANSLATE_REGISTER(aten.sign.default, aten.sgn.default,
                                   check=lambda n: n.meta["val"].dtype in (torch.float32, torch.bfloat16, torch.float16))
def _sign(ctx, node):
    """sign(x) = (x > 0) - (x < 0) in x's type (NaN gives 0 here, NaN in torch)."""
    x = ctx.val(node.args[0])
    zero = ctx.g.constant(0.0, x.dtype)
    pos = ctx.g.add_op("convert_to", [ctx.g.add_op("compare", [x, zero], {"kind": "GT"})], {"dtype": x.dtype})
    neg = ctx.g.add_op("convert_to", [ctx.g.add_op("compare", [x, zero], {"kind": "LT"})], {"dtype": x.dtype})
    return ctx.g.add_op("sub", [pos, neg])


# ---------------------------------------------------------------- reductions / normalisation / pooling
def _reduce(name):
    def tr(ctx, node):
        x = ctx.val(node.args[0])
        dims = node.args[1] if len(node.args) > 1 else list(range(x.rank))
        if isinstance(dims, int):
            dims = [dims]
        axes = tuple(sorted(d % x.rank for d in dims)) if len(dims) else tuple(range(x.rank))
        keepdim = node.args[2] if len(node.args) > 2 else False
        r = ctx.g.add_op(name, [x], {"axis": axes})
        if keepdim:
            r = _reshape_to(ctx, r, _out_shape(node))
        return r
    return tr


def _float_reduce(node):
    """The reduce kernels take f32, bf16 and f16 and give the same type back: a sum over a bool mask (int64 in
    torch; the backward of amax makes one) or over integers stays in eager."""
    v = node.args[0].meta.get("val")
    out = node.meta.get("val")
    floats = (torch.float32, torch.bfloat16, torch.float16)
    return isinstance(v, torch.Tensor) and v.dtype in floats and isinstance(out, torch.Tensor) and out.dtype == v.dtype


TORCH_FUNCTION_TRANSLATE_REGISTER(aten.amax.default, check=_float_reduce)(_reduce("reduce_max"))
TORCH_FUNCTION_TRANSLATE_REGISTER(aten.amin.default, check=_float_reduce)(_reduce("reduce_min"))
TORCH_FUNCTION_TRANSLATE_REGISTER(aten.sum.dim_IntList, check=_float_reduce)(_reduce("reduce_sum"))
TORCH_FUNCTION_TRANSLATE_REGISTER(prims.sum.default, check=_float_reduce)(_reduce("reduce_sum"))  # (x, dims): never keepdim


@TORCH_FUNCTION_TRANSLATE_REGISTER(prims.collapse_view.default)
def _collapse_view(ctx, node):
    """Dims start .. end (inclusive) become one (fx_op_translate/reshape_ops.py:89-107)."""
    return _reshape_to(ctx, ctx.val(node.args[0]), _out_shape(node))


def _mean_ok(node):
    shape = node.args[0].meta["val"].shape
    dims = node.args[1]
    return all(isinstance(shape[d], int) for d in dims) and _float_reduce(node)


@TORCH_FUNCTION_TRANSLATE_REGISTER(aten.mean.dim, check=_mean_ok)
def _mean(ctx, node):
    x = ctx.val(node.args[0])
    dims = tuple(sorted(d % x.rank for d in node.args[1]))
    keepdim = node.args[2] if len(node.args) > 2 else False
    if x.rank == 4 and dims == (2, 3):
        r = ctx.g.add_op("adaptive_average_pool", [x], {"out_size": (1, 1)})
        return r if keepdim else _reshape_to(ctx, r, _out_shape(node))
    count = 1
    for d in dims:
        count *= x.shape[d]
    r = ctx.g.add_op("reduce_sum", [x], {"axis": dims})
    r = ctx.g.add_op("div", [r, ctx.g.constant(float(count), x.dtype)])
    return _reshape_to(ctx, r, _out_shape(node)) if keepdim else r


@TORCH_FUNCTION_TRANSLATE_REGISTER(aten._adaptive_avg_pool2d.default, aten.adaptive_avg_pool2d.default,
                                   check=lambda n: list(n.args[1]) == [1, 1])
def _adaptive_avg_pool(ctx, node):
    return ctx.g.add_op("adaptive_average_pool", [ctx.val(node.args[0])], {"out_size": (1, 1)})


@TORCH_FUNCTION_TRANSLATE_REGISTER(aten._softmax.default,
                                   check=lambda n: n.args[1] % n.args[0].meta["val"].dim() == n.args[0].meta["val"].dim() - 1)
def _softmax(ctx, node):
    x = ctx.val(node.args[0])
    dt = _out_dtype(node)  # half_to_float: a 16-bit input with an fp32 result
    if x.dtype != dt:
        # torch computes and returns fp32 probabilities from the 16-bit input: widen first, so that they are not
        # rounded to the storage type on the way
        x = ctx.g.add_op("convert_to", [x], {"dtype": dt})
    return ctx.g.add_op("softmax", [x], {"axis": x.rank - 1})


def _sdpa_args(node):
    """(q, k, v, bias, dropout, causal, scale) of the two fused-attention ops aot autograd puts in place of
    F.scaled_dot_product_attention on a GPU."""
    a, kw = list(node.args), node.kwargs
    if node.target is aten._scaled_dot_product_efficient_attention.default:
        a += [None] * (7 - len(a))
        return a[0], a[1], a[2], a[3], (a[5] if a[5] is not None else 0.0), bool(a[6]), kw.get("scale")
    a += [None] * (6 - len(a))
    return a[0], a[1], a[2], None, (a[3] if a[3] is not None else 0.0), bool(a[4]), kw.get("scale")


def _sdpa_ok(node):
    q, k, v, bias, dropout, causal, scale = _sdpa_args(node)
    if bias is not None or dropout != 0.0 or causal or not _first_result_only(node):
        return False  # masks, dropout and the statistics a backward graph reads stay with torch's kernel
    shapes = [t.meta["val"].shape for t in (q, k, v)]
    return all(len(sh) == 4 and isinstance(sh[3], int) for sh in shapes) and shapes[0][3] == shapes[1][3] == shapes[2][3] and \
        tuple(shapes[0][:2]) == tuple(shapes[1][:2]) == tuple(shapes[2][:2])


@TORCH_FUNCTION_TRANSLATE_REGISTER(aten._scaled_dot_product_flash_attention.default,
                                   aten._scaled_dot_product_efficient_attention.default, check=_sdpa_ok)
def _sdpa(ctx, node):
    """F.scaled_dot_product_attention without mask or dropout, spelt as the group the reference's importer gets from an
    attention layer written out by hand (llcompiler/test_models/models/multi_head_attention.py:20-33): batch_matmul of
    q with the transposed keys, the scale, softmax over the keys, batch_matmul with v.  The planner folds the scale
    into the first product and the engine runs the group as one fused kernel where the head dim allows."""
    q, k, v, _, _, _, scale = _sdpa_args(node)
    g = ctx.g
    qv, kv, vv = ctx.val(q), ctx.val(k), ctx.val(v)
    b, h, sq, d = qv.shape
    skv = kv.shape[2]
    if scale is None:
        scale = float(d) ** -0.5
    q3, v3 = (_reshape_to(ctx, t, (b * h, t.shape[2], d)) for t in (qv, vv))
    # the keys are transposed as the rank-4 tensor they are, then flattened (what torch.matmul(q, k.transpose(-2, -1))
    # decomposes to): a transpose of the flattened view would have to be made in memory first
    kt3 = _reshape_to(ctx, g.add_op("transpose", [kv], {"perms": (0, 1, 3, 2)}), (b * h, d, skv))
    scores = g.add_op("batch_matmul", [q3, kt3])
    scores = g.add_op("mul", [scores, g.constant(float(scale), scores.dtype)])
    probs = g.add_op("softmax", [scores], {"axis": 2})
    out = _reshape_to(ctx, g.add_op("batch_matmul", [probs, v3]), (b, h, sq, d))
    return (out,) + (None,) * (len(node.meta["val"]) - 1)


def _first_result_only(node):
    """The translators of multi-result ATen ops produce the first result only (the output; not the saved
    statistics or pooling indices a backward graph asks for): a node whose other results are used stays in eager."""
    return all(u.op == "call_function" and u.target is operator.getitem and u.args[1] == 0 for u in node.users)


def _as(ctx, v, dtype):
    return v if v.dtype == dtype else ctx.g.add_op("convert_to", [v], {"dtype": dtype})


def _sum_keep_last(ctx, v):
    """Sum over the last dim, kept as an extent of 1 (what broadcasts back over the rows)."""
    r = ctx.g.add_op("reduce_sum", [v], {"axis": (v.rank - 1,)})
    return _reshape_to(ctx, r, tuple(v.shape[:-1]) + (1,))


def _used_results(node):
    return set(u.args[1] for u in node.users if u.op == "call_function" and u.target is operator.getitem)


def _last_dim_static(node):
    return len(node.args[1]) == 1 and isinstance(node.args[0].meta["val"].shape[-1], int)


@TORCH_FUNCTION_TRANSLATE_REGISTER(aten.native_layer_norm.default,
                                   check=lambda n: len(n.args[1]) == 1 and (_first_result_only(n) or _last_dim_static(n)))
def _layer_norm(ctx, node):
    """The output is llh.layer_norm; the saved statistics a backward graph asks for (mean and 1/std of every row, kept
    as [.., 1]) are spelt with reductions and elementwise ops in fp32, as torch computes them."""
    x, shape, w, b, eps = node.args
    ops = [ctx.val(x)] + [ctx.val(t) for t in (w, b) if t is not None]
    attrs = {"epsilon": float(eps), "axis": -1, "has_scale": w is not None, "has_bias": b is not None}
    y = ctx.g.add_op("layer_norm", ops, attrs)
    used = _used_results(node)
    if not (used - {0}):
        return (y, None, None)
    g = ctx.g
    x32 = _as(ctx, ctx.val(x), torch.float32)
    n = float(x32.shape[-1])
    mean = g.add_op("div", [_sum_keep_last(ctx, x32), g.constant(n, torch.float32)])
    d = g.add_op("sub", [x32, mean])
    var = g.add_op("div", [_sum_keep_last(ctx, g.add_op("mul", [d, d])), g.constant(n, torch.float32)])
    rstd = g.add_op("rsqrt", [g.add_op("add", [var, g.constant(float(eps), torch.float32)])])
    vals = node.meta["val"]
    return (y, _as(ctx, mean, vals[1].dtype), _as(ctx, rstd, vals[2].dtype))


@TORCH_FUNCTION_TRANSLATE_REGISTER(aten.native_layer_norm_backward.default,
                                   check=lambda n: len(n.args[2]) == 1 and isinstance(n.args[1].meta["val"].shape[-1], int))
def _layer_norm_backward(ctx, node):
    """dx = rstd (g w - mean(g w) - xhat mean(g w xhat)), dw = sum over rows of g xhat, db = sum over rows of g, with
    xhat = (x - mean) rstd from the saved statistics; fp32 arithmetic whatever the storage type (torch's own)."""
    go, x, shape, mean, rstd, w, b, mask = node.args
    g = ctx.g
    f32 = torch.float32
    go32, x32 = _as(ctx, ctx.val(go), f32), _as(ctx, ctx.val(x), f32)
    mean32, rstd32 = _as(ctx, ctx.val(mean), f32), _as(ctx, ctx.val(rstd), f32)
    n = float(x32.shape[-1])
    xhat = g.add_op("mul", [g.add_op("sub", [x32, mean32]), rstd32])
    vals = node.meta["val"]
    dx = dw = db = None
    if mask[0]:
        gw = g.add_op("mul", [go32, _as(ctx, ctx.val(w), f32)]) if w is not None else go32
        m1 = g.add_op("div", [_sum_keep_last(ctx, gw), g.constant(n, f32)])
        m2 = g.add_op("div", [_sum_keep_last(ctx, g.add_op("mul", [gw, xhat])), g.constant(n, f32)])
        inner = g.add_op("sub", [g.add_op("sub", [gw, m1]), g.add_op("mul", [xhat, m2])])
        dx = _as(ctx, g.add_op("mul", [inner, rstd32]), vals[0].dtype)
    rows = tuple(range(x32.rank - 1))
    if mask[1] and w is not None:
        dw = _as(ctx, g.add_op("reduce_sum", [g.add_op("mul", [go32, xhat])], {"axis": rows}), vals[1].dtype)
    if mask[2] and b is not None:
        db = _as(ctx, g.add_op("reduce_sum", [go32], {"axis": rows}), vals[2].dtype)
    return (dx, dw, db)


@TORCH_FUNCTION_TRANSLATE_REGISTER(aten._softmax_backward_data.default,
                                   check=lambda n: n.args[2] % n.args[0].meta["val"].dim() == n.args[0].meta["val"].dim() - 1)
def _softmax_backward(ctx, node):
    """dx = y (g - sum(g y)) over the last dim, in fp32."""
    go, y = _as(ctx, ctx.val(node.args[0]), torch.float32), _as(ctx, ctx.val(node.args[1]), torch.float32)
    g = ctx.g
    s = _sum_keep_last(ctx, g.add_op("mul", [go, y]))
    return _as(ctx, g.add_op("mul", [y, g.add_op("sub", [go, s])]), _out_dtype(node))


@TORCH_FUNCTION_TRANSLATE_REGISTER(aten.gelu_backward.default, check=lambda n: n.kwargs.get("approximate", "none") == "none")
def _gelu_backward(ctx, node):
    """g (Phi(x) + x phi(x)): the derivative of x Phi(x), one elementwise program after fusion."""
    g = ctx.g
    f32 = torch.float32
    go, x = _as(ctx, ctx.val(node.args[0]), f32), _as(ctx, ctx.val(node.args[1]), f32)

    def c(v):
        return g.constant(v, f32)
    cdf = g.add_op("mul", [g.add_op("add", [g.add_op("erf", [g.add_op("mul", [x, c(0.7071067811865476)])]), c(1.0)]), c(0.5)])
    pdf = g.add_op("mul", [g.add_op("exp", [g.add_op("mul", [g.add_op("mul", [x, x]), c(-0.5)])]), c(0.3989422804014327)])
    return _as(ctx, g.add_op("mul", [go, g.add_op("add", [cdf, g.add_op("mul", [x, pdf])])]), _out_dtype(node))


@TORCH_FUNCTION_TRANSLATE_REGISTER(aten._native_batch_norm_legit_no_training.default, check=_first_result_only)
def _batch_norm(ctx, node):
    x, w, b, mean, var, momentum, eps = node.args
    xv = ctx.val(x)
    c = xv.shape[1]
    wv = ctx.val(w) if w is not None else _ones_like_channels(ctx, c, xv.dtype, 1.0)
    bv = ctx.val(b) if b is not None else _ones_like_channels(ctx, c, xv.dtype, 0.0)
    y = ctx.g.add_op("batch_norm_inference", [xv, wv, bv, ctx.val(mean), ctx.val(var)],
                     {"epsilon": float(eps), "momentum": float(momentum), "feature_index": 1})
    return (y, None, None)


def _bn_eval_only(node):
    return node.args[5] is False and _first_result_only(node)


@TORCH_FUNCTION_TRANSLATE_REGISTER(aten.native_batch_norm.default, aten._native_batch_norm_legit.default,
                                   aten.miopen_batch_norm.default, aten.cudnn_batch_norm.default, check=_bn_eval_only)
def _batch_norm_native(ctx, node):
    """The batch-norm entry points a GPU module dispatches to in eval mode; all share the signature
    (input, weight, bias, running_mean, running_var, training=False, momentum, eps)."""
    x, w, b, mean, var, training, momentum, eps = node.args
    xv = ctx.val(x)
    c = xv.shape[1]
    wv = ctx.val(w) if w is not None else _ones_like_channels(ctx, c, xv.dtype, 1.0)
    bv = ctx.val(b) if b is not None else _ones_like_channels(ctx, c, xv.dtype, 0.0)
    y = ctx.g.add_op("batch_norm_inference", [xv, wv, bv, ctx.val(mean), ctx.val(var)],
                     {"epsilon": float(eps), "momentum": float(momentum), "feature_index": 1})
    return (y, None, None)


def _ones_like_channels(ctx, c, dtype, value):
    k = ctx.g.constant(value, dtype)
    return ctx.g.add_op("broadcast_to", [k], {"shape": (c,), "cast_dims": (0,)})


def _maxpool_ok(node):
    a = list(node.args) + [None] * 6
    return not a[5] and _first_result_only(node)  # no ceil_mode, no indices


@TORCH_FUNCTION_TRANSLATE_REGISTER(aten.max_pool2d_with_indices.default, check=_maxpool_ok)
def _max_pool(ctx, node):
    a = list(node.args) + [None] * (6 - len(node.args))
    x, k = ctx.val(a[0]), tuple(a[1])
    if len(k) == 1:
        k = (k[0], k[0])
    stride = tuple(a[2]) if a[2] else k
    pad = tuple(a[3]) if a[3] else (0, 0)
    dil = tuple(a[4]) if a[4] else (1, 1)
    def two(t): return t if len(t) == 2 else (t[0], t[0])
    stride, pad, dil = two(stride), two(pad), two(dil)
    y = ctx.g.add_op("max_pool", [x], {"ceil_mode": False, "dilation": dil, "kernel_shape": k,
                                        "pad": (pad[0], pad[1], pad[0], pad[1]), "stride": stride, "layout": "NCHW"})
    return (y, None)


@TORCH_FUNCTION_TRANSLATE_REGISTER(aten.embedding.default)
def _embedding(ctx, node):
    idx = ctx.val(node.args[1])
    if idx.dtype != torch.int64:  # the row gather takes int64 indices; torch also accepts int32
        idx = ctx.g.add_op("convert_to", [idx], {"dtype": torch.int64})
    return ctx.g.add_op("gather", [ctx.val(node.args[0]), idx])


@TORCH_FUNCTION_TRANSLATE_REGISTER(operator.getitem)
def _getitem(ctx, node):
    src = ctx.env[node.args[0]]
    return src[node.args[1]]


# Arithmetic on symbolic scalars (the reference translates the same targets to scalar llh ops,
# fx_op_translate/binary_ops.py:39-76, unary_ops.py:79, lowered at src/Conversion/LLHToArith/LLHToArith.cpp:112-144).
# Shapes take their extents from each node's fake value; the value of the node itself is kept as an expression
# for the places where it is an operand of a tensor op.
_SYMBOLIC_TARGETS = {aten.sym_size.int, aten.sym_numel.default, operator.mul, operator.add, operator.sub,
                     operator.floordiv, operator.truediv, operator.neg, operator.pow}
if hasattr(torch, "_sym_sqrt"):
    _SYMBOLIC_TARGETS.add(torch._sym_sqrt)
if hasattr(torch, "sym_float"):
    _SYMBOLIC_TARGETS.add(torch.sym_float)
_SYMBOLIC_BINARY = {operator.mul: operator.mul, operator.add: operator.add, operator.sub: operator.sub,
                    operator.floordiv: operator.floordiv, operator.truediv: operator.truediv, operator.pow: operator.pow}


def _symbolic_value(ctx, node):
    """The value of a symbolic scalar node: a number, or an expression over the graph's symbols."""
    def arg(a):
        if isinstance(a, torch.fx.Node):
            v = ctx.env[a]
            if v is None or isinstance(v, (Value, tuple)):
                raise NotImplementedError("scalar arithmetic on %s" % a)
            return v
        return a
    t = node.target
    if t is aten.sym_size.int:
        x = ctx.val(node.args[0])
        return x.shape[node.args[1] % x.rank]
    if t is aten.sym_numel.default:
        return sym.product(ctx.val(node.args[0]).shape)
    if t in _SYMBOLIC_BINARY:
        return _SYMBOLIC_BINARY[t](arg(node.args[0]), arg(node.args[1]))
    if t is operator.neg:
        return -arg(node.args[0])
    if t is getattr(torch, "_sym_sqrt", None):
        return sym.sqrt(arg(node.args[0]))
    if t is getattr(torch, "sym_float", None):
        return sym.to_float(arg(node.args[0]))
    raise NotImplementedError("symbolic scalar target %s" % (t,))


def _symbolic_scalar(a):
    return isinstance(a, torch.fx.Node) and isinstance(a.meta.get("val", a.meta.get("example_value")),
                                                      (torch.SymInt, torch.SymFloat, torch.SymBool, int, float))


def _symbolic_ok(a):
    """Whether the scalar node `a` is arithmetic the importer can keep as an expression."""
    if not isinstance(a, torch.fx.Node):
        return isinstance(a, (int, float)) and not isinstance(a, bool)
    if a.op == "placeholder":
        return isinstance(a.meta.get("val", a.meta.get("example_value")), (torch.SymInt, int))
    if a.op != "call_function" or a.target not in _SYMBOLIC_TARGETS:
        return False
    if a.target in (aten.sym_size.int, aten.sym_numel.default):
        return True
    return all(_symbolic_ok(x) for x in a.args)


def is_supported(node):
    """Whether a call_function node can be compiled (the reference's LLC_SUPPORT_DICT lookup,
    llcompiler/compiler/torch_compile_config.py:29-132, extended with per-node attribute checks)."""
    if node.target in _SYMBOLIC_TARGETS:
        return True
    if node.target not in TORCH_FUNCTION_TRANSLATE:
        register_inductor_prims()
    if node.target not in TORCH_FUNCTION_TRANSLATE:
        return False
    # a symbol-valued scalar as a direct operand (x / x.shape[0]): only the translators that build their operands
    # with tensor_or_const take one, and only when its arithmetic can be kept as an expression
    for a in node.args:
        if _symbolic_scalar(a) and not (node.target in _SCALAR_OPERAND_TARGETS and _symbolic_ok(a)):
            return False
    chk = _SUPPORT_CHECKS.get(node.target)
    try:
        return True if chk is None else bool(chk(node))
    except Exception:
        return False


def _as_traced(ctx, v, node):
    """The translated value with the rank torch traced.  Python scalars enter the graph as tensor<1xT> constants
    (TorchToLLH keeps them that way), so an op between a 0-d tensor and a number comes out as tensor<1xT> where torch
    has a 0-d tensor (`num_batches_tracked + 1` of a batch norm in training mode, whose result aot autograd copies back
    into the 0-d buffer): same elements, a reshape to the traced shape."""
    val = node.meta.get("val")
    if not isinstance(v, Value) or not isinstance(val, torch.Tensor):
        return v
    want = meta_shape(val)
    if len(want) == v.rank or any(not isinstance(d, int) for d in tuple(want) + tuple(v.shape)):
        return v
    n_want = n_have = 1
    for d in want:
        n_want *= d
    for d in v.shape:
        n_have *= d
    return _reshape_to(ctx, v, want) if n_want == n_have else v


def torch_translate_to_llh_graph(gm, weight_files=None):
    """Counterpart of torch_translate_to_mlir_module (llcompiler/importer/fx_translate.py:517-521).

    weight_files: {placeholder name: .npy path}.  Those placeholders become llh.weight ops that name their file
    (fx_translate.py:415-435 does this for the parameters of the traced module) instead of run-time inputs."""
    register_inductor_prims()
    g = Graph()
    ctx = Ctx(g)
    weight_files = weight_files or {}
    for node in gm.graph.nodes:
        if node.op == "placeholder":
            val = node.meta.get("val", node.meta.get("example_value"))
            if node.name in weight_files:
                if not isinstance(val, torch.Tensor) or any(not isinstance(d, int) for d in meta_shape(val)):
                    raise TypeError("weight %s must be a tensor of static shape" % node.name)
                ctx.env[node] = g.add_op("weight", [], {"weight_file": weight_files[node.name]}, shapes=[meta_shape(val)],
                                         dtypes=[val.dtype])
            elif isinstance(val, torch.Tensor):
                ctx.env[node] = g.add_input(meta_shape(val), val.dtype, name=node.name)
            elif isinstance(val, (torch.SymInt, int)):
                # dynamo passes SymInts as leading int arguments (fx_translate.py:373-406)
                e = dim_of(val)
                name = e.args[0] if isinstance(e, Expr) and e.kind == "sym" else str(e)
                g.add_symbol_arg(name)
                ctx.env[node] = e
            elif val is None:
                g.arg_kinds.append(("none", None))
                ctx.env[node] = None
            else:
                raise TypeError("Unsupported type: %s" % type(val))
        elif node.op == "call_function":
            if node.target in _SYMBOLIC_TARGETS:
                try:
                    ctx.env[node] = _symbolic_value(ctx, node)
                except (NotImplementedError, TypeError, ZeroDivisionError):
                    ctx.env[node] = None  # still good for shapes, which come from the fake values
                continue
            tr = TORCH_FUNCTION_TRANSLATE.get(node.target)
            if tr is None:
                raise NotImplementedError("no LLH translation for %s" % (node.target,))
            ctx.env[node] = _as_traced(ctx, tr(ctx, node), node)
        elif node.op == "output":
            outs = node.args[0]
            single = not isinstance(outs, (tuple, list))
            seq = [outs] if single else list(outs)
            res = []
            for o in seq:
                if o is None:
                    res.append(None)
                elif isinstance(o, torch.fx.Node):
                    v = ctx.env[o]
                    if v is None or isinstance(v, (Expr, int, float)):  # a symbolic int result
                        res.append(dim_of(o.meta["val"]))
                    else:
                        res.append(v)
                else:
                    res.append(o)
            g.set_outputs(res)
            g.single_output = single
        else:
            raise NotImplementedError("fx node kind %s" % node.op)
    return g
