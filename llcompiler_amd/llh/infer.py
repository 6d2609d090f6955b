"""Result shapes and element types of LLH ops: the rules of the reference's symbolic shape inference
(src/Dialect/LLH/IR/LLHinfersymbolShape.cpp) over int-or-Expr extents."""
import torch

from .expr import Expr, ceildiv, product


def _same_dim(a, b):
    return (isinstance(a, int) and isinstance(b, int) and a == b) or (isinstance(a, Expr) and a == b)


def broadcast_shapes(*shapes):
    """numpy-style broadcast; a lower rank is aligned on the right (the reference reshapes it to
    rank-aligned 1s first, src/Dialect/LLH/Utils/LLHUtilitys.cpp:80-150)."""
    rank = max(len(s) for s in shapes)
    out = []
    for i in range(rank):
        d = 1
        for s in shapes:
            j = i - (rank - len(s))
            if j < 0:
                continue
            x = s[j]
            if isinstance(x, int) and x == 1:
                continue
            if isinstance(d, int) and d == 1:
                d = x
            elif not _same_dim(d, x):
                if isinstance(d, int) and isinstance(x, int):
                    raise ValueError("shapes %s do not broadcast" % (shapes,))
                # two different symbolic spellings of what must be the same extent: keep the first
        out.append(d)
    return tuple(out)


def window_out(n, pad_lo, pad_hi, dil, k, stride):
    """LLHinfersymbolShape.cpp:265-266 (static) / :274-279 (symbolic): floor division."""
    return (n + (pad_lo + pad_hi - dil * (k - 1) - 1)) // stride + 1


def infer(name, operands, attrs):
    shapes = [o.shape for o in operands]
    dt = operands[0].dtype if operands else None
    if name in ("abs", "sqrt", "exp", "relu", "rsqrt", "neg", "gelu", "tanh", "erf", "sigmoid", "log", "recip", "identity",
                "softmax", "drop"):
        return [shapes[0]], [dt]
    if name in ("add", "sub", "mul", "div", "max", "min", "pow"):
        return [broadcast_shapes(*shapes)], [torch.promote_types(operands[0].dtype, operands[1].dtype)]
    if name == "compare":
        return [broadcast_shapes(*shapes)], [torch.bool]
    if name == "where":
        return [broadcast_shapes(*shapes)], [torch.promote_types(operands[1].dtype, operands[2].dtype)]
    if name == "convert_to":
        return [shapes[0]], [attrs["dtype"]]
    if name == "matmul":  # LLHinfersymbolShape.cpp:531-556
        (m, k), (k2, n) = shapes
        return [(m, n)], [dt]
    if name == "batch_matmul":  # :558-585
        (b, m, k), (b2, k2, n) = shapes
        return [(b, m, n)], [dt]
    if name in ("conv", "conv_bias"):  # :214-331
        # layout NCHW: x [N,C,H,W], w [F,C,KH,KW]; layout NHWC: x [N,H,W,C], w [F,KH,KW,C] (LLHEnums.td:61-75)
        nhwc = attrs.get("layout", "NCHW") == "NHWC"
        n, h, w = (shapes[0][0], shapes[0][1], shapes[0][2]) if nhwc else (shapes[0][0], shapes[0][2], shapes[0][3])
        f = shapes[1][0]
        kh, kw = attrs["kernel_shape"]
        p, s, d = attrs["pad"], attrs["stride"], attrs["dilation"]
        oh, ow = window_out(h, p[0], p[2], d[0], kh, s[0]), window_out(w, p[1], p[3], d[1], kw, s[1])
        return [(n, oh, ow, f) if nhwc else (n, f, oh, ow)], [dt]
    if name == "max_pool":
        n, c, h, w = shapes[0]
        kh, kw = attrs["kernel_shape"]
        p, s, d = attrs["pad"], attrs["stride"], attrs["dilation"]
        return [(n, c, window_out(h, p[0], p[2], d[0], kh, s[0]), window_out(w, p[1], p[3], d[1], kw, s[1]))], [dt]
    if name == "adaptive_average_pool":  # :587-613
        out_size = tuple(attrs["out_size"])
        return [tuple(shapes[0][:len(shapes[0]) - len(out_size)]) + out_size], [dt]
    if name in ("batch_norm_inference", "layer_norm"):
        return [shapes[0]], [dt]
    if name in ("reduce_sum", "reduce_max", "reduce_min"):  # :185-212
        rank = len(shapes[0])
        axes = [a % rank for a in attrs["axis"]]
        return [tuple(d for i, d in enumerate(shapes[0]) if i not in axes)], [dt]
    if name == "reshape":
        return [resolve_reshape(shapes[0], attrs["shape"])], [dt]
    if name == "transpose":
        return [tuple(shapes[0][p] for p in attrs["perms"])], [dt]
    if name == "broadcast_to":
        return [tuple(attrs["shape"])], [dt]
    if name == "stride_slice":  # size = ceildiv(end - start, stride), StablehlotoLinalgExtension.cpp:68-118
        return [tuple(ceildiv(e - s, st) for s, e, st in zip(attrs["start"], attrs["end"], attrs["stride"]))], [dt]
    if name == "extract":  # the row of dim 0 with the dim dropped; a rank-1 input keeps one element as tensor<1>
        return [tuple(shapes[0][1:]) if len(shapes[0]) > 1 else (1,)], [dt]  # (LLHinfersymbolShape.cpp:504-529)
    if name == "gather":
        return [tuple(shapes[1]) + tuple(shapes[0][1:])], [dt]
    raise NotImplementedError("no shape rule for llh.%s" % name)


def resolve_reshape(in_shape, new_shape):
    """-1 resolution as in the reshape canonicaliser (src/Dialect/LLH/IR/LLHCanonicalize.cpp:418-455)."""
    new_shape = list(new_shape)
    if -1 in [d for d in new_shape if isinstance(d, int)]:
        i = new_shape.index(-1)
        known = product([d for j, d in enumerate(new_shape) if j != i])
        total = product(in_shape)
        if isinstance(known, int) and isinstance(total, int):
            new_shape[i] = total // known
        else:
            new_shape[i] = total // known
    return tuple(new_shape)
