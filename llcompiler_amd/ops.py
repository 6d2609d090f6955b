"""Kernel calls: one thin Python function per C-ABI entry point of libllc_hip.so.

Each function allocates the output with torch (device memory only), builds the descriptors and
enqueues the kernel on torch's current HIP stream.  No arithmetic happens in Python or in torch.
With defer=True a function returns a `Call` whose launch() only crosses the C-ABI, for callers
that issue the same call many times on fixed buffers (plans, benchmarks).
"""
import ctypes

import torch

from . import _capi as C


def _dev(t):
    if not t.is_cuda:
        raise RuntimeError("llcompiler_amd kernels run on the GPU only; got a %s tensor (no CPU fallback)" % t.device)
    C.init(t.device.index or 0)
    return t.device


class Call:
    """A kernel call with its descriptors already built."""

    __slots__ = ("fn", "args", "keep", "out", "device")

    def __init__(self, fn, args, keep, out, device):
        self.fn, self.args, self.keep, self.out, self.device = fn, args, keep, out, device

    def launch(self, stream=None):
        """stream: a ctypes stream handle to launch on (C.current_stream(device) when None; callers that
        launch many calls in a row look it up once)."""
        st = self.fn(*self.args, C.current_stream(self.device) if stream is None else stream)
        if st != 0:
            C.check(st)
        return self.out


def _launch(fn, args, keep, out, device, defer):
    """args: everything but the trailing stream argument."""
    call = Call(fn, args, keep, out, device)
    return call if defer else call.launch()


def window_out(n, pad_lo, pad_hi, dil, k, stride):
    """LLHinfersymbolShape.cpp:257-268"""
    return (n + pad_lo + pad_hi - dil * (k - 1) - 1) // stride + 1


class Epilogue:
    """act(alpha * acc + bias + residual) fused into a contraction."""

    def __init__(self, alpha=1.0, bias=None, residual=None, act="none"):
        self.alpha, self.bias, self.residual = float(alpha), bias, residual
        self.act = {"none": C.ACT_NONE, "relu": C.ACT_RELU, "gelu": C.ACT_GELU}[act]

    def build(self):
        self._b = C.tensor_ref(self.bias)
        self._r = C.tensor_ref(self.residual) if self.residual is not None else None
        self._s = C.LlcEpilogue(self.alpha, self._b.ptr if self._b else None, self._r.ptr if self._r else None,
                                self.act)
        return ctypes.pointer(self._s)


def _epi(e):
    return e.build() if e is not None else None


def matmul(a, b, epilogue=None, out=None, defer=False):
    dev = _dev(a)
    if out is None:
        out = torch.empty((a.shape[0], b.shape[1]), dtype=a.dtype, device=dev)
    ra, rb, ro = C.tensor_ref(a), C.tensor_ref(b), C.tensor_ref(out)
    return _launch(C.lib().llc_hip_matmul, (ra.ptr, rb.ptr, _epi(epilogue), ro.ptr), (ra, rb, ro, epilogue), out, dev,
                   defer)


def matmul_static(a, b, out, epilogue=None, defer=False):
    """llc_hip_matmul_static: the same product through the entry point that allocates nothing (split reductions
    keep their partial sums in the library's static device array).  `out` is the caller's, as in the C-ABI."""
    dev = _dev(a)
    ra, rb, ro = C.tensor_ref(a), C.tensor_ref(b), C.tensor_ref(out)
    return _launch(C.lib().llc_hip_matmul_static, (ra.ptr, rb.ptr, _epi(epilogue), ro.ptr), (ra, rb, ro, epilogue), out,
                   dev, defer)


def batch_matmul(a, b, epilogue=None, out=None, defer=False):
    dev = _dev(a)
    if out is None:
        nb = 1
        for d in a.shape[:-2]:
            nb *= d
        out = torch.empty((nb, a.shape[-2], b.shape[-1]), dtype=a.dtype, device=dev)
    ra, rb, ro = C.tensor_ref(a), C.tensor_ref(b), C.tensor_ref(out)
    return _launch(C.lib().llc_hip_batch_matmul, (ra.ptr, rb.ptr, _epi(epilogue), ro.ptr), (ra, rb, ro, epilogue), out,
                   dev, defer)


def conv2d(x, w, pad=(0, 0, 0, 0), stride=(1, 1), dilation=(1, 1), group=1, epilogue=None, out=None, defer=False):
    """pad = (h_lo, w_lo, h_hi, w_hi), the LLH attribute order."""
    dev = _dev(x)
    N, _, H, W = x.shape
    F, _, KH, KW = w.shape
    OH = window_out(H, pad[0], pad[2], dilation[0], KH, stride[0])
    OW = window_out(W, pad[1], pad[3], dilation[1], KW, stride[1])
    if out is None:
        out = torch.empty((N, F, OH, OW), dtype=x.dtype, device=dev)
    attrs = C.LlcConvAttrs((ctypes.c_int64 * 2)(*dilation), (ctypes.c_int64 * 2)(KH, KW), (ctypes.c_int64 * 4)(*pad),
                           (ctypes.c_int64 * 2)(*stride), group)
    rx, rw, ro = C.tensor_ref(x), C.tensor_ref(w), C.tensor_ref(out)
    return _launch(C.lib().llc_hip_conv2d, (rx.ptr, rw.ptr, ctypes.pointer(attrs), _epi(epilogue), ro.ptr),
                   (rx, rw, ro, attrs, epilogue), out, dev, defer)


def make_program(insts, result=0, integer=False):
    """insts: list of (op, dst, a[, b[, c]]) with operands 'r0'..'r3', 'in0'..'in5' or one number (the immediate)."""
    prog = C.LlcEwProgram()
    if len(insts) > C.EW_MAX_INSTS:
        raise ValueError("elementwise chain of %d instructions (max %d)" % (len(insts), C.EW_MAX_INSTS))
    prog.n_insts = len(insts)
    prog.integer = 1 if integer else 0

    def sel(x):
        if isinstance(x, str):
            return int(x[1:]) if x[0] == "r" else C.EW_IN0 + int(x[2:])
        return C.EW_IMM

    for i, ins in enumerate(insts):
        op, dst, *srcs = ins
        imm = [s for s in srcs if not isinstance(s, str)]
        if len(imm) > 1:
            raise ValueError("one immediate per instruction")
        srcs = list(srcs) + ["r0"] * (3 - len(srcs))
        prog.insts[i] = C.LlcEwInst(C.EW_OPCODES[op], sel(dst), sel(srcs[0]), sel(srcs[1]), sel(srcs[2]),
                                    float(imm[0]) if imm else 0.0)
    prog.result = sel(result) if isinstance(result, str) else int(result)
    return prog


def elementwise(prog, inputs, out_shape, out_dtype, out=None, defer=False):
    if not inputs:
        raise ValueError("an elementwise program reads at least one tensor")
    dev = _dev(inputs[0])
    if out is None:
        out = torch.empty(tuple(out_shape), dtype=out_dtype, device=dev)
    refs = []
    for t in inputs:
        # rank-align on the left with 1s, as the reference's canonicaliser does before broadcast_to
        # (src/Dialect/LLH/Utils/LLHUtilitys.cpp:80-150)
        pad = len(out_shape) - t.dim()
        refs.append(C.tensor_ref(t, (1,) * pad + tuple(t.shape), (0,) * pad + tuple(t.stride())))
    arr = (ctypes.POINTER(C.LlcTensor) * max(len(refs), 1))(*[r.ptr for r in refs])
    ro = C.tensor_ref(out)
    return _launch(C.lib().llc_hip_elementwise, (ctypes.pointer(prog), arr, len(refs), ro.ptr), (prog, refs, arr, ro),
                   out, dev, defer)


def reduce(kind, x, axes, out=None, defer=False):
    dev = _dev(x)
    axes = [a % x.dim() for a in axes]
    if out is None:
        out = torch.empty([s for d, s in enumerate(x.shape) if d not in axes], dtype=x.dtype, device=dev)
    code = {"sum": C.REDUCE_SUM, "max": C.REDUCE_MAX, "min": C.REDUCE_MIN}[kind]
    rx, ro = C.tensor_ref(x), C.tensor_ref(out)
    ax = C.i64_array(axes)
    return _launch(C.lib().llc_hip_reduce, (code, rx.ptr, ax, len(axes), ro.ptr), (rx, ro, ax), out, dev, defer)


def softmax(x, out=None, defer=False):
    dev = _dev(x)
    if out is None:
        out = torch.empty_like(x)
    rx, ro = C.tensor_ref(x), C.tensor_ref(out)
    return _launch(C.lib().llc_hip_softmax, (rx.ptr, ro.ptr), (rx, ro), out, dev, defer)


def layer_norm(x, scale=None, bias=None, eps=1e-5, out=None, defer=False):
    dev = _dev(x)
    if out is None:
        out = torch.empty_like(x)
    rx, ro, rs, rb = C.tensor_ref(x), C.tensor_ref(out), C.tensor_ref(scale), C.tensor_ref(bias)
    return _launch(C.lib().llc_hip_layer_norm, (rx.ptr, rs.ptr if rs else None, rb.ptr if rb else None, float(eps),
                                                ro.ptr), (rx, ro, rs, rb), out, dev, defer)


def max_pool(x, kernel, pad=(0, 0, 0, 0), stride=(1, 1), dilation=(1, 1), init_zero=False, out=None, defer=False):
    dev = _dev(x)
    N, Cc, H, W = x.shape
    OH = window_out(H, pad[0], pad[2], dilation[0], kernel[0], stride[0])
    OW = window_out(W, pad[1], pad[3], dilation[1], kernel[1], stride[1])
    if out is None:
        out = torch.empty((N, Cc, OH, OW), dtype=x.dtype, device=dev)
    attrs = C.LlcPoolAttrs((ctypes.c_int64 * 2)(*dilation), (ctypes.c_int64 * 2)(*kernel), (ctypes.c_int64 * 4)(*pad),
                           (ctypes.c_int64 * 2)(*stride), 1 if init_zero else 0)
    rx, ro = C.tensor_ref(x), C.tensor_ref(out)
    return _launch(C.lib().llc_hip_max_pool, (rx.ptr, ctypes.pointer(attrs), ro.ptr), (rx, ro, attrs), out, dev, defer)


def global_avg_pool(x, keepdim=False, out=None, defer=False):
    dev = _dev(x)
    if out is None:
        shape = (x.shape[0], x.shape[1], 1, 1) if keepdim else (x.shape[0], x.shape[1])
        out = torch.empty(shape, dtype=x.dtype, device=dev)
    rx, ro = C.tensor_ref(x), C.tensor_ref(out)
    return _launch(C.lib().llc_hip_global_avg_pool, (rx.ptr, ro.ptr), (rx, ro), out, dev, defer)


def transpose(x, perms, out=None, defer=False):
    dev = _dev(x)
    if out is None:
        out = torch.empty([x.shape[p] for p in perms], dtype=x.dtype, device=dev)
    rx, ro = C.tensor_ref(x), C.tensor_ref(out)
    pm = C.i64_array(perms)
    return _launch(C.lib().llc_hip_transpose, (rx.ptr, pm, ro.ptr), (rx, ro, pm), out, dev, defer)


def stride_slice(x, start, end, step, out=None, defer=False):
    dev = _dev(x)
    if out is None:
        out = torch.empty([max(0, -(-(e - s) // st)) for s, e, st in zip(start, end, step)], dtype=x.dtype, device=dev)
    rx, ro = C.tensor_ref(x), C.tensor_ref(out)
    a, b, c = C.i64_array(start), C.i64_array(end), C.i64_array(step)
    return _launch(C.lib().llc_hip_stride_slice, (rx.ptr, a, b, c, ro.ptr), (rx, ro, a, b, c), out, dev, defer)


def extract(x, index, out=None, defer=False):
    """llh.extract: row `index` of dim 0 with the dim dropped; a negative index counts from the end
    (src/Dialect/LLH/IR/LLHCanonicalize.cpp:337-354); one element of a vector comes back as tensor<1>
    (src/Dialect/LLH/IR/LLHinfersymbolShape.cpp:513-516)."""
    dev = _dev(x)
    if index < 0:
        index += x.shape[0]
    if out is None:
        out = torch.empty(tuple(x.shape[1:]) if x.dim() > 1 else (1,), dtype=x.dtype, device=dev)
    if x.dim() == 1:
        rx, ro = C.tensor_ref(x), C.tensor_ref(out)
        a, b, c = C.i64_array([index]), C.i64_array([index + 1]), C.i64_array([1])
        return _launch(C.lib().llc_hip_stride_slice, (rx.ptr, a, b, c, ro.ptr), (rx, ro, a, b, c), out, dev, defer)
    start = [index] + [0] * (x.dim() - 1)
    end = [index + 1] + list(x.shape[1:])
    ro = C.tensor_ref(out, (1,) + tuple(out.shape), (max(out.numel(), 1),) + tuple(out.stride()))
    rx = C.tensor_ref(x)
    a, b, c = C.i64_array(start), C.i64_array(end), C.i64_array([1] * x.dim())
    return _launch(C.lib().llc_hip_stride_slice, (rx.ptr, a, b, c, ro.ptr), (rx, ro, a, b, c), out, dev, defer)


def broadcast_to(x, shape, out=None, defer=False):
    dev = _dev(x)
    if out is None:
        out = torch.empty(tuple(shape), dtype=x.dtype, device=dev)
    rx, ro = C.tensor_ref(x), C.tensor_ref(out)
    return _launch(C.lib().llc_hip_broadcast_to, (rx.ptr, ro.ptr), (rx, ro), out, dev, defer)


def copy(x, out=None, defer=False):
    """Materialises any strided view into a contiguous tensor."""
    dev = _dev(x)
    if out is None:
        out = torch.empty(tuple(x.shape), dtype=x.dtype, device=dev)
    rx, ro = C.tensor_ref(x), C.tensor_ref(out)
    return _launch(C.lib().llc_hip_copy, (rx.ptr, ro.ptr), (rx, ro), out, dev, defer)


def gather_rows(table, idx, out=None, defer=False):
    dev = _dev(table)
    if out is None:
        out = torch.empty(tuple(idx.shape) + tuple(table.shape[1:]), dtype=table.dtype, device=dev)
    rt, ri, ro = C.tensor_ref(table), C.tensor_ref(idx), C.tensor_ref(out)
    return _launch(C.lib().llc_hip_gather_rows, (rt.ptr, ri.ptr, ro.ptr), (rt, ri, ro), out, dev, defer)


def convert(x, dtype, out=None, defer=False):
    dev = _dev(x)
    if out is None:
        out = torch.empty(tuple(x.shape), dtype=dtype, device=dev)
    rx, ro = C.tensor_ref(x), C.tensor_ref(out)
    return _launch(C.lib().llc_hip_convert, (rx.ptr, ro.ptr), (rx, ro), out, dev, defer)


def attention(q, k, v, mask=None, scale=1.0, out=None, defer=False):
    """softmax(scale * q k^T + mask) v.  q, out: [B, H, Sq, D]; k, v: [B, H, Skv, D] (strided views allowed, last
    dim contiguous; D = 64, or 32 or 128 in bf16 / f16); mask: None or [B, Skv]."""
    dev = _dev(q)
    if out is None:
        out = torch.empty(tuple(q.shape), dtype=q.dtype, device=dev)
    rq, rk, rv, ro, rm = C.tensor_ref(q), C.tensor_ref(k), C.tensor_ref(v), C.tensor_ref(out), C.tensor_ref(mask)
    return _launch(C.lib().llc_hip_attention, (rq.ptr, rk.ptr, rv.ptr, rm.ptr if rm else None, float(scale), ro.ptr),
                   (rq, rk, rv, ro, rm), out, dev, defer)
