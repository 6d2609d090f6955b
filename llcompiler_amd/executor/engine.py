"""Run-time side of a compiled LLH graph: device buffers, symbolic-shape dispatch and the call
convention of the reference's executor.

`Torch_ExecutionEngine.run(*args)` keeps the reference's convention
(llcompiler/executor/engine.py:56-78): tensors positional, Python ints are symbol values, the
result is a tensor or a list.  What changes underneath:

  * output shapes come from evaluating the graph's symbolic extents with the bound symbols, not
    from re-tracing the FX graph with FakeTensorProp on every call
    (llcompiler/executor/out_put_call.py:154-170);
  * for every distinct binding (symbol values + input layouts) the plan is specialised once into an
    `Instance`: concrete shapes, intermediate device buffers (reused by liveness), and prepared
    kernel calls.  Later calls with the same binding only patch the input/output pointers into the
    descriptors and launch;
  * tensors live on the GPU; nothing is copied to the host.
"""
import ctypes
import os

import torch

from .. import _capi as C
from .. import ops
from ..llh.expr import Expr, evaluate
from ..llh.graph import Value
from .plan_runner import ParamBlock, Plan
from .planner import make_plan
from .weights import WeightStore

# same codes as the reference's map (engine.py:11), extended with bf16 / f16 / i32
TORCH_DTYPE_TO_TYPE = C.TORCH_DTYPE_TO_TYPE


# HIP-graph replay of an instance's launch sequence, opt-in (LLC_GRAPHS=1).  Measured on the five benchmark
# configurations it does not pay: they are GPU-bound from a few kernels upwards (host cost per launch ~3 us),
# and for the two-kernel MLP the staging copy, the replay call and the output clone cost more on the host than
# two launches do (57 us against 34 us per call).  It helps a caller that is host-bound for other reasons.
USE_GRAPHS = os.environ.get("LLC_GRAPHS", "0") == "1"
MIN_CALLS_FOR_GRAPH = 2
# The first run of an instance records its kernel calls into a native plan (llc_plan_t); later runs fill the
# reference's packed parameter block and make one call into the library, which replays the launches.  With
# False every run launches kernel by kernel from Python (same kernels, same arguments).
USE_PLAN = True
# batch_matmul -> softmax -> batch_matmul groups of attention layers with head dim 64 (32 and 128 too in the 16-bit
# types) become one fused kernel
FUSE_ATTENTION = True
# convolutions whose channel count is a multiple of 128 bytes' worth of values (32 fp32, 64 bf16 / f16) run on
# channels-last (NHWC) copies of their operands: the kernel for that layout needs no gather arithmetic.  Results keep the layout as strided views (logical shape NCHW), so a chain of
# convolutions converts once; anything that needs NCHW memory copies back through the usual contiguity path.
CHANNELS_LAST = True
# linear layers that read the same rows with weights that are graph inputs (q, k, v projections) run as one
# product against a stacked copy of the weights
FUSE_PROJECTIONS = True
PROJ_TILE_LIMIT = 1024  # projections of the same rows are stacked while one of them has fewer 64x64 tiles than this


def _concrete(shape, env):
    return tuple(evaluate(d, env) if isinstance(d, Expr) else int(d) for d in shape)


def _alias_signature(inputs):
    """Which inputs share a storage, and at what distance: an instance binds descriptors to inputs by address,
    so calls that differ in this are different bindings."""
    first, sig = {}, []
    for i, t in enumerate(inputs):
        j = first.setdefault(t.untyped_storage().data_ptr(), i)
        if j != i:
            sig.append((j, i, t.data_ptr() - inputs[j].data_ptr()))
    return tuple(sig)


class _Pool:
    """Intermediate device buffers, reused once their last reader has been enqueued (all kernels of
    an instance run in order on one stream, so reuse needs no further synchronisation)."""

    def __init__(self, device):
        self.device = device
        self.free = {}
        self.all = []

    def take(self, nbytes):
        size = max(256, (nbytes + 255) // 256 * 256)
        lst = self.free.get(size)
        if lst:
            return lst.pop()
        buf = torch.empty(size, dtype=torch.uint8, device=self.device)
        self.all.append(buf)
        return buf

    def give(self, buf):
        self.free.setdefault(buf.numel(), []).append(buf)


def _is_channels_last(t):
    """A 4-D tensor that is NHWC in memory and not also NCHW-contiguous."""
    return isinstance(t, torch.Tensor) and t.dim() == 4 and not t.is_contiguous() and \
        t.is_contiguous(memory_format=torch.channels_last)


class _LazyReshape:
    """A reshape that is not a view of its source (e.g. the head split [B,S,H,D] -> permute -> [B*H,S,D]): the
    copy is made only if a consumer needs the reshaped tensor; batch_matmul reads the 4-D source in place."""

    __slots__ = ("src", "shape", "done")

    def __init__(self, src, shape):
        self.src, self.shape, self.done = src, tuple(shape), None


class Instance:
    """A plan specialised to concrete extents: a flat list of prepared kernel calls."""

    def __init__(self, graph, steps, env, inputs, device, weights=None):
        self.graph, self.env, self.device = graph, env, device
        self.weights = weights     # WeightStore of the engine: tensors of llh.weight ops, loaded once
        self.calls = []
        self.prep_calls = []       # run before `calls` when an input listed in prep_inputs changed
        self.prep_inputs = []
        self._prep_key = None
        self._preparing = None     # while a prepared step is built: the graph inputs its result depends on
        self.patches = []          # (TensorRef, "in"|"out", index, byte offset from that tensor's data_ptr)
        self.keep = []
        self._roots = {}           # storage data_ptr -> ("in"|"out", index, base data_ptr)
        self.out_meta = []         # (shape, dtype) of every tensor output
        self.example_outputs = []
        self._build(steps, inputs)

    # ---- bookkeeping of per-call storages ----
    def _register_root(self, kind, index, t):
        self._roots.setdefault(t.untyped_storage().data_ptr(), (kind, index, t.data_ptr()))

    def _launch_later(self, call):
        if self._preparing is not None:
            # a step that computes a derived weight (batch norm folded into a convolution's filters)
            return self._prepare_later(call, self._preparing)
        # every descriptor the call holds is checked against the per-call storages
        for item in call.keep:
            self._scan(item)
        self.calls.append(call)

    def _prepare_later(self, call, input_index):
        """A call whose result depends only on graph inputs that are weights (`input_index`: one index or several; a
        layout copy of a weight, folded filters): it runs before the instance's other calls, and again only when
        one of those inputs' address or version counter changed."""
        for item in call.keep:
            self._scan(item)
        self.prep_calls.append(call)
        for i in ([input_index] if isinstance(input_index, int) else input_index):
            if i not in self.prep_inputs:
                self.prep_inputs.append(i)

    def _channels_last_ok(self, st, ins, out, natural):
        if not CHANNELS_LAST or out.dtype not in (torch.float32, torch.bfloat16, torch.float16) or \
                st.attrs["group"] != 1 or len(natural) != 4:
            return False
        x, w = ins
        if tuple(natural) != tuple(out.shape) or not out.numel() or x.dim() != 4 or w.dim() != 4:
            return False
        return x.shape[1] % (128 // out.dtype.itemsize) == 0 and w.shape[0] % 4 == 0 and w.shape[2] * w.shape[3] <= 64 and \
            x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0

    def _first_layer_channels_last_ok(self, st, x, w, out, natural, res):
        """Whether the NCHW convolution `st` (an image network's first layer: few channels, 64 filters, stride 2) may
        write its result channels-last, for the channels-last layers after it: the shapes the row kernels of
        llc_hip_conv2d take with NCHW operands and a channels-last result."""
        if not CHANNELS_LAST or res is not None or st.attrs["group"] != 1 or len(natural) != 4 or \
                tuple(natural) != tuple(out.shape) or x.dim() != 4 or w.dim() != 4:
            return False
        a = st.attrs
        (n, c, h, wd), (f, _, kh, kw), (oh, ow) = x.shape, w.shape, natural[2:]
        pw, es = a["pad"][1], out.dtype.itemsize
        if f != 64 or tuple(a["dilation"]) != (1, 1) or a["stride"][1] != 2 or n * oh < 256 or ow % 4 or \
                x.data_ptr() % 16 or w.data_ptr() % 16:
            return False
        if es == 4:
            return out.dtype == torch.float32 and c * kh * kw <= 148 and c * kh <= 21 and wd % 4 == 0 and wd <= 224 and \
                pw <= min(256 - wd, 32) and ow <= 112 and 2 * 111 + kw - 1 - pw <= 255
        shift = pw & 1
        return out.dtype in (torch.bfloat16, torch.float16) and c * kh <= 24 and kw + shift <= 8 and wd % 8 == 0 and \
            wd <= 256 - (pw + shift) and pw + shift <= 64 and ow <= 128 and 2 * (16 * ((ow + 15) // 16) - 1) - pw - shift + 7 <= 255

    def _scan(self, item):
        if isinstance(item, C.TensorRef):
            t = item._keep
            if isinstance(t, torch.Tensor):
                root = self._roots.get(t.untyped_storage().data_ptr())
                if root is not None:
                    self.patches.append((item, root[0], root[1], t.data_ptr() - root[2]))
        elif isinstance(item, ops.Epilogue):
            for r in (getattr(item, "_b", None), getattr(item, "_r", None)):
                if r is not None:
                    self._scan(r)
        elif isinstance(item, (list, tuple)):
            for x in item:
                self._scan(x)

    # ---- building ----
    def _build(self, steps, inputs):
        g = self.graph
        dev = self.device
        val = {}
        for i, (v, t) in enumerate(zip(g.inputs, inputs)):
            val[id(v)] = t
            self._register_root("in", i, t)
        out_ids = {}
        for k, o in enumerate(g.outputs):
            if isinstance(o, Value):
                out_ids.setdefault(id(o), []).append(k)
        # A graph output that is a chain of views of a kernel's result (the [B S, N] product of a Linear layer seen as
        # [B, S, N]): the kernel writes into an output buffer and the output is that view, with no copy at the end.
        made_by = {id(st.output): st for st in steps}
        out_roots = set()
        for o in g.outputs:
            st = made_by.get(id(o)) if isinstance(o, Value) else None
            hops = 0
            while st is not None and st.kind == "view" and hops < 16:
                root, hops = st.inputs[0], hops + 1
                st = made_by.get(id(root))
                if st is not None and st.kind not in ("view", "constant") and not st.attrs.get("prepared"):
                    out_roots.add(id(root))
        # liveness per backing buffer: a value and every view derived from it share one root; the
        # root's buffer returns to the pool after the last step that reads any of them
        root_of = {}
        for st in steps:
            if st.kind == "view":
                src = id(st.inputs[0])
                root_of[id(st.output)] = root_of.get(src, src)
        last_use = {}
        for si, st in enumerate(steps):
            reads = list(st.inputs)
            e = st.attrs.get("epilogue") if isinstance(st.attrs, dict) else None
            if e:
                reads += [x for x in (e.get("bias"), e.get("residual")) if x is not None]
            for r in reads:
                rid = root_of.get(id(r), id(r))
                last_use[rid] = si
        for o in g.outputs:
            if isinstance(o, Value):
                last_use[root_of.get(id(o), id(o))] = len(steps)  # read by the output copy at the end
        pool = _Pool(dev)
        self.pool = pool
        owner = {}      # id(root value) -> pool buffer backing it
        temps = []      # staging copies made for the current step
        n_out_bufs = 0

        def new_tensor(v, shape=None):
            nonlocal n_out_bufs
            shape = _concrete(v.shape if shape is None else shape, self.env)
            if id(v) in out_ids or (id(v) in out_roots and self._preparing is None):
                t = torch.empty(shape, dtype=v.dtype, device=dev)
                self._register_root("out", n_out_bufs, t)
                self.out_buffers.append(t)
                n_out_bufs += 1
                return t
            if self._preparing is not None:
                # written ahead of every other call and read by every run: never a buffer of the reuse pool
                t = torch.empty(shape, dtype=v.dtype, device=dev)
                self.keep.append(t)
                return t
            n = 1
            for d in shape:
                n *= d
            buf = pool.take(n * v.dtype.itemsize)
            owner[id(v)] = buf
            return buf[: n * v.dtype.itemsize].view(v.dtype).view(shape)

        self.out_buffers = []

        def contiguous(t):
            if t.is_contiguous():
                return t
            n = t.numel()
            buf = pool.take(n * t.dtype.itemsize)
            temps.append(buf)
            c = buf[: n * t.dtype.itemsize].view(t.dtype).view(tuple(t.shape))
            if n:
                self._launch_later(ops.copy(t, out=c, defer=True))
            return c

        def materialise(x):
            if isinstance(x, _LazyReshape):
                if x.done is None:
                    n = x.src.numel()
                    buf = pool.take(n * x.src.dtype.itemsize)
                    self.keep.append(buf)  # stays private to this instance
                    c = buf[: n * x.src.dtype.itemsize].view(x.src.dtype).view(tuple(x.src.shape))
                    if n:
                        self._launch_later(ops.copy(x.src, out=c, defer=True))
                    x.done = c.view(x.shape)
                return x.done
            return x

        def batched_operand(x):
            """A lazy [B0*B1, R, C] reshape of a 4-D tensor goes to batch_matmul as that 4-D tensor."""
            if isinstance(x, _LazyReshape) and x.done is None and x.src.dim() == 4 and \
                    x.shape == (x.src.shape[0] * x.src.shape[1], x.src.shape[2], x.src.shape[3]):
                return x.src
            return materialise(x)

        cl_copies = {}   # id(value) -> its channels-last copy
        prep_deps = {}   # id(value written by a prepared step) -> indices of the graph inputs it depends on

        def prep_root(v):
            """The dependencies of `v` when it is a derived weight or a view of one, else None."""
            seen = 0
            while id(v) not in prep_deps and seen < 16:
                st = producer.get(id(v))
                if st is None or st.kind != "view":
                    return None
                v, seen = st.inputs[0], seen + 1
            return prep_deps.get(id(v))

        def to_channels_last(v, t):
            """`t` (the tensor of value `v`, logical NCHW) as a channels-last tensor: itself if it already is, else a
            copy made once per value.  Copies of graph inputs (weights) are made by the instance's preparation
            calls, which run again only when such an input moved or was written to."""
            if t.is_contiguous(memory_format=torch.channels_last):
                return t
            c = cl_copies.get(id(v))
            if c is None:
                n = t.numel()
                root = self._roots.get(t.untyped_storage().data_ptr())
                prepared = root is not None and root[0] == "in" and id(v) in input_ids
                deps = root[1] if prepared else None
                if not prepared and prep_root(v) is not None:
                    prepared, deps = True, prep_root(v)  # a derived weight: its copy is made where it is made
                if prepared:
                    # written ahead of every other call and kept: never a buffer that earlier steps have used
                    nhwc = torch.empty((t.shape[0], t.shape[2], t.shape[3], t.shape[1]), dtype=t.dtype, device=dev)
                    self.keep.append(nhwc)
                else:
                    buf = pool.take(n * t.dtype.itemsize)
                    self.keep.append(buf)
                    nhwc = buf[: n * t.dtype.itemsize].view(t.dtype).view(t.shape[0], t.shape[2], t.shape[3], t.shape[1])
                call = ops.copy(t.permute(0, 2, 3, 1), out=nhwc, defer=True)
                if prepared:
                    self._prepare_later(call, deps)
                else:
                    self._launch_later(call)
                c = cl_copies[id(v)] = nhwc.permute(0, 3, 1, 2)
            return c

        def epi_of(st):
            """The step's epilogue with a symbol-valued scale (x / x.shape[0] folded into alpha) as this binding's number."""
            e = st.attrs["epilogue"]
            if isinstance(e["alpha"], Expr):
                e = dict(e, alpha=float(evaluate(e["alpha"], self.env)))
            return e

        input_ids = set(id(v) for v in g.inputs)
        consumers = {}
        for st in steps:
            reads = list(st.inputs)
            e = st.attrs.get("epilogue") if isinstance(st.attrs, dict) else None
            if e:
                reads += [x for x in (e.get("bias"), e.get("residual")) if x is not None]
            for v in reads:
                consumers.setdefault(id(v), []).append(st)
        skip = set()

        def only_consumer(v):
            u = consumers.get(id(v), [])
            return u[0] if len(u) == 1 and id(v) not in out_ids else None

        producer = {id(st.output): st for st in steps}

        def resolve_early(v):
            """Makes val[v] available ahead of its turn when v is only views away from a value that exists."""
            if id(v) in val:
                return True
            st = producer.get(id(v))
            if st is None or st.kind != "view" or not resolve_early(st.inputs[0]):
                return False
            val[id(v)] = self._view(st, materialise(val[id(st.inputs[0])]), contiguous)
            skip.add(id(st))
            return True

        def attention_group(st):
            """scores = batch_matmul(q, k^T) {alpha, mask rows} -> softmax over the keys -> batch_matmul(p, v), every
            intermediate read once and only reshaped in between: returns (softmax step, second product, the
            reshapes) or None."""
            e = epi_of(st)
            if e["act"] or e["residual"] is not None or e["alpha"] <= 0 or (e["bias"] is not None and not e.get("bias_rows")):
                return None
            if st.output.dtype not in (torch.bfloat16, torch.float16, torch.float32):
                return None
            between = []

            def through_reshapes(v):
                u = only_consumer(v)
                while u is not None and u.kind == "view" and u.attrs["op"] in ("reshape", "flatten"):
                    between.append(u)
                    v = u.output
                    u = only_consumer(v)
                return v, u

            v, u = through_reshapes(st.output)
            if u is None or u.kind != "softmax":
                return None
            n_keys = _concrete(st.attrs["natural_shape"], self.env)[-1]
            if _concrete(u.inputs[0].shape, self.env)[-1] != n_keys:
                return None
            sm = u
            v, u = through_reshapes(sm.output)
            if u is None or u.kind != "batch_matmul" or u.inputs[0] is not v or u.inputs[1] is v:
                return None
            e2 = epi_of(u)
            if e2["act"] or e2["residual"] is not None or e2["bias"] is not None or e2["alpha"] != 1.0:
                return None
            return sm, u, between

        def fused_attention(st):
            """Emits one attention call for the group that starts at `st` when the operands allow it (head dim 64, or
            32 or 128 in the 16-bit types; rows addressable as [B, H, S, D] views); returns False to leave the group to
            its own kernels."""
            grp = attention_group(st)
            if grp is None:
                return False
            sm, second, between = grp
            if not resolve_early(second.inputs[1]):
                return False
            e = epi_of(st)
            qa, ka = (batched_operand(val[id(v)]) for v in st.inputs)
            va = batched_operand(val[id(second.inputs[1])])
            nat = _concrete(st.attrs["natural_shape"], self.env)
            if e.get("bias_rows"):
                full = _concrete(st.output.shape, self.env)
                b0, b1 = full[0], full[1]
            else:
                four = [t for t in (qa, ka, va) if t.dim() == 4]
                merge = head_merge(second, nat[0], nat[1], 64)
                if four:
                    b0, b1 = four[0].shape[0], four[0].shape[1]
                elif merge is not None:
                    # every operand already lies as [B * H, S, 64] (a batch of one): the head merge that follows
                    # says how B * H splits
                    b0, b1 = merge[1], merge[2]
                else:
                    b0, b1 = nat[0], 1

            def as4(t):
                if t.dim() == 4:
                    return t if tuple(t.shape[:2]) == (b0, b1) else None
                if t.dim() != 3 or t.shape[0] != b0 * b1:
                    return None
                return t.as_strided((b0, b1, t.shape[1], t.shape[2]), (b1 * t.stride(0), t.stride(0), t.stride(1), t.stride(2)))

            q4, k4, v4 = as4(qa), as4(ka), as4(va)
            if q4 is None or k4 is None or v4 is None:
                return False
            k4 = k4.transpose(-1, -2)
            for t in (q4, k4, v4):
                dims = (64,) if t.dtype == torch.float32 else (32, 64, 128)
                if t.shape[3] not in dims or t.stride(3) != 1 or any(s % 8 for s in t.stride()[:3]) or t.data_ptr() % 16:
                    return False
            if k4.shape[2] != v4.shape[2] or k4.shape[2] != nat[2] or q4.shape[2] != nat[1] or k4.shape[2] == 0:
                return False
            mask = None
            if e["bias"] is not None:
                mask = materialise(val[id(e["bias"])])
                mask = contiguous(mask.reshape(-1) if mask.is_contiguous() else mask).reshape(-1).view(b0, nat[2])
            out = new_tensor(second.output)
            sq, hd = nat[1], q4.shape[3]
            o4 = out.view(b0, b1, sq, hd)
            hm = head_merge(second, b0 * b1, sq, hd)
            if hm is not None and (hm[1], hm[2]) == (b0, b1):
                # the head merge that follows, [B, H, S, D] -> [B, S, H, D], is done by the kernel's stores
                o4 = out.view(-1).view(b0, sq, b1, hd).permute(0, 2, 1, 3)
                val[id(hm[0].output)] = o4
                skip.add(id(hm[0]))
            if out.numel():
                self._launch_later(ops.attention(q4, k4, v4, mask, scale=e["alpha"], out=o4, defer=True))
            val[id(second.output)] = out
            for x in [sm, second] + between:
                skip.add(id(x))
            return True

        def head_merge(st, nb, m, n):
            """batch_matmul -> reshape [B0,B1,M,N] -> transpose (0,2,1,3), each read once: returns (reshape step,
            B0, B1) so that the product can be written in the transposed layout directly."""
            u = consumers.get(id(st.output), [])
            if len(u) != 1 or u[0].kind != "view" or u[0].attrs["op"] not in ("reshape", "flatten") or id(st.output) in out_ids:
                return None
            shp = _concrete(u[0].output.shape, self.env)
            if len(shp) != 4 or shp[0] * shp[1] != nb or shp[2] != m or shp[3] != n or id(u[0].output) in out_ids:
                return None
            u2 = consumers.get(id(u[0].output), [])
            if len(u2) != 1 or u2[0].kind != "view" or u2[0].attrs["op"] != "transpose" or tuple(u2[0].attrs["perms"]) != (0, 2, 1, 3):
                return None
            return u[0], shp[0], shp[1]

        def weight_like(t, shape):
            """A tensor of the given shape that lies contiguous in a graph input's storage (a parameter)."""
            if not isinstance(t, torch.Tensor) or tuple(t.shape) != tuple(shape) or not t.is_contiguous():
                return None
            root = self._roots.get(t.untyped_storage().data_ptr())
            return root[1] if root is not None and root[0] == "in" else None

        def fused_projections(st, si):
            """Several linear layers over the same rows (the q, k and v projections of an attention block) run as one
            product against the stacked weights: [M,K] x [K, N1+N2+..].  The stacked weight and bias are copies made
            by the instance's preparation calls; every layer's result is a column slice of the one output."""
            e = epi_of(st)
            if e["residual"] is not None or e.get("bias_rows") or id(st.output) in out_ids:
                return False
            nat = _concrete(st.attrs["natural_shape"], self.env)
            if len(nat) != 2 or nat[0] == 0:
                return False
            x = materialise(val[id(st.inputs[0])])
            if x.dim() != 2:
                return False
            m, kdim = x.shape
            # worth it while one layer's product leaves CUs idle or fills them unevenly; with more rows the separate
            # products are as fast and their results lie denser for the attention kernel (measured on the bf16
            # encoder block: 17% faster at 512 rows, 9% faster at 4096, 3% slower at 16384; BERT-base fp32 at
            # 4096 rows 1.5% faster)
            if ((m + 63) // 64) * ((nat[1] + 63) // 64) >= PROJ_TILE_LIMIT:
                return False

            def member(s2):
                """(weight as [N,K], its input index, bias, its input index) when s2 can join, else None."""
                if s2.kind != "matmul":
                    return None
                e2 = epi_of(s2)
                if s2.kind != "matmul" or id(s2) in skip or id(s2.output) in out_ids or s2.output.dtype != st.output.dtype:
                    return None
                if e2["residual"] is not None or e2.get("bias_rows") or e2["act"] != e["act"] or e2["alpha"] != e["alpha"] or \
                        (e2["bias"] is None) != (e["bias"] is None):
                    return None
                n2 = _concrete(s2.attrs["natural_shape"], self.env)
                if len(n2) != 2 or n2[0] != m or not resolve_early(s2.inputs[0]) or not resolve_early(s2.inputs[1]):
                    return None
                x2, w2 = val[id(s2.inputs[0])], val[id(s2.inputs[1])]
                if not isinstance(x2, torch.Tensor) or not isinstance(w2, torch.Tensor) or x2.data_ptr() != x.data_ptr() or \
                        tuple(x2.shape) != tuple(x.shape) or x2.stride() != x.stride() or w2.dim() != 2:
                    return None
                wi = weight_like(w2.t(), (n2[1], kdim))
                if wi is None:
                    return None
                b2, bi = None, None
                if e2["bias"] is not None:
                    if not resolve_early(e2["bias"]):
                        return None
                    b2 = val[id(e2["bias"])]
                    b2 = b2.reshape(-1) if isinstance(b2, torch.Tensor) and b2.is_contiguous() else None
                    bi = weight_like(b2, (n2[1],))
                    if bi is None:
                        return None
                try:
                    # the result will be a column slice (row pitch > N): its shape must be a view of that
                    torch.empty_strided((m, n2[1]), (n2[1] + 16, 1), dtype=x.dtype, device="meta").view(
                        _concrete(s2.output.shape, self.env))
                except RuntimeError:
                    return None
                return w2.t(), wi, b2, bi, n2[1]

            group = []
            for s2 in [st] + [s for s in steps[si + 1: si + 1 + 24] if s.kind == "matmul"]:
                mem = member(s2)
                if mem is not None:
                    group.append((s2, mem))
                elif s2 is st:
                    return False
            if len(group) < 2:
                return False
            dt, isz = st.output.dtype, st.output.dtype.itemsize
            ntot = sum(mem[4] for _, mem in group)
            if (ntot * isz) % 16 or any((mem[4] * isz) % 16 for _, mem in group):
                return False
            # written by the preparation calls, ahead of every other call: never a buffer of the reuse pool
            wcat = torch.empty((ntot, kdim), dtype=dt, device=dev)
            bcat = torch.empty((ntot,), dtype=dt, device=dev) if e["bias"] is not None else None
            self.keep.append((wcat, bcat))
            obuf = pool.take(m * ntot * isz)
            owner[id(st.output)] = obuf
            cat = obuf[: m * ntot * isz].view(dt).view(m, ntot)
            off = 0
            for s2, (w2, wi, b2, bi, n2) in group:
                self._prepare_later(ops.copy(w2, out=wcat[off:off + n2], defer=True), wi)
                if bcat is not None:
                    self._prepare_later(ops.copy(b2, out=bcat[off:off + n2], defer=True), bi)
                val[id(s2.output)] = cat[:, off:off + n2].view(_concrete(s2.output.shape, self.env))
                rid = id(s2.output)
                last_use[id(st.output)] = max(last_use.get(id(st.output), si), last_use.get(rid, si))
                if s2 is not st:
                    skip.add(id(s2))
                off += n2
            epi = None
            if bcat is not None or e["act"] or e["alpha"] != 1.0:
                epi = ops.Epilogue(alpha=e["alpha"], bias=bcat, residual=None, act=e["act"] or "none")
            self._launch_later(ops.matmul(x, wcat.t(), epi, out=cat, defer=True))
            return True

        for si, st in enumerate(steps):
            k = st.kind
            if id(st) in skip:
                continue
            self._preparing = None
            if isinstance(st.attrs, dict) and st.attrs.get("prepared") and k in ("ew", "view") and id(st.output) not in out_ids:
                deps = set()
                for v in st.inputs:
                    if id(v) in input_ids:
                        deps.add(g.inputs.index(v))
                    else:
                        deps.update(prep_root(v) or ())
                self._preparing = sorted(deps)
                prep_deps[id(st.output)] = self._preparing
            if k == "matmul" and FUSE_PROJECTIONS and fused_projections(st, si):
                for buf in temps:
                    pool.give(buf)
                del temps[:]
                continue
            if k == "batch_matmul" and FUSE_ATTENTION and fused_attention(st):
                for buf in temps:
                    pool.give(buf)
                del temps[:]
                continue
            if k == "batch_matmul":
                ins = [batched_operand(val[id(v)]) for v in st.inputs]
            else:
                ins = [materialise(val[id(v)]) for v in st.inputs]
            if k == "view":
                before = len(temps)
                val[id(st.output)] = self._view(st, ins[0], contiguous)
                if len(temps) > before:
                    # the reshape needed a contiguous copy: the view now lives in that copy, which stays
                    # private to this instance (later views of it are not tracked for reuse)
                    self.keep.append(temps.pop())
            elif k == "constant":
                shape, v = _concrete(st.output.shape, self.env), st.attrs["value"]
                if isinstance(v, Expr):  # llh.scalar_cast of a symbol's value: this binding's number
                    v = evaluate(v, self.env)
                if isinstance(v, (list, tuple)):  # a dense constant spelt element by element (LLH text)
                    c = torch.tensor(v, dtype=st.output.dtype).reshape(shape).to(dev)
                else:
                    c = torch.full(shape, v, dtype=st.output.dtype, device=dev)
                self.keep.append(c)
                val[id(st.output)] = c
            elif k == "weight":
                val[id(st.output)] = self.weights.get(st.attrs["weight_file"], _concrete(st.output.shape, self.env), st.output.dtype)
            elif k == "ew":
                out = new_tensor(st.output)
                insts = st.attrs["insts"]
                if any(isinstance(x, Expr) for ins in insts for x in ins):
                    insts = [tuple(float(evaluate(x, self.env)) if isinstance(x, Expr) else x for x in ins) for ins in insts]
                prog = ops.make_program(insts, st.attrs["result"], st.attrs["integer"])
                if out.numel():
                    self._launch_later(ops.elementwise(prog, ins, tuple(out.shape), out.dtype, out=out, defer=True))
                val[id(st.output)] = out
            elif k in ("matmul", "batch_matmul", "conv"):
                e = epi_of(st)
                out = new_tensor(st.output)
                natural = _concrete(st.attrs["natural_shape"], self.env)
                bias = materialise(val[id(e["bias"])]) if e["bias"] is not None else None
                res = materialise(val[id(e["residual"])]) if e["residual"] is not None else None
                bias_rows = bool(e.get("bias_rows"))
                if bias is not None:
                    bias = contiguous(bias.reshape(-1) if bias.is_contiguous() else bias).reshape(-1)
                    if bias_rows:  # [B0,1,1,N] -> [B0,N]; the kernel then needs the 4-D shape of the product
                        full = _concrete(st.output.shape, self.env)
                        bias = bias.view(full[0], full[3])
                        natural = full
                if k == "conv" and st.attrs.get("layout", "NCHW") == "NHWC":
                    # operands and result are [N,H,W,C] / [F,KH,KW,C] / [N,OH,OW,F] tensors: their NCHW-shaped views
                    # are channels-last tensors, which is what the kernel for that memory layout takes
                    n_, oh_, ow_, f_ = natural
                    x4, w4 = ins[0].permute(0, 3, 1, 2), ins[1].permute(0, 3, 1, 2)
                    r4 = res.permute(0, 3, 1, 2) if res is not None else None
                    kernel_ok = CHANNELS_LAST and st.attrs["group"] == 1 and out.numel() and \
                        x4.shape[1] % (128 // out.dtype.itemsize) == 0 and f_ % 4 == 0 and w4.shape[2] * w4.shape[3] <= 64
                    if kernel_ok:
                        xc, wc = to_channels_last(st.inputs[0], x4), to_channels_last(st.inputs[1], w4)
                        kernel_ok = xc.data_ptr() % 16 == 0 and wc.data_ptr() % 16 == 0
                    if kernel_ok:
                        epi = None
                        if bias is not None or r4 is not None or e["act"] or e["alpha"] != 1.0:
                            epi = ops.Epilogue(alpha=e["alpha"], bias=bias, act=e["act"] or "none",
                                               residual=to_channels_last(e["residual"], r4) if r4 is not None else None)
                        self._launch_later(ops.conv2d(xc, wc, pad=st.attrs["pad"], stride=st.attrs["stride"],
                                                      dilation=st.attrs["dilation"], group=1, epilogue=epi,
                                                      out=out.view(natural).permute(0, 3, 1, 2), defer=True))
                    elif out.numel():
                        # shapes the channels-last kernel does not take: NCHW copies, the NCHW kernel, and a copy back
                        epi = None
                        if bias is not None or r4 is not None or e["act"] or e["alpha"] != 1.0:
                            epi = ops.Epilogue(alpha=e["alpha"], bias=bias, act=e["act"] or "none",
                                               residual=contiguous(r4) if r4 is not None else None)
                        nbytes = out.numel() * out.dtype.itemsize
                        buf = pool.take(nbytes)
                        temps.append(buf)
                        t4 = buf[:nbytes].view(out.dtype).view(n_, f_, oh_, ow_)
                        self._launch_later(ops.conv2d(contiguous(x4), contiguous(w4), pad=st.attrs["pad"], stride=st.attrs["stride"],
                                                      dilation=st.attrs["dilation"], group=st.attrs["group"], epilogue=epi,
                                                      out=t4, defer=True))
                        self._launch_later(ops.copy(t4.permute(0, 2, 3, 1), out=out.view(natural), defer=True))
                    val[id(st.output)] = out
                else:
                    cl = k == "conv" and self._channels_last_ok(st, ins, out, natural)
                    first = k == "conv" and not cl and self._first_layer_channels_last_ok(st, ins[0], ins[1], out, natural, res)
                    if res is not None and not cl:
                        res = contiguous(res)
                    epi = None
                    if bias is not None or res is not None or e["act"] or e["alpha"] != 1.0:
                        epi = ops.Epilogue(alpha=e["alpha"], bias=bias, residual=res, act=e["act"] or "none")
                    o = out.view(natural)
                    if k == "matmul":
                        call = ops.matmul(ins[0], ins[1], epi, out=o, defer=True)
                    elif k == "batch_matmul":
                        hm = head_merge(st, natural[0], natural[1], natural[2]) if (res is None and len(natural) == 3) else None
                        if hm is not None:
                            # the head merge that follows, [B0,B1,M,N] -> [B0,M,B1,N], is done by the kernel's stores
                            r1, b0, b1 = hm
                            o = out.view(-1).view(b0, natural[1], b1, natural[2]).permute(0, 2, 1, 3)
                            val[id(r1.output)] = o
                            skip.add(id(r1))
                        call = ops.batch_matmul(ins[0], ins[1], epi, out=o, defer=True)
                    elif cl:
                        xc = to_channels_last(st.inputs[0], ins[0])
                        wc = to_channels_last(st.inputs[1], ins[1])
                        if res is not None:
                            epi = ops.Epilogue(alpha=e["alpha"], bias=bias, residual=to_channels_last(e["residual"], res),
                                               act=e["act"] or "none")
                        n_, f_, oh_, ow_ = natural
                        out = out.view(-1).view(n_, oh_, ow_, f_).permute(0, 3, 1, 2)  # NCHW shape over NHWC memory
                        call = ops.conv2d(xc, wc, pad=st.attrs["pad"], stride=st.attrs["stride"], dilation=st.attrs["dilation"],
                                          group=1, epilogue=epi, out=out, defer=True)
                    else:
                        if first:
                            n_, f_, oh_, ow_ = natural
                            out = o = out.view(-1).view(n_, oh_, ow_, f_).permute(0, 3, 1, 2)  # NCHW shape over NHWC memory
                        call = ops.conv2d(contiguous(ins[0]), contiguous(ins[1]), pad=st.attrs["pad"], stride=st.attrs["stride"],
                                          dilation=st.attrs["dilation"], group=st.attrs["group"], epilogue=epi, out=o, defer=True)
                    if out.numel():
                        self._launch_later(call)
                    val[id(st.output)] = out
            elif k == "softmax":
                out = new_tensor(st.output)
                if out.numel():
                    self._launch_later(ops.softmax(contiguous(ins[0]), out=out, defer=True))
                val[id(st.output)] = out
            elif k == "layer_norm":
                out = new_tensor(st.output)
                rest = ins[1:]
                scale = contiguous(rest.pop(0)) if st.attrs.get("has_scale", True) and rest else None
                bias = contiguous(rest.pop(0)) if st.attrs.get("has_bias", True) and rest else None
                if out.numel():
                    self._launch_later(ops.layer_norm(contiguous(ins[0]), scale, bias, st.attrs["epsilon"], out=out, defer=True))
                val[id(st.output)] = out
            elif k == "reduce":
                out = new_tensor(st.output)
                x = contiguous(ins[0])
                axes = sorted(a % x.dim() for a in st.attrs["axis"])
                self._reduce(st.attrs["kind"], x, axes, out, pool)
                val[id(st.output)] = out
            elif k == "max_pool":
                out = new_tensor(st.output)
                a = st.attrs
                x = ins[0]
                if _is_channels_last(x) and x.shape[1] % (16 // x.dtype.itemsize) == 0 and x.data_ptr() % 16 == 0 and out.dim() == 4:
                    # a channels-last input gives a channels-last result: NCHW shape over NHWC memory
                    n_, c_, oh_, ow_ = out.shape
                    out = out.view(-1).view(n_, oh_, ow_, c_).permute(0, 3, 1, 2)
                else:
                    x = contiguous(x)
                if out.numel():
                    self._launch_later(ops.max_pool(x, a["kernel_shape"], pad=a["pad"], stride=a["stride"],
                                                    dilation=a["dilation"], init_zero=False, out=out, defer=True))
                val[id(st.output)] = out
            elif k == "avg_pool":
                out = new_tensor(st.output)
                x = ins[0] if _is_channels_last(ins[0]) else contiguous(ins[0])
                if out.numel():
                    self._launch_later(ops.global_avg_pool(x, out=out, defer=True))
                val[id(st.output)] = out
            elif k == "gather":
                out = new_tensor(st.output)
                if out.numel():
                    self._launch_later(ops.gather_rows(contiguous(ins[0]), contiguous(ins[1]), out=out, defer=True))
                val[id(st.output)] = out
            else:
                raise NotImplementedError(k)
            # buffers whose last reader has now been enqueued go back to the pool
            for buf in temps:
                pool.give(buf)
            del temps[:]
            for rid in [r for r in owner if last_use.get(r, si) <= si]:
                pool.give(owner.pop(rid))
        self._preparing = None
        # graph outputs
        self.output_plan = []
        for o in g.outputs:
            if isinstance(o, Value):
                t = materialise(val[id(o)])
                root = self._roots.get(t.untyped_storage().data_ptr())
                if root is None or root[0] != "out" or not t.is_contiguous():
                    # an output that aliases an input or an intermediate view: materialise it per call
                    fresh = torch.empty(tuple(t.shape), dtype=t.dtype, device=dev)
                    self._register_root("out", n_out_bufs, fresh)
                    self.out_buffers.append(fresh)
                    if fresh.numel():
                        self._launch_later(ops.copy(t, out=fresh, defer=True))
                    self.output_plan.append(("tensor", n_out_bufs, tuple(fresh.shape), tuple(fresh.stride()), 0))
                    n_out_bufs += 1
                else:
                    off = (t.data_ptr() - root[2]) // t.dtype.itemsize
                    self.output_plan.append(("tensor", root[1], tuple(t.shape), tuple(t.stride()), off))
            elif isinstance(o, Expr):
                self.output_plan.append(("int", evaluate(o, self.env)))
            else:
                self.output_plan.append(("const", o))
        self.out_specs = [(tuple(b.shape), b.dtype) for b in self.out_buffers]
        self._first = True
        self._runs = 0
        self._last_in_ptrs = None
        self._graph = None
        self._graph_failed = False
        self._plan = None
        self._block = None

    def _view(self, st, t, contiguous):
        a = st.attrs
        op = a["op"]
        if op in ("identity",):
            return t
        if op in ("reshape", "flatten"):
            shape = _concrete(st.output.shape, self.env)
            try:
                return t.view(shape)
            except RuntimeError:
                return _LazyReshape(t, shape)
        if op == "transpose":
            return t.permute(*a["perms"])
        if op == "broadcast_to":
            return t.expand(*_concrete(st.output.shape, self.env))
        if op == "stride_slice":
            idx = tuple(slice(evaluate(s, self.env) if isinstance(s, Expr) else s, evaluate(e, self.env) if isinstance(e, Expr) else e,
                              st_) for s, e, st_ in zip(a["start"], a["end"], a["stride"]))
            return t[idx]
        if op == "extract":
            if t.dim() == 1:  # one element of a vector stays a tensor<1> (LLHinfersymbolShape.cpp:513-516)
                i = a["index"] % t.shape[0]
                return t[i:i + 1]
            return t[a["index"]]
        raise NotImplementedError(op)

    def _reduce(self, kind, x, axes, out, pool):
        """The kernel reduces one run of adjacent axes; split axes are reduced run by run, innermost first."""
        runs = []
        for a in axes:
            if runs and runs[-1][-1] == a - 1:
                runs[-1].append(a)
            else:
                runs.append([a])
        cur = x
        for i, run in enumerate(reversed(runs)):
            last = i == len(runs) - 1
            shape = [s for d, s in enumerate(cur.shape) if d not in run]
            if last:
                dst = out.view(shape) if out.numel() else out
            else:
                n = 1
                for s in shape:
                    n *= s
                buf = pool.take(n * x.dtype.itemsize)
                self.keep.append(buf)  # partial results stay private to this step
                dst = buf[: n * x.dtype.itemsize].view(x.dtype).view(shape)
            if dst.numel():
                self._launch_later(ops.reduce(kind, cur, run, out=dst, defer=True))
            cur = dst

    # ---- execution ----
    def _patch(self, in_ptrs, out_ptrs):
        for ref, kind, idx, delta in self.patches:
            p = (in_ptrs[idx] if kind == "in" else out_ptrs[idx]) + delta
            ref.desc.data = p
            ref.desc.base = p

    def _results(self, outs):
        results = []
        for spec in self.output_plan:
            if spec[0] == "tensor":
                _, idx, shape, stride, off = spec
                t = outs[idx]
                results.append(t if (tuple(t.shape) == shape and off == 0) else t.as_strided(shape, stride, off))
            else:
                results.append(spec[1])
        return results

    def run(self, inputs):
        if self._graph is not None:
            res = self._replay(inputs)
            if res is not None:
                return res
        if self._first:
            outs = self.out_buffers
            self._first = False
        else:
            outs = [torch.empty(s, dtype=d, device=self.device) for s, d in self.out_specs]
        in_ptrs = [t.data_ptr() for t in inputs]
        stream = C.current_stream(self.device)
        if self.prep_calls:
            key = [(in_ptrs[i], inputs[i]._version) for i in self.prep_inputs]
            if key != self._prep_key:
                self._patch(in_ptrs, [t.data_ptr() for t in outs])
                for c in self.prep_calls:
                    c.launch(stream)
                self._prep_key = key
        if self._plan is not None:
            blk = self._block
            last = self._last_in_ptrs
            if in_ptrs != last:
                for k, p in enumerate(in_ptrs):
                    if p != last[k]:
                        blk.set_pointer(k, p)
                self._last_in_ptrs = in_ptrs
            n_in = len(in_ptrs)
            for k, t in enumerate(outs):
                blk.set_pointer(n_in + k, t.data_ptr())
            try:
                self._plan.run(blk, stream)
            except C.LlcHipError as err:
                if err.status != C.ERR_LAYOUT:
                    raise
                # an input at another address modulo 16 than when the plan was recorded (a view with a storage offset):
                # the recorded kernel choices do not apply; the per-kernel entry points choose again for these addresses
                self._patch(in_ptrs, [t.data_ptr() for t in outs])
                for c in self.calls:
                    c.launch(stream)
            return self._results(outs)
        self._patch(in_ptrs, [t.data_ptr() for t in outs])
        if USE_PLAN and not USE_GRAPHS:
            # this run launches every kernel as usual and records the calls on the way
            plan = Plan()
            for t in inputs:
                plan.declare_io(t, False)
            for t in outs:
                plan.declare_io(t, True)
            with plan.recording():
                for c in self.calls:
                    c.launch(stream)
            self._block = ParamBlock(list(inputs) + list(outs))
            self._plan = plan
            self._last_in_ptrs = in_ptrs
            return self._results(outs)
        for c in self.calls:
            c.launch(stream)
        # After two eager runs the launch sequence is recorded as a HIP graph: the host then pays one replay
        # instead of one launch per kernel.  Inputs whose address did not change between those runs (weights)
        # are used in place, the others are copied into fixed staging tensors before every replay.
        self._runs += 1
        if USE_GRAPHS and self._graph is None and not self._graph_failed and self._runs >= 2 and \
                len(self.calls) >= MIN_CALLS_FOR_GRAPH and self._last_in_ptrs is not None:
            self._capture(inputs, in_ptrs)
        self._last_in_ptrs = in_ptrs
        return self._results(outs)

    def _capture(self, inputs, in_ptrs):
        dev = self.device
        try:
            stable = [a == b for a, b in zip(in_ptrs, self._last_in_ptrs)]
            staging = [None if st else torch.empty_strided(tuple(t.shape), tuple(t.stride()), dtype=t.dtype, device=dev)
                       for st, t in zip(stable, inputs)]
            g_outs = [torch.empty(s, dtype=d, device=dev) for s, d in self.out_specs]
            g_in_ptrs = [p if s is None else s.data_ptr() for p, s in zip(in_ptrs, staging)]
            self._patch(g_in_ptrs, [t.data_ptr() for t in g_outs])
            side = torch.cuda.Stream(device=dev)
            side.wait_stream(torch.cuda.current_stream(dev))
            # One run on the capture stream ahead of the capture: the library keeps scratch memory per stream and
            # cannot allocate while a stream is being captured.  The graph then addresses that stream's buffer, so the
            # stream stays with the instance and nothing else is ever issued to it.
            with torch.cuda.stream(side):
                sh = C.current_stream(dev)
                for c in self.calls:
                    c.launch(sh)
            side.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=side):
                sh = C.current_stream(dev)
                for c in self.calls:
                    c.launch(sh)
            self._graph, self._g_staging, self._g_outs, self._g_in_ptrs = graph, staging, g_outs, g_in_ptrs
            self._g_stream = side
        except Exception:  # capture is an optimisation: fall back to per-kernel launches for this instance
            self._graph_failed = True
            self._graph = None

    def _replay(self, inputs):
        """Returns None when a weight moved since capture (the caller then runs the eager path)."""
        for t, st, p in zip(inputs, self._g_staging, self._g_in_ptrs):
            if st is None:
                if t.data_ptr() != p:
                    return None
            else:
                st.copy_(t, non_blocking=True)
        self._graph.replay()
        # the graph writes into fixed buffers; callers get their own tensors, as in the eager path
        return self._results([t.clone() for t in self._g_outs])


class ExecutionEngine:
    """Base of the reference's engines (engine.py:15-26): holds the compiled artefact, is callable."""

    def __init__(self, graph):
        self.graph = graph
        self.steps = make_plan(graph)
        self.instances = {}
        self._fast = {}
        self._weights = None

    def run(self, *args):
        raise NotImplementedError

    def __call__(self, *args):
        return self.run(*args)


class Torch_ExecutionEngine(ExecutionEngine):
    def trans_to_tensor(self, *args):
        """The reference wraps every torch tensor in its C++ Tensor descriptor here (engine.py:34-54);
        this build keeps the torch tensor and builds descriptors once per specialised instance."""
        inputs = []
        for arg in args:
            if isinstance(arg, torch.Tensor):
                if arg.dtype not in TORCH_DTYPE_TO_TYPE:
                    raise TypeError("Unsupported type: %s" % arg.dtype)
                inputs.append(arg)
            elif isinstance(arg, int) or arg is None:
                pass
            else:
                raise TypeError("Unsupported type: %s" % type(arg))
        return inputs

    def bind_symbols(self, args, inputs):
        g = self.graph
        env = {}
        ints = [a for a in args if isinstance(a, int) and not isinstance(a, bool)]
        if len(ints) != len(g.symbol_args):
            raise ValueError("expected %d symbol values (python ints), got %d" % (len(g.symbol_args), len(ints)))
        for name, v in zip(g.symbol_args, ints):
            env[name] = v
        for name, (i, d) in g.symbol_sources.items():
            env.setdefault(name, inputs[i].shape[d])
        derived = self._derived_symbols()
        if derived[0]:
            self._solve_derived(env, inputs, derived)
        return env

    def _derived_symbols(self):
        """Symbols the graph uses that no int argument and no input dim states directly: a partition of a dynamically
        shaped graph may see a symbol only inside its inputs' extents (every tensor it gets is a strided convolution's
        result, of extent (s - 1) // 2 + 1).  Returns (names, [(input index, dim, extent expression)]), computed once."""
        d = getattr(self, "_derived", None)
        if d is None:
            g = self.graph
            known = set(g.symbol_args) | set(g.symbol_sources)
            names = sorted(n for n in g.symbols() if n not in known)
            eqs = []
            if names:
                for i, v in enumerate(g.inputs):
                    for k, e in enumerate(v.shape):
                        if isinstance(e, Expr) and e.kind != "sym" and any(n in names for n in e.symbols()):
                            eqs.append((i, k, e))
            d = self._derived = (names, eqs, {})
        return d

    def _solve_derived(self, env, inputs, derived):
        """Values for the derived symbols from the extents that contain them.  The graph's other extents are functions
        of its inputs' extents, so ANY value that reproduces those gives the right shapes everywhere; extents are
        non-decreasing in their symbols (window arithmetic: sums, products and floor divisions by positive numbers),
        so each is found by bisection on an equation with one unknown left, and every equation is checked at the end."""
        names, eqs, cache = derived
        key = tuple(inputs[i].shape[k] for i, k, _ in eqs)
        found = cache.get(key)
        if found is None:
            trial = dict(env)
            left = [n for n in names if n not in trial]
            progress = True
            while left and progress:
                progress = False
                for (i, k, e), want in zip(eqs, key):
                    unknown = [n for n in e.symbols() if n not in trial]
                    if len(unknown) != 1:
                        continue
                    n, lo, hi = unknown[0], 0, 1
                    while evaluate(e, dict(trial, **{n: hi})) < want and hi < (1 << 40):
                        hi *= 2
                    while lo < hi:  # smallest value whose extent reaches `want`
                        mid = (lo + hi) // 2
                        if evaluate(e, dict(trial, **{n: mid})) < want:
                            lo = mid + 1
                        else:
                            hi = mid
                    trial[n] = lo
                    left.remove(n)
                    progress = True
            ok = not left and all(evaluate(e, trial) == want for (_, _, e), want in zip(eqs, key))
            found = cache[key] = {n: trial[n] for n in names} if ok else False
        if found is False:
            missing = [n for n in names if n not in env]
            raise KeyError("symbol %s is not bound by any input of this call" % ", ".join(missing))
        for n, v in found.items():
            env.setdefault(n, v)

    def save_plan(self, path, *args):
        """Runs the graph for `args` (so that the plan for those extents exists and is recorded), writes that plan
        to `path` and a description of its parameter block to `path + ".json"`: the tensors in block order
        (inputs, then outputs) with type, shape and strides, the symbol values it is specialised for, and the
        output views.  Another process loads the file with `Plan.load` (or `llc_plan_load` from C) and runs it
        with a block of that layout: the counterpart of the reference's compile-to-shared-object followed by
        `ExecutionEngine.load` (src/Compiler/Compiler.cpp:306-330, llcompiler/executor/engine.py:15-26).  Weights
        that are graph inputs stay parameters of the block; weights taken from .npy files are part of the file.
        Returns the description."""
        import json
        if not USE_PLAN or USE_GRAPHS:
            raise RuntimeError("save_plan needs the recorded-plan execution path (engine.USE_PLAN)")
        self.run(*args)
        self.run(*args)
        tensors = [a for a in self.trans_to_tensor(*args)]
        env = self.bind_symbols(args, tensors)
        device = tensors[0].device if tensors else torch.device("cuda", torch.cuda.current_device())
        key = (tuple(sorted(env.items())), tuple((tuple(t.shape), tuple(t.stride())) for t in tensors), device.index,
               _alias_signature(tensors))
        inst = self.instances[key]
        if inst._plan is None:
            raise RuntimeError("the instance has no recorded plan")
        if inst.prep_calls:
            torch.cuda.synchronize(device)  # prepared weight copies are part of the file: they must be complete
        inst._plan.save(path)

        def describe(t):
            return {"dtype": str(t.dtype).replace("torch.", ""), "shape": list(t.shape), "stride": list(t.stride())}
        meta = {"symbols": {k: int(v) for k, v in sorted(env.items())},
                "inputs": [dict(describe(t), name=v.name) for v, t in zip(self.graph.inputs, tensors)],
                "outputs": [{"dtype": str(d).replace("torch.", ""), "shape": list(s), "stride": list(torch.empty(s, device="meta").stride())}
                            for s, d in inst.out_specs],
                "results": [list(spec) if spec[0] != "tensor" else
                            {"output": spec[1], "shape": list(spec[2]), "stride": list(spec[3]), "offset": spec[4]}
                            for spec in inst.output_plan],
                "steps": int(inst._plan.num_steps)}
        with open(str(path) + ".json", "w") as f:
            json.dump(meta, f, indent=1)
        return meta

    def bind_leading(self, tensors):
        """run() with `tensors` fixed as the first arguments (the parameters an ahead-of-time compiled module
        passes with every call): their part of the call signature is computed once, not per call."""
        lead = tuple(tensors)
        lead_key = tuple((a.dtype, a.shape, a.stride(), a.device) for a in lead)
        lead_list = list(lead)
        fast = self._fast

        def run(*args):
            key = lead_key + tuple(a if not isinstance(a, torch.Tensor) else (a.dtype, a.shape, a.stride(), a.device) for a in args)
            hit = fast.get(key)
            if hit is None:
                return self.run(*lead, *args)
            results = hit.run(lead_list + [a for a in args if isinstance(a, torch.Tensor)])
            if getattr(self.graph, "single_output", len(results) == 1) and len(results) == 1:
                return results[0]
            return results

        return run

    def run(self, *args):
        # ([inputs...]) case, as in the reference
        if len(args) == 1 and isinstance(args[0], (list, tuple)):
            args = tuple(args[0])
        # a call whose arguments look exactly like an earlier, validated one (same ints, same tensor types,
        # shapes, strides and devices) goes straight to that call's instance
        fast_key = tuple(a if not isinstance(a, torch.Tensor) else (a.dtype, a.shape, a.stride(), a.device) for a in args)
        hit = self._fast.get(fast_key)
        if hit is not None:
            results = hit.run([a for a in args if isinstance(a, torch.Tensor)])
            if getattr(self.graph, "single_output", len(results) == 1) and len(results) == 1:
                return results[0]
            return results
        inputs = self.trans_to_tensor(*args)
        g = self.graph
        if len(inputs) != len(g.inputs):
            raise ValueError("expected %d tensors, got %d" % (len(g.inputs), len(inputs)))
        env = self.bind_symbols(args, inputs)
        for v, t in zip(g.inputs, inputs):
            want = _concrete(v.shape, env)
            if tuple(t.shape) != want or t.dtype != v.dtype:
                raise ValueError("input %s: expected %s %s, got %s %s" % (v.name, want, v.dtype, tuple(t.shape), t.dtype))
        device = None
        for t in inputs:
            if not t.is_cuda:
                raise RuntimeError("llcompiler_amd executes on the GPU only; got a %s tensor (no CPU fallback)" % t.device)
            device = t.device
        if device is None:
            device = torch.device("cuda", torch.cuda.current_device())
        key = (tuple(sorted(env.items())), tuple((tuple(t.shape), tuple(t.stride())) for t in inputs), device.index,
               _alias_signature(inputs))
        inst = self.instances.get(key)
        if inst is None:
            C.init(device.index or 0)
            if self._weights is None or self._weights.device != device:
                self._weights = WeightStore(device)
            inst = Instance(g, self.steps, env, inputs, device, self._weights)
            self.instances[key] = inst
        if not key[3]:
            # (an instance built from inputs that share memory is only valid while they do: such calls keep
            # coming this way, where the key checks it)
            self._fast[fast_key] = inst
        results = inst.run(inputs)
        if getattr(g, "single_output", len(results) == 1) and len(results) == 1:
            return results[0]
        return results
