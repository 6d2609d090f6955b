"""ctypes binding of libllc_hip.so: the C-ABI declared in include/llc_hip.h.

Torch only supplies device memory and the current stream; every computation goes through the
library.  There is no fallback: if the library is missing or a call fails, an exception is raised.
"""
import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libllc_hip.so")
ENTRY_LIB_PATH = os.path.join(_HERE, "lib", "libllc_entry.so")

LLC_MAX_RANK = 8
# element type codes: 0-6 are the reference's enum Type (include/llcompiler/Compiler/Tensor.h:25-33)
INT8, INT16, INT32, INT64, FLOAT32, DOUBLE64, INT1, BFLOAT16, FLOAT16 = range(9)
TORCH_DTYPE_TO_TYPE = {
    torch.int8: INT8, torch.int16: INT16, torch.int32: INT32, torch.int64: INT64, torch.float32: FLOAT32,
    torch.float64: DOUBLE64, torch.bool: INT1, torch.bfloat16: BFLOAT16, torch.float16: FLOAT16,
}
TYPE_TO_TORCH_DTYPE = {v: k for k, v in TORCH_DTYPE_TO_TYPE.items()}

OK, ERR_BAD_ARG, ERR_DTYPE, ERR_SHAPE, ERR_LAYOUT, ERR_UNSUPPORTED, ERR_HIP, ERR_NO_DEVICE, ERR_TOO_LARGE = \
    0, -1, -2, -3, -4, -5, -6, -7, -8
ACT_NONE, ACT_RELU, ACT_GELU = 0, 1, 2
REDUCE_SUM, REDUCE_MAX, REDUCE_MIN = 0, 1, 2

EW_OPCODES = {
    "abs": 0, "sqrt": 1, "exp": 2, "relu": 3, "rsqrt": 4, "neg": 5, "gelu": 6, "tanh": 7, "erf": 8, "sigmoid": 9,
    "log": 10, "recip": 11, "mov": 15,
    "add": 16, "sub": 17, "mul": 18, "div": 19, "max": 20, "min": 21, "pow": 22,
    # 32 + CompareKind (include/llcompiler/Dialect/LLH/IR/LLHEnums.td:111-116)
    "eq": 33, "ge": 34, "le": 35, "gt": 36, "lt": 37, "ne": 38,
    "where": 48,
}
EW_MAX_REGS, EW_MAX_INPUTS, EW_MAX_INSTS, EW_IN0, EW_IMM = 4, 6, 24, 16, 64


class LlcTensor(ctypes.Structure):
    _fields_ = [("data", ctypes.c_void_p), ("base", ctypes.c_void_p), ("type", ctypes.c_size_t),
                ("offset", ctypes.c_size_t), ("rank", ctypes.c_size_t),
                ("size", ctypes.POINTER(ctypes.c_size_t)), ("stride", ctypes.POINTER(ctypes.c_size_t))]


class LlcEpilogue(ctypes.Structure):
    _fields_ = [("alpha", ctypes.c_float), ("bias", ctypes.POINTER(LlcTensor)),
                ("residual", ctypes.POINTER(LlcTensor)), ("act", ctypes.c_int)]


class LlcConvAttrs(ctypes.Structure):
    _fields_ = [("dilation", ctypes.c_int64 * 2), ("kernel_shape", ctypes.c_int64 * 2), ("pad", ctypes.c_int64 * 4),
                ("stride", ctypes.c_int64 * 2), ("group", ctypes.c_int64)]


class LlcPoolAttrs(ctypes.Structure):
    _fields_ = [("dilation", ctypes.c_int64 * 2), ("kernel_shape", ctypes.c_int64 * 2), ("pad", ctypes.c_int64 * 4),
                ("stride", ctypes.c_int64 * 2), ("init_zero", ctypes.c_int32)]


class LlcEwInst(ctypes.Structure):
    _fields_ = [("op", ctypes.c_int32), ("dst", ctypes.c_int32), ("a", ctypes.c_int32), ("b", ctypes.c_int32),
                ("c", ctypes.c_int32), ("imm", ctypes.c_float)]


class LlcEwProgram(ctypes.Structure):
    _fields_ = [("n_insts", ctypes.c_int32), ("result", ctypes.c_int32), ("integer", ctypes.c_int32),
                ("insts", LlcEwInst * EW_MAX_INSTS)]


# every symbol include/llc_hip.h declares
EXPORTS = [
    "llc_hip_abi_version", "llc_hip_init", "llc_hip_last_error", "llc_hip_status_string", "llc_hip_scratch_bytes",
    "llc_hip_trim", "llc_hip_matmul",
    "llc_hip_matmul_static",
    "llc_hip_batch_matmul", "llc_hip_conv2d", "llc_hip_elementwise", "llc_hip_reduce", "llc_hip_softmax",
    "llc_hip_layer_norm", "llc_hip_max_pool", "llc_hip_global_avg_pool", "llc_hip_transpose",
    "llc_hip_stride_slice", "llc_hip_broadcast_to", "llc_hip_copy", "llc_hip_gather_rows", "llc_hip_convert",
    "llc_hip_attention",
    "llc_hip_unpack_params",
    "llc_plan_create", "llc_plan_destroy", "llc_plan_alloc", "llc_plan_upload", "llc_plan_declare_io",
    "llc_plan_expect_symbols", "llc_plan_begin", "llc_plan_end", "llc_plan_num_steps", "llc_plan_num_params",
    "llc_hip_run", "llc_hip_bind_entry", "llc_hip_entry", "llc_hip_entry_status",
    "llc_npy_info", "llc_plan_load_npy", "llc_plan_save", "llc_plan_load",
    "llc_plan_num_io", "llc_plan_io_info", "llc_hip_download",
]


class LlcHipError(RuntimeError):
    def __init__(self, status, message):
        super().__init__("llc_hip error %d: %s" % (status, message))
        self.status = status


_lib = None


def lib():
    """Loads the kernel library.  Raises if it has not been built: there is no other path."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError("%s is missing: build it with `python -m llcompiler_amd.build` "
                               "(there is no CPU or eager fallback)" % LIB_PATH)
        L = ctypes.CDLL(LIB_PATH)
        L.llc_hip_last_error.restype = ctypes.c_char_p
        L.llc_hip_status_string.restype = ctypes.c_char_p
        L.llc_hip_status_string.argtypes = [ctypes.c_int]
        P = ctypes.POINTER
        T = P(LlcTensor)
        vp = ctypes.c_void_p
        i64p = P(ctypes.c_int64)
        L.llc_hip_matmul.argtypes = [T, T, P(LlcEpilogue), T, vp]
        L.llc_hip_matmul_static.argtypes = [T, T, P(LlcEpilogue), T, vp]
        L.llc_hip_batch_matmul.argtypes = [T, T, P(LlcEpilogue), T, vp]
        L.llc_hip_conv2d.argtypes = [T, T, P(LlcConvAttrs), P(LlcEpilogue), T, vp]
        L.llc_hip_elementwise.argtypes = [P(LlcEwProgram), P(T), ctypes.c_size_t, T, vp]
        L.llc_hip_reduce.argtypes = [ctypes.c_int, T, i64p, ctypes.c_size_t, T, vp]
        L.llc_hip_softmax.argtypes = [T, T, vp]
        L.llc_hip_layer_norm.argtypes = [T, T, T, ctypes.c_double, T, vp]
        L.llc_hip_max_pool.argtypes = [T, P(LlcPoolAttrs), T, vp]
        L.llc_hip_global_avg_pool.argtypes = [T, T, vp]
        L.llc_hip_transpose.argtypes = [T, i64p, T, vp]
        L.llc_hip_stride_slice.argtypes = [T, i64p, i64p, i64p, T, vp]
        L.llc_hip_broadcast_to.argtypes = [T, T, vp]
        L.llc_hip_copy.argtypes = [T, T, vp]
        L.llc_hip_gather_rows.argtypes = [T, T, T, vp]
        L.llc_hip_convert.argtypes = [T, T, vp]
        L.llc_hip_attention.argtypes = [T, T, T, T, ctypes.c_float, T, vp]
        L.llc_hip_init.argtypes = [ctypes.c_int]
        L.llc_hip_scratch_bytes.argtypes = [ctypes.c_int, P(ctypes.c_size_t), P(ctypes.c_size_t)]
        L.llc_hip_trim.argtypes = [ctypes.c_int]
        L.llc_hip_unpack_params.argtypes = [P(vp), ctypes.c_size_t, P(ctypes.c_size_t), P(ctypes.c_size_t), T,
                                            P(i64p)]
        L.llc_plan_create.argtypes = [P(vp)]
        L.llc_plan_destroy.argtypes = [vp]
        L.llc_plan_alloc.argtypes = [vp, ctypes.c_size_t, P(vp)]
        L.llc_plan_upload.argtypes = [vp, vp, ctypes.c_size_t, P(vp)]
        L.llc_plan_declare_io.argtypes = [vp, ctypes.c_int, T]
        L.llc_plan_expect_symbols.argtypes = [vp, i64p, ctypes.c_size_t]
        L.llc_plan_begin.argtypes = [vp]
        L.llc_plan_end.argtypes = [vp]
        L.llc_plan_num_steps.argtypes = [vp]
        L.llc_plan_num_steps.restype = ctypes.c_int64
        L.llc_plan_num_params.argtypes = [vp]
        L.llc_plan_num_params.restype = ctypes.c_int64
        L.llc_hip_run.argtypes = [vp, P(vp), vp]
        L.llc_hip_bind_entry.argtypes = [vp, vp]
        L.llc_hip_entry.argtypes = [P(vp)]
        L.llc_hip_entry.restype = None
        szp = P(ctypes.c_size_t)
        L.llc_npy_info.argtypes = [ctypes.c_char_p, ctypes.c_int, szp, szp, szp, szp]
        L.llc_plan_load_npy.argtypes = [vp, ctypes.c_char_p, ctypes.c_int, T, szp, szp]
        L.llc_plan_save.argtypes = [vp, ctypes.c_char_p]
        L.llc_plan_load.argtypes = [ctypes.c_char_p, P(vp)]
        L.llc_plan_num_io.argtypes = [vp, szp, szp]
        L.llc_plan_io_info.argtypes = [vp, ctypes.c_size_t, T, szp, szp]
        L.llc_hip_download.argtypes = [vp, vp, ctypes.c_size_t, vp]
        _lib = L
    return _lib


def check(status):
    if status != 0:
        raise LlcHipError(status, lib().llc_hip_last_error().decode("utf-8", "replace"))


_initialised = set()


def init(device=0):
    if device not in _initialised:
        check(lib().llc_hip_init(device))
        _initialised.add(device)


class TensorRef:
    """Keeps an LlcTensor and the ctypes arrays it points to alive together."""

    __slots__ = ("desc", "_size", "_stride", "_keep")

    def __init__(self, data_ptr, dtype_code, shape, stride, keep=None):
        n = len(shape)
        self._size = (ctypes.c_size_t * max(n, 1))(*shape)
        self._stride = (ctypes.c_size_t * max(n, 1))(*stride)
        self.desc = LlcTensor(data_ptr, data_ptr, dtype_code, 0, n, self._size, self._stride)
        self._keep = keep

    @property
    def ptr(self):
        return ctypes.pointer(self.desc)


def tensor_ref(t, shape=None, stride=None):
    """Descriptor of a torch tensor (or of a view of it given by shape/stride, in elements).

    `data` is data_ptr() (which already includes the storage offset) and `offset` is 0: the
    reference passes storage_offset again (llcompiler/executor/engine.py:38-46), which double
    counts it for views."""
    if t is None:
        return None
    code = TORCH_DTYPE_TO_TYPE.get(t.dtype)
    if code is None:
        raise TypeError("Unsupported type: %s" % t.dtype)
    return TensorRef(t.data_ptr(), code, tuple(t.shape) if shape is None else tuple(shape),
                     tuple(t.stride()) if stride is None else tuple(stride), keep=t)


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def current_stream(device):
    """torch's current HIP stream on `device` as a handle for the C-ABI.  The raw accessor skips the Stream object
    that torch.cuda.current_stream builds on every call (4 us, a third of a small compiled graph's host time)."""
    if _raw_stream is not None:
        idx = device.index if isinstance(device, torch.device) else device
        if idx is None:
            idx = torch.cuda.current_device()
        return ctypes.c_void_p(_raw_stream(idx))
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def i64_array(values):
    return (ctypes.c_int64 * max(len(values), 1))(*[int(v) for v in values])
