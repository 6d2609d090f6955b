"""Python handle of a recorded plan (llc_plan_t) and of the packed parameter block it is run from.

The block is the reference's `main(void** params)` argument (src/Compiler/Execution.cpp:21-66): slot 0 holds
the symbol values (or NULL), then five slots per tensor, inputs first: base, data, &offset, size[], stride[].
"""
import contextlib
import ctypes
import os
import weakref

from .. import _capi as C


class ParamBlock:
    """The packed block for a fixed list of tensor layouts; only the base/data slots change between calls."""

    def __init__(self, tensors, symbols=None):
        n = len(tensors)
        self.n = n
        self.arr = (ctypes.c_void_p * (1 + 5 * n))()
        self._keep = []
        if symbols:
            sym = C.i64_array(symbols)
            self._keep.append(sym)
            self.arr[0] = ctypes.addressof(sym)
        for k, t in enumerate(tensors):
            rank = t.dim()
            off = ctypes.c_size_t(0)  # data_ptr() already includes the storage offset
            size = (ctypes.c_size_t * max(rank, 1))(*t.shape)
            stride = (ctypes.c_size_t * max(rank, 1))(*t.stride())
            self._keep += [off, size, stride]
            s = 1 + 5 * k
            self.arr[s + 2] = ctypes.addressof(off)
            self.arr[s + 3] = ctypes.addressof(size)
            self.arr[s + 4] = ctypes.addressof(stride)
            self.set_pointer(k, t.data_ptr())

    def set_pointer(self, k, ptr):
        s = 1 + 5 * k
        self.arr[s] = ptr
        self.arr[s + 1] = ptr


class Plan:
    """Owns an llc_plan_t.  Usage: declare the tensors of the block, record the kernel calls once, run."""

    def __init__(self, _handle=None):
        self._lib = C.lib()
        h = _handle
        if h is None:
            h = ctypes.c_void_p()
            C.check(self._lib.llc_plan_create(ctypes.byref(h)))
        self.handle = h
        self._refs = []
        weakref.finalize(self, self._lib.llc_plan_destroy, h)

    def save(self, path):
        """Writes the recorded plan to `path`: steps, declared tensors, and the device memory the steps address
        outside those tensors (constants with their contents, intermediates by size)."""
        C.check(self._lib.llc_plan_save(self.handle, os.fsencode(path)))

    @classmethod
    def load(cls, path):
        """A plan read back from a file written by `save`, with memory of its own on the current device."""
        h = ctypes.c_void_p()
        C.check(C.lib().llc_plan_load(os.fsencode(path), ctypes.byref(h)))
        return cls(_handle=h)

    def declare_io(self, t, is_output):
        r = C.tensor_ref(t)
        self._refs.append(r)
        C.check(self._lib.llc_plan_declare_io(self.handle, 1 if is_output else 0, r.ptr))

    def expect_symbols(self, values):
        arr = C.i64_array(values)
        C.check(self._lib.llc_plan_expect_symbols(self.handle, arr, len(values)))

    def alloc(self, nbytes):
        p = ctypes.c_void_p()
        C.check(self._lib.llc_plan_alloc(self.handle, nbytes, ctypes.byref(p)))
        return p.value

    def upload(self, host_ptr, nbytes):
        p = ctypes.c_void_p()
        C.check(self._lib.llc_plan_upload(self.handle, host_ptr, nbytes, ctypes.byref(p)))
        return p.value

    def load_npy(self, path, expect_dtype=-1):
        """Uploads the data of a .npy file into memory owned by this plan; returns (device pointer, type code, shape)."""
        desc = C.LlcTensor()
        size = (ctypes.c_size_t * C.LLC_MAX_RANK)()
        stride = (ctypes.c_size_t * C.LLC_MAX_RANK)()
        C.check(self._lib.llc_plan_load_npy(self.handle, os.fsencode(path), expect_dtype, ctypes.byref(desc), size, stride))
        return desc.data or 0, int(desc.type), tuple(size[i] for i in range(desc.rank))

    @contextlib.contextmanager
    def recording(self):
        C.check(self._lib.llc_plan_begin(self.handle))
        try:
            yield self
        except BaseException:
            self._lib.llc_plan_end(self.handle)
            raise
        C.check(self._lib.llc_plan_end(self.handle))

    @property
    def num_steps(self):
        return self._lib.llc_plan_num_steps(self.handle)

    @property
    def num_params(self):
        return self._lib.llc_plan_num_params(self.handle)

    def run(self, block, stream):
        st = self._lib.llc_hip_run(self.handle, block.arr, stream)
        if st != 0:
            C.check(st)
