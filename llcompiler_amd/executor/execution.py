"""`Tensor` and `Execution` with the surface of the reference's pybind classes, over plan files.

The reference binds `Tensor(data, base, type, offset, size, stride)` (src/Pybind/Entrance.cpp:70-92; the struct is
include/llcompiler/Compiler/Tensor.h:36-48) and `Execution` with `load(file)`, `run(inputs, outputs)` and
`run_with_symbols(symbols, inputs, outputs)` (Entrance.cpp:113-119; src/Compiler/Execution.cpp:10-66): `load`
dlopens the compiled shared object, `run` packs one pointer array and calls its `main(void**)`.  Here the file is
a plan written by `llc_plan_save` / `Torch_ExecutionEngine.save_plan`, `load` is `llc_plan_load`, and `run` packs
the same array (slot 0 the symbol values or NULL, then base, data, &offset, size[], stride[] per tensor, inputs
first) and calls `llc_hip_run` with this object's plan handle, so that
llcompiler/executor/engine.py:34-78 works against these classes as it is written.  `data` and `base` are device
addresses; the element at index i is at data + (offset + sum i_k stride_k) elements, as in llc_tensor.  Every
object owns its plan: any number of them run side by side (on different streams too).
"""
import ctypes
import os

from .. import _capi as C


class Tensor:
    """Non-owning descriptor (Tensor.h:35: "does not allocate")."""

    def __init__(self, data, base, type, offset, size, stride):
        self.data, self.base, self.type, self.offset = int(data), int(base), int(type), int(offset)
        self.size, self.stride = [int(s) for s in size], [int(s) for s in stride]
        if len(self.size) != len(self.stride):
            raise ValueError("size and stride differ in length")

    def print(self):
        print("Tensor(data=0x%x, base=0x%x, type=%d, offset=%d, size=%s, stride=%s)"
              % (self.data, self.base, self.type, self.offset, self.size, self.stride))


class Execution:
    def __init__(self, stream=None):
        """stream: a hipStream_t as an integer (e.g. torch.cuda.Stream.cuda_stream); None = the default stream."""
        self._lib = C.lib()
        self._plan = None
        self.stream = stream

    def load(self, plan_file):
        h = ctypes.c_void_p()
        C.check(self._lib.llc_plan_load(os.fsencode(plan_file), ctypes.byref(h)))
        self._destroy()
        self._plan = h
        self._n_params = int(self._lib.llc_plan_num_params(h))

    def _destroy(self):
        if self._plan is not None:
            self._lib.llc_plan_destroy(self._plan)
            self._plan = None

    def __del__(self):
        try:
            self._destroy()
        except Exception:
            pass

    def _run(self, symbols, inputs, outputs):
        if self._plan is None:
            raise RuntimeError("Execution.run before Execution.load")
        tensors = list(inputs) + list(outputs)
        n_slots = 1 + 5 * len(tensors)
        if n_slots != self._n_params:
            raise ValueError("the plan takes %d tensors, %d were passed" % ((self._n_params - 1) // 5, len(tensors)))
        # Execution::run (Execution.cpp:21-45): slot 0, then five slots per tensor
        arr = (ctypes.c_void_p * n_slots)()
        keep = []
        if symbols:
            sym = C.i64_array(symbols)
            keep.append(sym)
            arr[0] = ctypes.addressof(sym)
        for k, t in enumerate(tensors):
            rank = len(t.size)
            off = ctypes.c_size_t(t.offset)
            size = (ctypes.c_size_t * max(rank, 1))(*t.size)
            stride = (ctypes.c_size_t * max(rank, 1))(*t.stride)
            keep += [off, size, stride]
            s = 1 + 5 * k
            arr[s], arr[s + 1] = t.base, t.data
            arr[s + 2], arr[s + 3], arr[s + 4] = ctypes.addressof(off), ctypes.addressof(size), ctypes.addressof(stride)
        C.check(self._lib.llc_hip_run(self._plan, arr, self.stream))

    def run(self, inputs, outputs):
        self._run(None, inputs, outputs)

    def run_with_symbols(self, symbols, inputs, outputs):
        self._run(list(symbols), inputs, outputs)
