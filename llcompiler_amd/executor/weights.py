"""Weights of llh.weight ops: .npy files uploaded once into device memory owned by a native plan.

The reference's importer writes every parameter with np.save and emits `llh.weight{weight_file}`
(llcompiler/importer/fx_translate.py:415-435); its LoadWeight pass turns the files into constants of the compiled
object (src/Dialect/LLH/Transforms/LoadWeight.cpp:58-171).  Here the files are read by the kernel library
(llc_plan_load_npy) when an engine first needs them and stay on the device for the engine's lifetime.
"""
import os
import tempfile

import numpy as np
import torch

from .. import _capi as C
from .plan_runner import Plan

_TYPESTR = {C.FLOAT32: "<f4", C.INT64: "<i8", C.DOUBLE64: "<f8", C.FLOAT16: "<f2", C.INT32: "<i4", C.INT16: "<i2",
            C.INT8: "|i1", C.INT1: "|b1", C.BFLOAT16: "<i2"}


class _DeviceArray:
    """Exposes plan-owned device memory through the CUDA array interface, so that torch can alias it."""

    def __init__(self, ptr, code, shape, owner):
        self.__cuda_array_interface__ = {"shape": tuple(shape), "typestr": _TYPESTR[code], "data": (ptr, False),
                                         "version": 2, "strides": None}
        self._owner = owner


def save_weight(tensor, path):
    """np.save of a parameter, as the reference's importer does; bf16 goes out as its bit patterns ('<u2')."""
    t = tensor.detach().cpu().contiguous()
    if t.dtype == torch.bfloat16:
        arr = t.view(torch.int16).numpy().view(np.uint16)
    else:
        arr = t.numpy()
    np.save(path, arr)
    return path if path.endswith(".npy") else path + ".npy"


def new_weight_dir(base=None):
    """A fresh directory for one compilation's weight files (the reference uses LLcompiler_weight_temp/<time stamp>)."""
    if base is not None:
        os.makedirs(base, exist_ok=True)
        return base
    return tempfile.mkdtemp(prefix="LLcompiler_weight_temp_")


class WeightStore:
    def __init__(self, device):
        self.device = device
        self._plan = None
        self._cache = {}

    def get(self, path, shape, dtype):
        key = (path, tuple(shape), dtype)
        t = self._cache.get(key)
        if t is None:
            C.init(self.device.index or 0)
            if self._plan is None:
                with torch.cuda.device(self.device):
                    self._plan = Plan()
            code = C.TORCH_DTYPE_TO_TYPE[dtype]
            with torch.cuda.device(self.device):
                ptr, got, got_shape = self._plan.load_npy(path, code)
            if tuple(got_shape) != tuple(shape):
                raise ValueError("%s holds shape %s, the graph expects %s" % (path, tuple(got_shape), tuple(shape)))
            n = 1
            for d in shape:
                n *= d
            if n == 0:
                t = torch.empty(tuple(shape), dtype=dtype, device=self.device)
            else:
                raw = torch.as_tensor(_DeviceArray(ptr, got, shape, self._plan), device=self.device)
                t = raw.view(torch.bfloat16) if dtype == torch.bfloat16 else raw
                if t.dtype != dtype:
                    raise TypeError("%s: %s read as %s" % (path, dtype, t.dtype))
            self._cache[key] = t
        return t
