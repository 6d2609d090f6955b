"""CPU-side checks of the boundary: the library loads, exports every symbol the header declares,
and the argument validation that needs no GPU reports errors instead of crashing."""
import ctypes
import os
import re

import pytest

from llcompiler_amd import _capi as C

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "llc_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(llc_(?:hip|plan|npy)_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_agree():
    assert declared_symbols() == sorted(C.EXPORTS)


def test_library_exports_every_declared_symbol():
    assert os.path.exists(C.LIB_PATH), "build the library first: python -m llcompiler_amd.build"
    L = ctypes.CDLL(C.LIB_PATH)
    for name in declared_symbols():
        assert hasattr(L, name), name
    assert L.llc_hip_abi_version() == 3


def test_status_strings_and_null_argument_errors():
    L = C.lib()
    assert L.llc_hip_status_string(0) == b"ok"
    assert b"shape" in L.llc_hip_status_string(-3)
    st = L.llc_hip_softmax(None, None, None)
    assert st == -1
    assert b"null" in L.llc_hip_last_error()
    with pytest.raises(C.LlcHipError):
        C.check(st)


def test_descriptor_layout_matches_reference_tensor_field_order():
    # include/llcompiler/Compiler/Tensor.h:42-47: data, base, type, offset, size, stride
    names = [f[0] for f in C.LlcTensor._fields_]
    assert names == ["data", "base", "type", "offset", "rank", "size", "stride"]
    # type codes 0-6 are the reference's enum (Tensor.h:25-33; engine.py:11 maps f32->4, i64->3, bool->6)
    import torch
    assert C.TORCH_DTYPE_TO_TYPE[torch.float32] == 4
    assert C.TORCH_DTYPE_TO_TYPE[torch.int64] == 3
    assert C.TORCH_DTYPE_TO_TYPE[torch.bool] == 6


def test_unpack_params_follows_execution_run_layout():
    # src/Compiler/Execution.cpp:21-41: [symbols|NULL] then per tensor base, data, &offset, size*, stride*
    L = C.lib()
    sizes = (ctypes.c_size_t * 2)(3, 5)
    strides = (ctypes.c_size_t * 2)(5, 1)
    off = ctypes.c_size_t(7)
    syms = (ctypes.c_int64 * 1)(42)
    params = (ctypes.c_void_p * 6)(ctypes.addressof(syms), 0x1000, 0x1040, ctypes.addressof(off),
                                   ctypes.addressof(sizes), ctypes.addressof(strides))
    ranks = (ctypes.c_size_t * 1)(2)
    types = (ctypes.c_size_t * 1)(C.FLOAT32)
    out = (C.LlcTensor * 1)()
    sym_out = ctypes.POINTER(ctypes.c_int64)()
    used = L.llc_hip_unpack_params(params, 1, ranks, types, out, ctypes.byref(sym_out))
    assert used == 6
    t = out[0]
    assert (t.base, t.data, t.offset, t.rank, t.type) == (0x1000, 0x1040, 7, 2, C.FLOAT32)
    assert [t.size[i] for i in range(2)] == [3, 5] and [t.stride[i] for i in range(2)] == [5, 1]
    assert sym_out[0] == 42
    # no symbols: slot 0 is NULL (Execution.cpp:24) and still consumed
    params[0] = None
    used = L.llc_hip_unpack_params(params, 1, ranks, types, out, ctypes.byref(sym_out))
    assert used == 6 and not sym_out


def test_plan_entry_points_validate_without_a_gpu():
    L = C.lib()
    assert L.llc_hip_run(None, None, None) == C.ERR_BAD_ARG
    assert L.llc_plan_begin(None) == C.ERR_BAD_ARG
    assert L.llc_plan_end(None) == C.ERR_BAD_ARG
    assert L.llc_plan_destroy(None) == 0
    assert L.llc_plan_num_steps(None) == -1
    # the void(void**) entry logs and keeps the status when no plan is bound (Execution.h:23 has no return value)
    assert L.llc_hip_bind_entry(None, None) == 0
    L.llc_hip_entry(None)
    assert L.llc_hip_entry_status() == C.ERR_BAD_ARG
    assert b"no plan is bound" in L.llc_hip_last_error()


def test_entry_library_exports_main_for_the_reference_loader():
    # src/Compiler/Execution.cpp:12-16 resolves "main" in the library it is given
    assert os.path.exists(C.ENTRY_LIB_PATH), "build the library first: python -m llcompiler_amd.build"
    E = ctypes.CDLL(C.ENTRY_LIB_PATH)
    assert hasattr(E, "main")


def test_cpu_tensor_is_refused_not_computed():
    import torch
    from llcompiler_amd import ops
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        ops.softmax(torch.zeros(2, 3))


def _npy_info(path, expect=-1):
    import ctypes as ct
    L = C.lib()
    dtype, rank, off = ct.c_size_t(), ct.c_size_t(), ct.c_size_t()
    size = (ct.c_size_t * C.LLC_MAX_RANK)()
    st = L.llc_npy_info(os.fsencode(path), expect, ct.byref(dtype), ct.byref(rank), size, ct.byref(off))
    return st, dtype.value, tuple(size[i] for i in range(rank.value)), off.value


def test_npy_header_parser_reads_what_np_save_writes(tmp_path):
    """The weight wire format: np.save output (llcompiler/importer/fx_translate.py:427-430), parsed like
    src/Dialect/LLH/Transforms/LoadWeight.cpp:58-132: type, shape, and the data right behind the header."""
    import numpy as np
    cases = [(np.arange(24, dtype=np.float32).reshape(2, 3, 4), C.FLOAT32), (np.arange(5, dtype=np.int64), C.INT64),
             (np.float32(3.5).reshape(()), C.FLOAT32), (np.ones((4, 0, 2), np.float16), C.FLOAT16),
             (np.array([[True, False]]), C.INT1), (np.arange(6, dtype=np.int32).reshape(3, 2), C.INT32)]
    for k, (arr, code) in enumerate(cases):
        path = str(tmp_path / ("w%d.npy" % k))
        np.save(path, arr)
        st, dtype, shape, off = _npy_info(path)
        assert (st, dtype, shape) == (0, code, arr.shape), (path, st, C.lib().llc_hip_last_error())
        raw = open(path, "rb").read()
        assert raw[off:] == arr.tobytes()          # the data starts where the parser says, in C order
        assert _npy_info(path, code)[0] == 0 and _npy_info(path, C.INT16)[0] == C.ERR_DTYPE
    # bf16 travels as its bit patterns: '<u2' is accepted only when the caller expects bf16
    bits = str(tmp_path / "bits.npy")
    np.save(bits, np.arange(8, dtype=np.uint16))
    assert _npy_info(bits)[0] == C.ERR_DTYPE and _npy_info(bits, C.BFLOAT16)[:3] == (0, C.BFLOAT16, (8,))
    # format version 2 (four-byte header length)
    v2 = str(tmp_path / "v2.npy")
    with open(v2, "wb") as f:
        np.lib.format.write_array(f, np.arange(6, dtype=np.float32).reshape(2, 3), version=(2, 0))
    assert _npy_info(v2)[:3] == (0, C.FLOAT32, (2, 3))
    # Fortran order (the reference reads such a file as if it were C ordered), big-endian data, not a .npy file
    fo = str(tmp_path / "f.npy")
    np.save(fo, np.asfortranarray(np.arange(6, dtype=np.float32).reshape(2, 3)))
    assert _npy_info(fo)[0] == C.ERR_LAYOUT
    be = str(tmp_path / "be.npy")
    np.save(be, np.arange(4, dtype=">f4"))
    assert _npy_info(be)[0] == C.ERR_DTYPE
    junk = str(tmp_path / "junk.npy")
    open(junk, "wb").write(b"not a numpy file at all")
    assert _npy_info(junk)[0] == C.ERR_BAD_ARG and _npy_info(str(tmp_path / "missing.npy"))[0] == C.ERR_BAD_ARG


def test_plan_files_are_checked_before_anything_touches_a_device(tmp_path):
    """llc_plan_load refuses what is not a plan file (missing, wrong magic, another ABI version) and
    llc_plan_save refuses null arguments: all of it host logic."""
    import ctypes
    import struct
    from llcompiler_amd import _capi as C
    L = C.lib()
    h = ctypes.c_void_p()
    assert L.llc_plan_load(str(tmp_path / "missing.llcplan").encode(), ctypes.byref(h)) == C.ERR_BAD_ARG
    assert b"cannot open" in L.llc_hip_last_error()
    junk = tmp_path / "junk.llcplan"
    junk.write_bytes(b"not a plan at all, just bytes")
    assert L.llc_plan_load(str(junk).encode(), ctypes.byref(h)) == C.ERR_BAD_ARG and not h.value
    assert b"not a plan file" in L.llc_hip_last_error()
    other = tmp_path / "other_abi.llcplan"
    other.write_bytes(b"LLCPLAN1" + struct.pack("<Q", 10 ** 6))
    assert L.llc_plan_load(str(other).encode(), ctypes.byref(h)) == C.ERR_UNSUPPORTED and not h.value
    assert L.llc_plan_save(None, b"x") == C.ERR_BAD_ARG
    assert L.llc_plan_load(None, ctypes.byref(h)) == C.ERR_BAD_ARG
