"""llcompiler_amd: an MI355X (gfx950) execution backend for LLCompiler's compiled-op path.

    from llcompiler_amd import LLCompiler
    model = torch.compile(model, backend=LLCompiler())

Kernels live in csrc/ behind the C-ABI of include/llc_hip.h (libllc_hip.so); `ops` holds one thin
call per entry point; `importer`, `llh`, `executor` and `compiler` mirror the reference's
importer, dialect passes, executor and torch.compile backend for this path.
"""
from . import _capi  # noqa: F401


def __getattr__(name):
    if name == "LLCompiler":
        from .compiler.compiler import LLCompiler
        return LLCompiler
    if name == "Torch_ExecutionEngine":
        from .executor.engine import Torch_ExecutionEngine
        return Torch_ExecutionEngine
    raise AttributeError(name)
