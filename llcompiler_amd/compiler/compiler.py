"""torch.compile backend: the counterpart of llcompiler/compiler/compiler.py.

    model = torch.compile(model, backend=LLCompiler(mode="inference", target="gfx950", pipeline="hip"))

Flow (reference: compiler.py:84-168): dynamo + AOT-autograd hand over an ATen graph; supported
nodes are carved into fused submodules by CapabilityBasedPartitioner; each submodule is imported
into an LLH graph, run through the LLH pipeline, planned into kernel calls and replaced by a
Torch_ExecutionEngine.  Unsupported nodes stay in torch eager.  Nothing is shelled out to and no
shared library is generated per model: the "compiled artefact" is the kernel plan.
"""
from typing import Any, List

import os

import torch
import torch.fx
from torch._decomp import get_decompositions
from torch._dynamo.backends.common import aot_autograd
from torch.fx.passes.infra.partitioner import CapabilityBasedPartitioner

from ..executor.engine import Torch_ExecutionEngine
from ..importer.fx_importer import torch_translate_to_llh_graph
from ..llh.passes import run_llh_pipeline
from .torch_compile_config import LLC_DECOMPOSITIONS, LLCOperatorSupport

TARGETS = ("gfx950",)
# "transform" is the reference's name for its one pipeline (include/llcompiler/Support/Enums.td:28-34; what its driver
# passes, main.py:98): here it names the same thing, the LLH passes followed by this backend's kernel plan
PIPELINES = ("hip", "transform")


class LLCompiler:
    """
    example:
        compiler = LLCompiler()
        opt = torch.compile(model, backend=compiler)
        out = opt(*inputs)
    """

    def __init__(self, mode: str = "inference", target: str = "gfx950", pipeline: str = "hip", index_bit_width: int = 64,
                 symbol_infer=True, target_layout="NCHW", vebose_first_ir=False, log_root: str = "", log_level: str = "debug",
                 log_llvm: bool = True, cpu="", mtriple="", **kwargs) -> None:
        # the reference generates code for x86 / x86_64 (include/llcompiler/Support/Enums.td:28-34,
        # src/Compiler/Compiler.cpp:144-148); nothing here runs on the host, so those targets are an error
        if target not in TARGETS:
            raise ValueError("target %r: this backend generates code for %s only" % (target, ", ".join(TARGETS)))
        if pipeline not in PIPELINES:
            raise ValueError("pipeline %r: only %s is available" % (pipeline, ", ".join(PIPELINES)))
        # the layout convolutions are rewritten to by the layout transform (include/llcompiler/Dialect/LLH/IR/
        # LLHEnums.td:61-75, src/Dialect/LLH/Transforms/TransformLayout.cpp:141-198)
        if target_layout not in ("NCHW", "NHWC"):
            raise ValueError("target_layout %r: NCHW or NHWC" % (target_layout,))
        if mode not in ("inference", "training"):
            raise ValueError("mode %r" % (mode,))
        self.mode, self.target, self.pipeline = mode, target, pipeline
        self.vebose_first_ir = vebose_first_ir
        self.log_root, self.log_level = log_root, log_level
        self.target_layout = target_layout
        self.compile_count = 0
        self.engines = []

    def _log_dir(self):
        """With `log_root` set, every compiled graph leaves its IR in `<log_root>_<compile_count>`, as the reference's
        compiler does with its IR tree (llcompiler/compiler/compiler.py:101-105, src/Compiler/Compiler.cpp:50-58): here
        the imported LLH graph, the graph after the LLH passes and the kernel plan."""
        if not self.log_root:
            return ""
        d = "%s_%d" % (self.log_root, self.compile_count)
        os.makedirs(d, exist_ok=True)
        return d

    @staticmethod
    def _log(log_dir, name, graph):
        if not log_dir:
            return
        from ..llh.text import print_llh
        try:
            text = print_llh(graph)       # the reference's generic syntax, readable by the LLH text reader
        except Exception:                 # attributes the printer has no spelling for: the graph's own listing
            text = graph.dump()
        with open(os.path.join(log_dir, name + ".mlir"), "w") as f:
            f.write(text)

    def _process_fx(self, model: torch.fx.GraphModule, inputs: List[torch.Tensor], **kwargs):
        partition = CapabilityBasedPartitioner(model, LLCOperatorSupport(), allows_single_node_partition=True)
        return partition.partition_and_fuse()

    def not_compile(self, model: Any, inputs: List[torch.Tensor], **kwargs):
        return model

    def importer(self, model: torch.fx.GraphModule):
        return torch_translate_to_llh_graph(model)

    def compiler_fx(self, model: torch.fx.GraphModule, inputs: List[torch.Tensor], **kwargs):
        model = self._process_fx(model, inputs, **kwargs)
        for name, submodule in dict(model._modules).items():
            if not isinstance(submodule, torch.fx.GraphModule):
                continue
            executor = self.compiler_fx_submodule(submodule)
            model.delete_submodule(name)
            setattr(model, name, executor)
        return model.forward

    def compiler_fx_submodule(self, model: torch.fx.GraphModule, **kwargs):
        graph = self.importer(model)
        log_dir = self._log_dir()
        self._log(log_dir, "0_imported", graph)
        run_llh_pipeline(graph, self.target_layout)
        self._log(log_dir, "1_after_llh_passes", graph)
        if log_dir:
            from ..llh.plan_tool import plan_text
            with open(os.path.join(log_dir, "2_kernel_plan.txt"), "w") as f:
                f.write(plan_text(graph))
        if self.vebose_first_ir:
            print(graph.dump())
        self.compile_count += 1
        executor = _EngineModule(Torch_ExecutionEngine(graph))
        self.engines.append(executor.engine)
        return executor

    def __call__(self, model, inputs: List[torch.Tensor]) -> Any:
        if not isinstance(model, torch.fx.GraphModule):
            raise ValueError("Unsupported")
        bw_compiler = self.not_compile if self.mode == "inference" else self.compiler_fx
        return aot_autograd(fw_compiler=self.compiler_fx, bw_compiler=bw_compiler, inference_compiler=self.compiler_fx,
                            decompositions=get_decompositions(LLC_DECOMPOSITIONS))(model, inputs)


class _EngineModule(torch.nn.Module):
    """Lets an engine sit where the fused submodule was (GraphModule children must be Modules)."""

    def __init__(self, engine):
        super().__init__()
        self.engine = engine

    def forward(self, *args):
        return self.engine.run(*args)
