"""Ahead-of-time entry: compile a whole torch module into ONE engine with symbolic extents.

torch.compile guards re-specialise extents 0 and 1, so a batch-1 call would get a plan of its own.
`compile_module` exports the module once (torch.export with the given dynamic dims), runs the
same decompositions, importer and LLH pipeline as the torch.compile backend and returns a callable
whose single plan serves every value of the symbolic dims, batch 1 included.  Every node must be
translatable: there is no eager fallback on this entry.
"""
import os

import torch
from torch._decomp import get_decompositions

from ..executor.engine import Torch_ExecutionEngine
from ..importer.fx_importer import torch_translate_to_llh_graph
from ..llh.passes import run_llh_pipeline
from .torch_compile_config import LLC_DECOMPOSITIONS


class CompiledModule:
    def __init__(self, engine, lifted, n_user):
        self.engine, self.lifted, self.n_user = engine, lifted, n_user
        self._run = engine.bind_leading(lifted) if all(isinstance(t, torch.Tensor) for t in lifted) else None

    def __call__(self, *args):
        if len(args) != self.n_user:
            raise ValueError("expected %d inputs, got %d" % (self.n_user, len(args)))
        out = self._run(*args) if self._run is not None else self.engine.run(*self.lifted, *args)
        # export always returns a tuple; a single result is handed back bare, like the module would
        if isinstance(out, (list, tuple)) and len(out) == 1:
            return out[0]
        return out

    def save_plan(self, path, *args):
        """Writes the recorded kernel plan for the extents of `args` (the module's own inputs) to `path`, with its
        description beside it: see Torch_ExecutionEngine.save_plan.  Parameters that were lifted to graph inputs
        stay parameters of the plan's block (in front of `args`); with weights="npy" they are part of the file."""
        if len(args) != self.n_user:
            raise ValueError("expected %d inputs, got %d" % (self.n_user, len(args)))
        return self.engine.save_plan(path, *self.lifted, *args)


def compile_module(model, example_args, dynamic_shapes=None, verbose=False, weights=None, weight_dir=None,
                   target_layout="NCHW"):
    """target_layout: the layout convolutions are rewritten to (LLCompiler's keyword of the same name).
    weights="npy": parameters and buffers are written to .npy files (in weight_dir, or a fresh temporary
    directory) and enter the graph as llh.weight ops, the reference importer's convention
    (llcompiler/importer/fx_translate.py:415-435); the engine uploads each file once.  By default they stay
    torch tensors and are passed to the engine with every call."""
    model = model.eval()
    with torch.no_grad():
        ep = torch.export.export(model, tuple(example_args), dynamic_shapes=dynamic_shapes)
        # export keeps composite ops (layer_norm, linear, softmax.int ...) that AOT-autograd would already
        # have taken apart: start from the core-ATen table, then apply the backend's own set on top
        table = torch.export.default_decompositions()
        for k, v in get_decompositions(LLC_DECOMPOSITIONS).items():
            table[k] = v
        ep = ep.run_decompositions(table)
    gm = ep.graph_module
    sig = ep.graph_signature
    state = dict(ep.state_dict)
    state.update(getattr(ep, "constants", {}) or {})
    lifted = []
    n_user = 0
    for spec in sig.input_specs:
        kind = spec.kind.name
        if kind == "USER_INPUT":
            n_user += 1
        else:
            t = state[spec.target]
            lifted.append(t.detach() if isinstance(t, torch.Tensor) else t)
    if any(s.kind.name != "USER_INPUT" for s in sig.input_specs[len(lifted):]):
        raise NotImplementedError("lifted inputs must precede user inputs")
    weight_files = None
    if weights == "npy":
        from ..executor.weights import new_weight_dir, save_weight
        wdir = new_weight_dir(weight_dir)
        names = [n.name for n in gm.graph.nodes if n.op == "placeholder"][:len(lifted)]
        weight_files = {}
        for name, t in zip(names, lifted):
            if not isinstance(t, torch.Tensor):
                raise TypeError("weights=\"npy\": %s is not a tensor" % name)
            weight_files[name] = save_weight(t, os.path.join(wdir, name + ".npy"))
        lifted = []
    elif weights is not None:
        raise ValueError("weights must be None or \"npy\"")
    graph = torch_translate_to_llh_graph(gm, weight_files)
    run_llh_pipeline(graph, target_layout)
    if verbose:
        print(graph.dump())
    return CompiledModule(Torch_ExecutionEngine(graph), lifted, n_user)
