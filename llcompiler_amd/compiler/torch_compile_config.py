"""Decomposition set and operator support used when an FX graph is partitioned for compilation.

Counterpart of llcompiler/compiler/torch_compile_config.py.  LLC_DECOMPOSITIONS is the reference's
set (:12-28) without aten._softmax and aten.addmm: softmax has a kernel of its own here, so the op is
kept whole (a graph that arrives already decomposed is re-fused by llh.passes.fuse_softmax); addmm is
translated directly to matmul + add, and aten.add / sub / mul / div are translated as they are,
because their decompositions wrap every 16-bit op in converts to and from fp32 (the kernels compute in
fp32 and round once anyway), which also hides bias, residual and scale from the epilogue fusion.  Operator support
is "the importer has a translator and the node's attributes are ones the kernels implement";
everything else stays in torch eager, the reference's fallback rule (:94-98).
"""
import typing as t

import torch
from torch.fx.passes.operator_support import OperatorSupport

from ..importer.fx_importer import TORCH_FUNCTION_TRANSLATE, is_supported

aten = torch.ops.aten
prims = torch.ops.prims

LLC_DECOMPOSITIONS = {
    aten.expand,
    aten._unsafe_view,
    aten.transpose,
    aten.threshold_backward,
    aten.native_batch_norm_backward,
    aten.masked_fill,
    aten.where,
    aten.squeeze.dim,
    aten.squeeze.dims,
    aten.linear,
    aten.matmul,
    aten.t,
    # the GPU dispatch of eval-mode batch norm; both decompose to aten.native_batch_norm
    aten.miopen_batch_norm,
    aten.cudnn_batch_norm,
}
LLC_DECOMPOSITIONS.discard(aten.t)  # aten.t is translated directly (llh.transpose perms [1,0])

# name -> None ("any dtype"), the shape of the reference's LLC_SUPPORT_DICT
LLC_SUPPORT_DICT = {str(k): None for k in TORCH_FUNCTION_TRANSLATE}

SUPPORTED_DTYPES = (torch.float32, torch.bfloat16, torch.float16, torch.int64, torch.int32, torch.bool)


class LLCOperatorSupport(OperatorSupport):
    def __init__(self, support_dict: t.Optional[dict] = None):
        super().__init__()
        self._support_dict = support_dict or LLC_SUPPORT_DICT

    def is_node_supported(self, submodules, node: torch.fx.Node) -> bool:
        if node.op in ("placeholder", "output", "get_attr"):
            return False
        if node.op != "call_function":
            return False
        if not is_supported(node):
            return False
        val = node.meta.get("val")
        vals = val if isinstance(val, (tuple, list)) else [val]
        for v in vals:
            if isinstance(v, torch.Tensor) and v.dtype not in SUPPORTED_DTYPES:
                return False
        for a in node.all_input_nodes:
            v = a.meta.get("val")
            if isinstance(v, torch.Tensor) and v.dtype not in SUPPORTED_DTYPES:
                return False
        return True
