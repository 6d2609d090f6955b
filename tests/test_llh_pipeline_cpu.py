"""Pass-level tests on the LLH graph, mirroring the reference's lit/FileCheck cases (op names,
attributes and shapes after each rewrite; no numbers).  They run without a GPU: importing, the LLH
pipeline and kernel planning are host-side."""
import pytest
import torch

from llcompiler_amd.executor.planner import make_plan
from llcompiler_amd.llh.expr import Expr, ceildiv, evaluate
from llcompiler_amd.llh.graph import Graph
from llcompiler_amd.llh.passes import canonicalize, decompose_batch_norm, fuse_softmax, run_llh_pipeline, transform_layout

f32 = torch.float32
s0, s2 = Expr.sym("s0"), Expr.sym("s2")


# ---- shape inference known answers (test/Dialect/LLH/symbol_infer/infer_symbol_shape.mlir) ----
def test_infer_conv_static_and_dynamic():
    g = Graph()
    x = g.add_input((2, 3, 224, 224), f32)
    w = g.add_input((64, 3, 7, 7), f32)
    # :181-186
    y = g.add_op("conv", [x, w], {"dilation": (2, 3), "kernel_shape": (7, 7), "pad": (3, 2, 3, 2), "stride": (2, 1), "group": 1})
    assert y.shape == (2, 64, 109, 210)
    # :160-175: ?x3x?x? with k7 p3 s2 -> (s0, 64, f(s2), f(s2)); floor division is the run-time semantics
    g2 = Graph()
    xd = g2.add_input((s0, 3, s2, s2), f32)
    wd = g2.add_input((64, 3, 7, 7), f32)
    yd = g2.add_op("conv", [xd, wd], {"dilation": (1, 1), "kernel_shape": (7, 7), "pad": (3, 3, 3, 3), "stride": (2, 2), "group": 1})
    assert yd.shape[0] == s0 and yd.shape[1] == 64
    for n in (7, 8, 224, 225):
        assert evaluate(yd.shape[2], {"s0": 4, "s2": n}) == (n - 1) // 2 + 1
    assert g2.symbol_sources == {"s0": (0, 0), "s2": (0, 2)}


def test_infer_maxpool_matmul_bmm_reduce():
    g = Graph()
    x = g.add_input((2, 64, 9, 17), f32)
    # :73-78
    y = g.add_op("max_pool", [x], {"ceil_mode": False, "dilation": (2, 1), "kernel_shape": (7, 7), "pad": (3, 1, 3, 1), "stride": (2, 2)})
    assert y.shape == (2, 64, 2, 7)
    a = g.add_input((s0, 512), f32)
    b = g.add_input((512, 10), f32)
    assert g.add_op("matmul", [a, b]).shape == (s0, 10)  # :133-135
    p = g.add_input((12, s0, 512), f32)
    q = g.add_input((12, 512, 10), f32)
    assert g.add_op("batch_matmul", [p, q]).shape == (12, s0, 10)  # :212-214
    r = g.add_input((3, 3, s0, s2), f32)
    assert g.add_op("reduce_sum", [r], {"axis": (1, 2)}).shape == (3, s2)  # :266-268


def test_stride_slice_size_is_ceildiv():
    g = Graph()
    x = g.add_input((10, s0), f32)
    y = g.add_op("stride_slice", [x], {"start": (1, 0), "end": (10, s0), "stride": (4, 2)})
    assert y.shape[0] == 3 and evaluate(y.shape[1], {"s0": 7}) == 4
    assert ceildiv(9, 4) == 3


# ---- decompose_ops.mlir:10-20 ----
def test_batch_norm_decomposition_op_order():
    g = Graph()
    x = g.add_input((s0, 3, s2, s2), f32)
    w = [g.add_input((3,), f32) for _ in range(4)]
    y = g.add_op("batch_norm_inference", [x] + w, {"epsilon": 1e-5, "momentum": 0.1, "feature_index": 1})
    g.set_outputs([y])
    decompose_batch_norm(g)
    names = [n for n in g.op_names() if n != "constant"]
    assert names == ["add", "sqrt"] + ["reshape", "broadcast_to"] * 4 + ["sub", "mul", "div", "add"]
    assert "batch_norm_inference" not in g.op_names()
    # the whole chain becomes ONE elementwise kernel reading x and four per-channel vectors
    steps = [s for s in make_plan(g) if s.kind not in ("view", "constant")]
    assert [s.kind for s in steps] == ["ew", "ew"]
    assert [i[0] for i in steps[1].attrs["insts"]] == ["sub", "mul", "div", "add"]


# ---- canonicalisation ----
def test_canonicalize_folds_noops():
    g = Graph()
    x = g.add_input((4, 8), f32)
    one = g.constant(1.0)
    y = g.add_op("mul", [x, one])
    y = g.add_op("reshape", [y], {"shape": (4, 8)})
    y = g.add_op("identity", [y])
    y = g.add_op("broadcast_to", [y], {"shape": (4, 8), "cast_dims": (0, 1)})
    y = g.add_op("convert_to", [y], {"dtype": f32})
    y = g.add_op("relu", [y])
    g.set_outputs([y])
    canonicalize(g)
    assert g.op_names() == ["relu"]


def test_softmax_pattern_is_refused_into_one_op():
    # amax -> sub -> exp -> sum -> div, the decomposition of aten._softmax (torch_compile_config.py:24)
    g = Graph()
    x = g.add_input((s0, 12, 64, 64), f32)
    m = g.add_op("reduce_max", [x], {"axis": (3,)})
    m = g.add_op("reshape", [m], {"shape": (s0, 12, 64, 1)})
    m = g.add_op("broadcast_to", [m], {"shape": x.shape, "cast_dims": (0, 1, 2, 3)})
    e = g.add_op("exp", [g.add_op("sub", [x, m])])
    s = g.add_op("reduce_sum", [e], {"axis": (3,)})
    s = g.add_op("reshape", [s], {"shape": (s0, 12, 64, 1)})
    s = g.add_op("broadcast_to", [s], {"shape": x.shape, "cast_dims": (0, 1, 2, 3)})
    y = g.add_op("div", [e, s])
    g.set_outputs([y])
    fuse_softmax(g)
    assert g.op_names() == ["softmax"]
    assert [st.kind for st in make_plan(g)] == ["softmax"]


# ---- planning: epilogue and elementwise fusion ----
def _linear(g, x, n_out, act=None):
    w = g.add_input((n_out, x.shape[1]), f32)
    b = g.add_input((n_out,), f32)
    wt = g.add_op("transpose", [w], {"perms": (1, 0)})
    y = g.add_op("matmul", [x, wt])
    bb = g.add_op("reshape", [b], {"shape": (1, n_out)})
    bb = g.add_op("broadcast_to", [bb], {"shape": y.shape, "cast_dims": (0, 1)})
    y = g.add_op("add", [y, bb])
    return g.add_op(act, [y]) if act else y


def test_mlp_plans_to_two_kernels():
    g = Graph()
    x = g.add_input((4, 784), f32)
    y = _linear(g, _linear(g, x, 512, "relu"), 10)
    g.set_outputs([y])
    run_llh_pipeline(g)
    steps = [s for s in make_plan(g) if s.kind != "view"]
    assert [s.kind for s in steps] == ["matmul", "matmul"]
    assert steps[0].attrs["epilogue"]["act"] == "relu" and steps[0].attrs["epilogue"]["bias"] is not None
    assert steps[1].attrs["epilogue"]["act"] is None and steps[1].attrs["epilogue"]["bias"] is not None


def test_residual_block_tail_fuses_into_second_conv_only_once():
    g = Graph()
    x = g.add_input((2, 64, 14, 14), f32)
    attrs = {"dilation": (1, 1), "kernel_shape": (3, 3), "pad": (1, 1, 1, 1), "stride": (1, 1), "group": 1}
    w1, b1, w2, b2 = g.add_input((64, 64, 3, 3), f32), g.add_input((64,), f32), g.add_input((64, 64, 3, 3), f32), g.add_input((64,), f32)
    wd, bd = g.add_input((64, 64, 1, 1), f32), g.add_input((64,), f32)
    c1 = g.add_op("relu", [g.add_op("conv_bias", [x, w1, b1], attrs)])
    c2 = g.add_op("conv_bias", [c1, w2, b2], attrs)
    dn = g.add_op("conv_bias", [x, wd, bd], dict(attrs, kernel_shape=(1, 1), pad=(0, 0, 0, 0)))
    y = g.add_op("relu", [g.add_op("add", [c2, dn])])
    g.set_outputs([y])
    steps = [s for s in make_plan(g) if s.kind != "view"]
    assert [s.kind for s in steps] == ["conv", "conv", "conv"]
    by_out = {s.output.name: s for s in steps}
    tail = by_out[y.name]
    assert tail.attrs["epilogue"]["residual"] is dn and tail.attrs["epilogue"]["act"] == "relu"
    assert by_out[dn.name].attrs["epilogue"]["act"] is None and by_out[dn.name].attrs["epilogue"]["residual"] is None


def test_elementwise_chain_is_one_program():
    # ElewiseFusion1: x+x; -3; /2; relu; *x
    g = Graph()
    x = g.add_input((200, 3, 224, 224), f32)
    y = g.add_op("add", [x, x])
    y = g.add_op("sub", [y, g.constant(3.0)])
    y = g.add_op("div", [y, g.constant(2.0)])
    y = g.add_op("relu", [y])
    y = g.add_op("mul", [y, x])
    g.set_outputs([y])
    steps = [s for s in make_plan(g) if s.kind not in ("view", "constant")]
    assert len(steps) == 1 and steps[0].kind == "ew"
    assert [i[0] for i in steps[0].attrs["insts"]] == ["add", "sub", "div", "relu", "mul"]
    assert len(steps[0].inputs) == 1  # x is read once


def test_multi_use_value_is_not_fused_away():
    g = Graph()
    x = g.add_input((8, 8), f32)
    a = g.add_op("exp", [x])
    b = g.add_op("add", [a, a])
    c = g.add_op("mul", [a, b])
    g.set_outputs([b, c])
    steps = make_plan(g)
    assert [s.kind for s in steps] == ["ew", "ew", "ew"]  # a has two users, b is an output


# ---- importer on real FX graphs (no GPU needed up to planning) ----
def test_import_mlp_from_fx_and_plan():
    from llcompiler_amd import LLCompiler
    from llcompiler_amd.test_models import MLP, make_mlp_inputs
    comp = LLCompiler()
    graphs = []
    orig = comp.importer

    def spy(gm):
        g = orig(gm)
        graphs.append(g)
        return g

    comp.importer = spy
    opt = torch.compile(MLP().eval(), backend=comp, fullgraph=True)
    with torch.no_grad(), pytest.raises(RuntimeError, match="no CPU fallback"):
        opt(*make_mlp_inputs())  # compiles fine, then refuses to execute on CPU tensors
    assert len(graphs) == 1
    names = graphs[0].op_names()
    assert names.count("matmul") == 2 and "relu" in names and "transpose" in names
    # addmm is translated whole: matmul + add (the add folds into the matmul's epilogue when planned)
    assert names.count("add") == 2


def test_log_root_leaves_the_ir_of_every_compiled_graph(tmp_path):
    """log_root, as in the reference (compiler.py:101-105): one directory per compiled graph, named
    <log_root>_<compile_count>, here with the imported LLH, the LLH after the passes (both in the generic syntax the
    text reader takes back) and the kernel plan."""
    from llcompiler_amd import LLCompiler
    from llcompiler_amd.llh.text import parse_llh
    from llcompiler_amd.test_models import MLP, make_mlp_inputs
    torch._dynamo.reset()
    comp = LLCompiler(log_root=str(tmp_path / "ir"))
    opt = torch.compile(MLP().eval(), backend=comp, fullgraph=True)
    with torch.no_grad(), pytest.raises(RuntimeError, match="no CPU fallback"):
        opt(*make_mlp_inputs())
    d = tmp_path / "ir_0"
    assert sorted(p.name for p in d.iterdir()) == ["0_imported.mlir", "1_after_llh_passes.mlir", "2_kernel_plan.txt"]
    before = parse_llh((d / "0_imported.mlir").read_text())
    after = parse_llh((d / "1_after_llh_passes.mlir").read_text())
    assert before.op_names().count("matmul") == 2 and after.op_names().count("matmul") == 2
    plan = (d / "2_kernel_plan.txt").read_text()
    assert plan.count("matmul") == 2 and "relu" in plan
    torch._dynamo.reset()


def test_compiler_rejects_other_targets_and_pipelines():
    from llcompiler_amd import LLCompiler
    with pytest.raises(ValueError):
        LLCompiler(target="x86_64")
    with pytest.raises(ValueError):
        LLCompiler(pipeline="basic")
    LLCompiler(mode="inference", target="gfx950", pipeline="hip", symbol_infer=True, target_layout="NCHW", log_level="debug")
    # the keyword arguments of the reference's driver script (main.py:82-99), whose pipeline is called "transform"
    LLCompiler(mode="inference", ir_tree_dir="ir_tree", log_root="", log_level="debug", symbol_infer=True, target_layout="NCHW",
               pipeline="transform")


def test_engine_argument_convention_and_errors():
    from llcompiler_amd.executor.engine import Torch_ExecutionEngine
    g = Graph()
    x = g.add_input((s0, 8), f32)
    g.set_outputs([g.add_op("relu", [x])])
    eng = Torch_ExecutionEngine(g)
    with pytest.raises(TypeError, match="Unsupported type"):
        eng.run("not a tensor")
    with pytest.raises(ValueError, match="expected 1 tensors"):
        eng.run(torch.zeros(2, 8), torch.zeros(2, 8))
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        eng.run(torch.zeros(2, 8))
    with pytest.raises(ValueError, match="expected"):
        eng.run(torch.zeros(2, 9).to("meta") if False else torch.zeros(2, 9))


def test_parameters_become_weight_ops_naming_npy_files(tmp_path):
    """weights="npy": the reference importer's convention (llcompiler/importer/fx_translate.py:415-435): every
    parameter is written with np.save and enters the graph as llh.weight{weight_file}; only the user's tensors
    remain run-time inputs."""
    import numpy as np
    from llcompiler_amd.compiler.aot import compile_module
    from llcompiler_amd.test_models import MLP, make_mlp_inputs
    m = MLP().eval()
    cm = compile_module(m, make_mlp_inputs(), weights="npy", weight_dir=str(tmp_path))
    g = cm.engine.graph
    ws = [op for op in g.ops if op.name == "weight"]
    assert len(ws) == 4 and len(g.inputs) == 1 and cm.lifted == []
    want = {tuple(p.shape): p.detach().numpy() for p in m.parameters()}
    for op in ws:
        arr = np.load(op.attrs["weight_file"])
        assert arr.dtype == np.float32 and tuple(op.results[0].shape) == arr.shape
        np.testing.assert_array_equal(arr, want[arr.shape])
    kinds = [s.kind for s in cm.engine.steps if s.kind != "view"]
    assert kinds.count("weight") == 4 and kinds.count("matmul") == 2


def test_prims_level_nodes_are_translated():
    """Graphs that arrive at prims level (what inductor's decompositions leave): prims.collapse_view, prims.sum,
    prims.clone and prims.inductor_force_stride_order have translators like in the reference
    (fx_op_translate/reshape_ops.py:89-140, reduce_ops.py:85-118, identity.py:51-59)."""
    from torch.fx.experimental.proxy_tensor import make_fx
    from llcompiler_amd.importer.fx_importer import torch_translate_to_llh_graph
    import torch._inductor.inductor_prims  # noqa: F401  (defines prims.inductor_force_stride_order)
    from llcompiler_amd.importer.fx_importer import register_inductor_prims
    register_inductor_prims()
    prims = torch.ops.prims

    def f(x):
        y = prims.collapse_view(x, 1, 2)
        z = prims.sum(y, [1])
        return prims.clone(prims.inductor_force_stride_order(z, (5, 1)))

    gm = make_fx(f, tracing_mode="fake")(torch.zeros(3, 4, 6, 5))
    g = torch_translate_to_llh_graph(gm)
    names = g.op_names()
    assert names.count("reshape") == 1 and names.count("reduce_sum") == 1, names
    shapes = {op.name: tuple(op.results[0].shape) for op in g.ops}
    assert shapes["reshape"] == (3, 24, 5) and shapes["reduce_sum"] == (3, 5)
    from llcompiler_amd.llh.passes import run_llh_pipeline
    run_llh_pipeline(g)
    assert g.op_names() == ["reshape", "reduce_sum"]          # the identities are gone


def test_true_division_of_integers_is_imported_as_a_floating_point_div():
    """aten.div.Tensor / div.Scalar of integer tensors give floats in torch; the importer converts the operands to
    the result type before llh.div (an integer llh.div would floor), and prims.div of two integers (truncating in
    torch) is left to eager."""
    from torch.fx.experimental.proxy_tensor import make_fx
    from llcompiler_amd.importer.fx_importer import is_supported, torch_translate_to_llh_graph
    gm = make_fx(lambda a, b: (a / 2, a / b, 3 / a))(torch.tensor([7, -7]), torch.tensor([2, 3]))
    g = torch_translate_to_llh_graph(gm)
    divs = [op for op in g.ops if op.name in ("div", "recip")]  # 3 / a arrives as reciprocal(a) * 3
    assert len(divs) == 3
    for op in divs:
        assert op.results[0].dtype == torch.float32
        assert all(v.dtype == torch.float32 for v in op.operands)
    gm = make_fx(lambda a, b: torch.ops.prims.div(a, b))(torch.tensor([7, -7]), torch.tensor([2, 3]))
    node = [n for n in gm.graph.nodes if n.op == "call_function"][0]
    assert node.meta["val"].dtype == torch.int64 and not is_supported(node)


# ---- layout transform (test/Dialect/LLH/transform_layout.mlir) ----
CONV_ATTRS = {"dilation": (2, 2), "kernel_shape": (7, 7), "pad": (3, 3, 3, 3), "stride": (2, 2), "group": 1, "layout": "NCHW"}


def test_infer_conv_in_the_nhwc_layout():
    g = Graph()
    x = g.add_input((2, 224, 200, 3), f32)
    w = g.add_input((64, 7, 7, 3), f32)
    y = g.add_op("conv", [x, w], dict(CONV_ATTRS, dilation=(1, 1), layout="NHWC"))
    assert y.shape == (2, 112, 100, 64)


def test_transform_layout_wraps_a_conv_in_the_reference_transposes():
    """transform_layout.mlir conv_nchw_to_nhwc: transposes 0,2,3,1 on both operands, the conv, 0,3,1,2 on the result;
    dynamic extents move with their dims."""
    g = Graph()
    w = g.add_input((4, 3, 7, 7), f32)
    x = g.add_input((s0, 3, s2, s2), f32)
    y = g.add_op("conv", [x, w], dict(CONV_ATTRS))
    g.set_outputs([y])
    natural = y.shape
    transform_layout(g, "NHWC")
    assert g.op_names() == ["transpose", "transpose", "conv", "transpose"]
    tx, tw, conv, back = g.ops
    assert tuple(tx.attrs["perms"]) == (0, 2, 3, 1) and tuple(tw.attrs["perms"]) == (0, 2, 3, 1)
    assert tuple(back.attrs["perms"]) == (0, 3, 1, 2)
    assert conv.attrs["layout"] == "NHWC" and conv.attrs["weight_layout"] == "NHWC"
    assert tx.results[0].shape == (s0, s2, s2, 3) and tw.results[0].shape == (4, 7, 7, 3)
    assert conv.results[0].shape == (natural[0], natural[2], natural[3], 4)
    assert g.outputs[0] is back.results[0] and back.results[0].shape == natural
    # a conv already in the target layout is left alone, and the other direction uses the inverse permutations
    before = g.op_names()
    transform_layout(g, "NHWC")
    assert g.op_names() == before
    transform_layout(g, "NCHW")
    canonicalize(g)
    assert g.op_names() == ["conv"] and g.ops[0].attrs["layout"] == "NCHW"


def test_transposes_between_two_transformed_convs_cancel():
    g = Graph()
    x = g.add_input((2, 8, 16, 16), f32)
    w1 = g.add_input((8, 8, 3, 3), f32)
    w2 = g.add_input((8, 8, 3, 3), f32)
    a = {"dilation": (1, 1), "kernel_shape": (3, 3), "pad": (1, 1, 1, 1), "stride": (1, 1), "group": 1, "layout": "NCHW"}
    y = g.add_op("conv", [g.add_op("conv", [x, w1], dict(a)), w2], dict(a))
    g.set_outputs([y])
    run_llh_pipeline(g, "NHWC")
    assert g.op_names() == ["transpose", "transpose", "conv", "transpose", "conv", "transpose"]
    assert g.ops[4].operands[0] is g.ops[2].results[0]      # the second conv reads the first one's NHWC result


def test_compiler_takes_both_layouts_and_nothing_else():
    from llcompiler_amd import LLCompiler
    assert LLCompiler(target_layout="NHWC").target_layout == "NHWC"
    assert LLCompiler().target_layout == "NCHW"
    with pytest.raises(ValueError):
        LLCompiler(target_layout="NCWH")


def test_backward_ops_of_layer_norm_softmax_and_gelu_are_imported():
    """aten.native_layer_norm with its saved statistics, native_layer_norm_backward, _softmax_backward_data and
    gelu_backward are spelt with reductions and elementwise ops (fp32 arithmetic), so training-mode graphs of
    transformer blocks need no eager fallback for them."""
    from torch.fx.experimental.proxy_tensor import make_fx
    from llcompiler_amd.importer.fx_importer import is_supported, torch_translate_to_llh_graph
    aten = torch.ops.aten

    def f(x, w, b, go, y):
        out, mean, rstd = aten.native_layer_norm(x, [32], w, b, 1e-5)
        dx, dw, db = aten.native_layer_norm_backward(go, x, [32], mean, rstd, w, b, [True, True, True])
        ds = aten._softmax_backward_data(go, y, -1, torch.float32)
        dg = aten.gelu_backward(go, x)
        return out, dx, dw, db, ds, dg

    args = [torch.zeros(4, 6, 32), torch.zeros(32), torch.zeros(32), torch.zeros(4, 6, 32), torch.zeros(4, 6, 32)]
    gm = make_fx(f, tracing_mode="fake")(*args)
    calls = [n for n in gm.graph.nodes if n.op == "call_function"]
    assert all(is_supported(n) for n in calls), [str(n.target) for n in calls if not is_supported(n)]
    g = torch_translate_to_llh_graph(gm)
    names = g.op_names()
    assert names.count("layer_norm") == 1 and "rsqrt" in names and "erf" in names and "exp" in names
    shapes = [tuple(o.shape) for o in g.outputs]
    assert shapes == [(4, 6, 32), (4, 6, 32), (32,), (32,), (4, 6, 32), (4, 6, 32)]
    # the statistics are [.., 1] rows and the weight gradients reduce over every row dim
    red = [op for op in g.ops if op.name == "reduce_sum"]
    assert any(tuple(op.attrs["axis"]) == (0, 1) for op in red) and any(tuple(op.attrs["axis"]) == (2,) for op in red)
    run_llh_pipeline(g)
    kinds = [s.kind for s in make_plan(g)]
    assert "layer_norm" in kinds and kinds.count("reduce") >= 6


# ---- batch norm folded into the convolution it follows (the affine map of DecomposeOps.cpp:139-144 on the filters) ----
def _conv_bn_graph(with_conv_bias=False, second_reader=False, layout="NCHW"):
    g = Graph()
    x = g.add_input((2, 8, 16, 16) if layout == "NCHW" else (2, 16, 16, 8), f32, "x")
    w = g.add_input((8, 8, 3, 3) if layout == "NCHW" else (8, 3, 3, 8), f32, "w")
    params = [g.add_input((8,), f32, n) for n in ("scale", "bias", "mean", "var")]
    attrs = {"dilation": (1, 1), "kernel_shape": (3, 3), "pad": (1, 1, 1, 1), "stride": (1, 1), "group": 1, "layout": layout}
    if with_conv_bias:
        y = g.add_op("conv_bias", [x, w, g.add_input((8,), f32, "b")], attrs)
    else:
        y = g.add_op("conv", [x, w], attrs)
    z = g.add_op("batch_norm_inference", [y] + params, {"epsilon": 1e-5, "momentum": 0.1,
                                                         "feature_index": 1 if layout == "NCHW" else 3})
    r = g.add_op("relu", [z])
    g.set_outputs([r, y] if second_reader else [r])
    return g


@pytest.mark.parametrize("with_conv_bias", [False, True])
def test_batch_norm_behind_a_convolution_folds_into_its_filters(with_conv_bias):
    g = run_llh_pipeline(_conv_bn_graph(with_conv_bias))
    assert "batch_norm_inference" not in g.op_names()
    assert g.op_names().count("conv_bias") == 1 and "conv" not in g.op_names()
    steps = make_plan(g)
    per_call = [s for s in steps if not s.attrs.get("prepared") and s.kind not in ("view", "constant")]
    # every call launches ONE kernel: the convolution with the folded bias and the relu in its epilogue
    assert [s.kind for s in per_call] == ["conv"]
    assert per_call[0].attrs["epilogue"]["act"] == "relu" and per_call[0].attrs["epilogue"]["bias"] is not None
    prepared = [s for s in steps if s.attrs.get("prepared") and s.kind == "ew"]
    progs = [[i[0] for i in s.attrs["insts"]] for s in prepared]
    assert ["add", "sqrt", "div"] in progs and ["mul"] in progs
    assert (["sub", "mul", "add"] if with_conv_bias else ["neg", "mul", "add"]) in progs
    # every operand of the prepared programs is a graph input or another prepared value, never the activation
    for s in prepared:
        assert all(v.name != "x" for v in s.inputs)


def test_batch_norm_is_not_folded_when_the_convolution_has_another_reader_or_the_statistics_are_computed():
    g = run_llh_pipeline(_conv_bn_graph(second_reader=True))
    assert "conv" in g.op_names() and "conv_bias" not in g.op_names()
    assert [s.kind for s in make_plan(g) if s.kind not in ("view", "constant")] == ["conv", "ew", "ew"]
    # statistics that the graph computes (not weights) stay with the decomposition
    g2 = Graph()
    x = g2.add_input((2, 8, 16, 16), f32, "x")
    w = g2.add_input((8, 8, 3, 3), f32, "w")
    v = g2.add_input((8,), f32, "v")
    var = g2.add_op("exp", [v])
    y = g2.add_op("conv", [x, w], {"dilation": (1, 1), "kernel_shape": (3, 3), "pad": (1, 1, 1, 1), "stride": (1, 1), "group": 1})
    z = g2.add_op("batch_norm_inference", [y, v, v, v, var], {"epsilon": 1e-5, "momentum": 0.1, "feature_index": 1})
    g2.set_outputs([z])
    run_llh_pipeline(g2)
    assert "conv_bias" not in g2.op_names() and not g2.prepared


def test_batch_norm_fold_in_the_channels_last_layout():
    g = run_llh_pipeline(_conv_bn_graph(layout="NHWC"), target_layout="NHWC")
    per_call = [s for s in make_plan(g) if not s.attrs.get("prepared") and s.kind not in ("view", "constant")]
    assert [s.kind for s in per_call] == ["conv"] and per_call[0].attrs["layout"] == "NHWC"


# ---- a symbol's value as an operand of a tensor op: llh.scalar_cast (LLHOps.td:120-127; the importer writes
#      scalar_cast + convert_to, fx_translate.py:309-323) ----
def test_scalar_cast_of_a_symbol_becomes_an_immediate_of_the_program():
    from llcompiler_amd.llh.text import parse_llh, print_llh
    text = '''func.func @main(%arg0: tensor<?x4xf32> {func.input_symbol_0 = "s0"}) -> tensor<?x4xf32> attributes {entrance} {
      %0 = "llh.constant"() <{value = 0 : i64}> : () -> i64
      %1 = "llh.dim"(%arg0, %0) : (tensor<?x4xf32>, i64) -> i64
      %c = "llh.constant"() <{value = 2 : i64}> : () -> i64
      %2 = "llh.mul"(%1, %c) : (i64, i64) -> i64
      %3 = "llh.scalar_cast"(%2) : (i64) -> tensor<1xi64>
      %4 = "llh.convert_to"(%3) : (tensor<1xi64>) -> tensor<1xf32>
      %5 = "llh.div"(%arg0, %4) : (tensor<?x4xf32>, tensor<1xf32>) -> tensor<?x4xf32>
      return %5 : tensor<?x4xf32>
    }'''
    g = run_llh_pipeline(parse_llh(text))
    assert g.op_names() == ["scalar_cast", "div"]           # the convert folded into the cast
    cast = g.ops[0]
    assert cast.results[0].dtype == f32 and evaluate(cast.attrs["value"], {"s0": 5}) == 10
    ew = [s for s in make_plan(g) if s.kind == "ew"]
    assert len(ew) == 1 and [v.name for v in ew[0].inputs] == ["arg0"]
    (op, dst, a, b), = ew[0].attrs["insts"]
    assert op == "div" and a == "in0" and isinstance(b, Expr) and evaluate(b, {"s0": 3}) == 6
    # and it survives a trip through the printer
    again = run_llh_pipeline(parse_llh(print_llh(g)))
    (name,) = again.symbols()  # (the printer writes no symbol names: the reader makes one up for the dynamic extent)
    assert again.op_names() == ["scalar_cast", "div"] and evaluate(again.ops[0].attrs["value"], {name: 7}) == 14


def test_real_valued_symbol_expressions():
    from llcompiler_amd.llh.expr import is_float, sqrt, to_float
    e = 1.0 / sqrt(to_float(s0))
    assert is_float(e) and not is_float(s0 * 2 + 1) and is_float(s0 / 4) and not is_float(s0 // 4)
    assert evaluate(e, {"s0": 64}) == 0.125 and evaluate(s0 ** 2, {"s0": 3}) == 9 and evaluate(-(s0 / 4), {"s0": 2}) == -0.5
    assert sqrt(16) == 4.0 and to_float(3) == 3.0


def test_symbol_valued_operands_import_as_scalar_casts():
    """x / x.shape[0] + x.sum(0) * x.shape[0] with a dynamic batch: the importer keeps the extent as an expression,
    writes llh.scalar_cast for it (fx_translate.py:309-323 writes scalar_cast + convert_to) and the planner makes it an
    immediate; scores / sqrt(q.shape[-1]) becomes the product's epilogue scale.  Nodes whose scalar arithmetic cannot
    be kept are reported unsupported, so that the partitioner leaves them to eager instead of failing at import."""
    from torch.export import Dim
    from llcompiler_amd.compiler.aot import compile_module
    from llcompiler_amd.importer.fx_importer import is_supported

    class M(torch.nn.Module):
        def forward(self, x):
            return x / x.shape[0] + x.sum(0) * x.shape[0]

    class S(torch.nn.Module):
        def forward(self, q, k):
            return (q @ k.transpose(-1, -2)) / torch._sym_sqrt(q.shape[-1])

    cm = compile_module(M(), (torch.randn(4, 8),), dynamic_shapes=({0: Dim("b", min=2, max=64)},))
    g = cm.engine.graph
    casts = [op for op in g.ops if op.name == "scalar_cast"]
    assert len(casts) == 2 and all(c.results[0].dtype == f32 for c in casts)
    (name,) = g.symbols()
    assert all(evaluate(c.attrs["value"], {name: 12}) == 12 for c in casts)
    ew = [s for s in cm.engine.steps if s.kind == "ew"]
    assert sorted(i[0] for s in ew for i in s.attrs["insts"]) == ["add", "div", "mul"]
    d = Dim("d", min=2, max=64)
    cs = compile_module(S(), (torch.randn(3, 4, 8), torch.randn(3, 4, 8)), dynamic_shapes=({2: d}, {2: d}))
    (bmm,) = [s for s in cs.engine.steps if s.kind == "batch_matmul"]
    alpha = bmm.attrs["epilogue"]["alpha"]
    (name,) = cs.engine.graph.symbols()
    assert isinstance(alpha, Expr) and evaluate(alpha, {name: 64}) == 0.125
    # is_supported: a symbolic operand on a translator that has no place for one is refused up front
    gm = torch.export.export(M(), (torch.randn(4, 8),), dynamic_shapes=({0: Dim("b", min=2, max=64)},)).run_decompositions().graph_module
    calls = [n for n in gm.graph.nodes if n.op == "call_function"]
    assert all(is_supported(n) for n in calls)
    sym_node = next(n for n in calls if n.target is torch.ops.aten.sym_size.int)
    fake = next(n for n in calls if n.target is torch.ops.aten.sum.dim_IntList)
    saved = fake.args
    fake.args = (saved[0], sym_node)          # a reduction over a symbol-valued axis: no translator takes that
    assert not is_supported(fake)
    fake.args = saved


def test_softmax_half_to_float_widens_before_the_softmax():
    """aten._softmax(x, -1, half_to_float=True) on a 16-bit input returns fp32 probabilities computed in fp32: the
    convert sits in front of llh.softmax, not behind it."""
    from llcompiler_amd.compiler.aot import compile_module

    class S(torch.nn.Module):
        def forward(self, x):
            return torch.softmax(x, dim=-1, dtype=torch.float32)

    g = compile_module(S(), (torch.randn(4, 16).to(torch.float16),)).engine.graph
    names = g.op_names()
    assert names.index("convert_to") < names.index("softmax")
    sm = next(op for op in g.ops if op.name == "softmax")
    assert sm.operands[0].dtype == f32 and sm.results[0].dtype == f32


def test_integer_sums_of_extents_have_one_form():
    """Extents are compared structurally (a same-shape add behind a convolution becomes its residual only if the two
    shapes are equal), so sums, differences and integer multiples collapse to one canonical form: the extent of a
    padded stride-1 window is the extent it was computed from."""
    h, w = Expr.sym("s0"), Expr.sym("s1")
    assert (h + 1 + 1 - 2 - 1) // 1 + 1 == h           # 3x3 window, pad 1, stride 1
    assert (h + 3 + 3 - 6 - 1) // 1 + 1 == h           # 7x7 window, pad 3
    assert 2 * (h + 1) - 2 == 2 * h and h * 2 - h == h and (3 - h) + h == 3 and h - h == 0
    pooled = (h + 1 + 1 - 2 - 1) // 2 + 1              # 3x3 window, pad 1, stride 2: stays a quotient
    assert pooled == (h - 1) // 2 + 1 and (pooled + 2 - 3) // 1 + 1 == pooled
    assert (h + w) - w == h and (h * w + 4) - 4 == h * w
    for e, want in (((h + 1 + 1 - 2 - 1) // 2 + 1, 4), (2 * (h + 1) - 2 + w, 17), ((3 - h) * 2 + w, -5)):
        assert evaluate(e, {"s0": 7, "s1": 3}) == want
    assert repr(h / 2 + 1.5) == "((s0 / 2) + 1.5)"     # real-valued trees stay as written


def test_residual_adds_fuse_under_symbolic_image_extents():
    """A basic block traced with symbolic height and width: conv(3x3, pad 1) of a [N, C, H', W'] tensor has the shape
    of the block's input, and the add + relu behind it become the convolution's epilogue."""
    from llcompiler_amd.llh.passes import run_llh_pipeline
    g = Graph()
    n, hh, ww = Expr.sym("s0"), Expr.sym("s1"), Expr.sym("s2")
    x = g.add_input((n, 8, hh, ww), f32)
    w1 = g.add_input((8, 8, 3, 3), f32)
    w2 = g.add_input((8, 8, 3, 3), f32)
    attrs = {"dilation": (1, 1), "kernel_shape": (3, 3), "pad": (1, 1, 1, 1), "stride": (1, 1), "group": 1}
    y = g.add_op("relu", [g.add_op("conv", [x, w1], dict(attrs))])
    c2 = g.add_op("conv", [y, w2], dict(attrs))
    assert tuple(c2.shape) == tuple(x.shape)
    z = g.add_op("relu", [g.add_op("add", [c2, x])])
    g.set_outputs([z])
    run_llh_pipeline(g)
    steps = [s for s in make_plan(g) if s.kind not in ("view", "constant")]
    assert [s.kind for s in steps] == ["conv", "conv"]
    assert steps[1].attrs["epilogue"]["residual"] is not None and steps[1].attrs["epilogue"]["act"] == "relu"


def test_symbols_seen_only_inside_input_extents_are_solved_for():
    """A partition of a dynamically shaped graph whose inputs are all results of strided windows: the symbol of the
    image size appears only inside their extents.  Any value that reproduces the given extents serves (the other
    extents are functions of those), an inconsistent set of extents is refused."""
    from llcompiler_amd.executor.engine import Torch_ExecutionEngine

    class FakeInput:
        def __init__(self, shape):
            self.shape = shape
    g = Graph()
    s, b = Expr.sym("s7"), Expr.sym("s0")
    half = (s - 1) // 2 + 1
    quarter = (half - 1) // 2 + 1
    x = g.add_input((b, 8, half, half), f32)
    y = g.add_input((b, 8, quarter, quarter), f32)
    g.set_outputs([g.add_op("relu", [x])])
    eng = Torch_ExecutionEngine.__new__(Torch_ExecutionEngine)
    eng.graph = g
    env = eng.bind_symbols((), [FakeInput((4, 8, 32, 32)), FakeInput((4, 8, 16, 16))])
    assert env["s0"] == 4 and evaluate(half, env) == 32 and evaluate(quarter, env) == 16
    env = eng.bind_symbols((), [FakeInput((2, 8, 29, 29)), FakeInput((2, 8, 15, 15))])
    assert evaluate(half, env) == 29 and evaluate(quarter, env) == 15
    with pytest.raises(KeyError):
        eng.bind_symbols((), [FakeInput((2, 8, 29, 29)), FakeInput((2, 8, 11, 11))])
