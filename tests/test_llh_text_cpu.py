"""The LLH text reader and printer (MLIR generic op syntax, the wire format between the reference's importer and its
compiler and the language of its lit tests).  The programs below are written in that syntax after the reference's own
test inputs (test/RunnerTest/abs.mlir, test/Conversion/LLHToHLO/llh_to_hlo.mlir, preprocessing_llh_to_hlo.mlir):
same ops, same attribute spellings, same scalar (i64) side."""
import pytest
import torch

from llcompiler_amd.executor.planner import make_plan
from llcompiler_amd.llh.expr import Expr, evaluate
from llcompiler_amd.llh.passes import run_llh_pipeline
from llcompiler_amd.llh.text import LLHSyntaxError, parse_llh, print_llh

ABS_RUNNER = '''
module{
    func.func @main() -> () attributes {entrance} {
        %const = "llh.constant"() <{value = dense<-1.000000e+00> : tensor<2xf32>}> : () -> tensor<2xf32>
        %0 = "llh.abs"(%const) : (tensor<2xf32>) -> tensor<2xf32>
        // CHECK-NEXT: [1,  1]
        "llh.print"(%0) <{prefix_description = "abs"}>: (tensor<2xf32>) -> ()
        return
  }
}'''

CONV_AND_SHAPES = '''
// -----
func.func @conv_nchw_fchw(%arg0: tensor<4x3x5x5xf32> , %arg1: tensor<?x3x?x?xf32>) -> tensor<?x4x?x?xf32> attributes {entrance} {
    %2 = "llh.conv"(%arg1, %arg0) <{dilation = array<i64: 2, 2>, group = 1 : i64, kernel_shape = array<i64: 5, 5>, layout = #llh.Layout<NCHW>, pad = array<i64: 2, 2, 2, 2>, stride = array<i64: 2, 2>}> : (tensor<?x3x?x?xf32>, tensor<4x3x5x5xf32>) -> tensor<?x4x?x?xf32>
    return %2 : tensor<?x4x?x?xf32>
}
// -----
func.func @slice_reshape_broadcast(%arg0: tensor<?x?x?x?xf32>) -> tensor<1x?x?x?xf32> attributes {entrance} {
  %c0_i64 = "llh.constant"() <{value = 0 : i64}> : () -> i64
  %c1_i64 = "llh.constant"() <{value = 1 : i64}> : () -> i64
  %c2_i64 = "llh.constant"() <{value = 2 : i64}> : () -> i64
  %c3_i64 = "llh.constant"() <{value = 3 : i64}> : () -> i64
  %0 = "llh.dim"(%arg0, %c1_i64) <{symbol = @s1}> : (tensor<?x?x?x?xf32>, i64) -> i64
  %1 = "llh.dim"(%arg0, %c2_i64) : (tensor<?x?x?x?xf32>, i64) -> i64
  %2 = "llh.dim"(%arg0, %c3_i64) : (tensor<?x?x?x?xf32>, i64) -> i64
  %3 = "llh.stride_slice"(%arg0, %c0_i64, %c0_i64, %c0_i64, %c0_i64, %c1_i64, %0, %1, %2, %c1_i64, %c1_i64, %c1_i64, %c1_i64) <{operandSegmentSizes = array<i32: 1, 4, 4, 4>}> : (tensor<?x?x?x?xf32>, i64, i64, i64, i64, i64, i64, i64, i64, i64, i64, i64, i64) -> tensor<1x?x?x?xf32>
  %4 = "llh.constant"() <{value = dense<2.000000e+00> : tensor<1xf32>}> : () -> tensor<1xf32>
  %5 = "llh.reshape"(%4, %c1_i64, %c1_i64, %c1_i64, %c1_i64) : (tensor<1xf32>, i64, i64, i64, i64) -> tensor<1x1x1x1xf32>
  %10 = "llh.broadcast_to"(%5, %c1_i64, %0, %1, %2) <{cast_dims = array<i64: 0, 1, 2, 3>}> : (tensor<1x1x1x1xf32>, i64, i64, i64, i64) -> tensor<1x?x?x?xf32>
  %11 = "llh.mul"(%3, %10) : (tensor<1x?x?x?xf32>, tensor<1x?x?x?xf32>) -> tensor<1x?x?x?xf32>
  return %11 : tensor<1x?x?x?xf32>
}
'''


def test_runner_program_parses_to_constant_abs_and_returns_what_it_prints():
    g = parse_llh(ABS_RUNNER)
    assert g.op_names() == ["constant", "abs"] and g.inputs == []
    const = g.ops[0]
    assert tuple(const.results[0].shape) == (2,) and const.attrs["value"] == -1.0 and const.results[0].dtype == torch.float32
    assert g.outputs == [g.ops[1].results[0]]          # no func result: the printed value is the observable


def test_conv_attributes_and_symbolic_result_shape():
    g = parse_llh(CONV_AND_SHAPES, func="conv_nchw_fchw")
    (conv,) = g.ops
    assert conv.name == "conv" and [v.name for v in conv.operands] == ["arg1", "arg0"]
    assert conv.attrs == {"dilation": (2, 2), "kernel_shape": (5, 5), "pad": (2, 2, 2, 2), "stride": (2, 2), "group": 1,
                          "layout": "NCHW"}
    n, f, oh, ow = conv.results[0].shape
    assert f == 4 and isinstance(n, Expr) and isinstance(oh, Expr)
    # out = (in + 2 + 2 - 2 * (5 - 1) - 1) / 2 + 1 (src/Dialect/LLH/IR/LLHinfersymbolShape.cpp:257-268)
    x = g.inputs[1]
    env = {x.shape[0].args[0]: 3, x.shape[2].args[0]: 33, x.shape[3].args[0]: 18}
    assert (evaluate(n, env), evaluate(oh, env), evaluate(ow, env)) == (3, (33 + 4 - 8 - 1) // 2 + 1, (18 + 4 - 8 - 1) // 2 + 1)


def test_scalar_side_becomes_symbolic_extents():
    g = parse_llh(CONV_AND_SHAPES, func="slice_reshape_broadcast")
    assert g.op_names() == ["stride_slice", "constant", "reshape", "broadcast_to", "mul"]
    x = g.inputs[0]
    sl = g.ops[0]
    assert sl.attrs["start"] == (0, 0, 0, 0) and sl.attrs["stride"] == (1, 1, 1, 1)
    assert sl.attrs["end"] == (1,) + tuple(x.shape[1:])          # llh.dim(%arg0, k) is the k-th extent of %arg0
    assert tuple(sl.results[0].shape) == (1,) + tuple(x.shape[1:])
    assert tuple(g.ops[2].results[0].shape) == (1, 1, 1, 1)
    assert tuple(g.ops[3].results[0].shape) == (1,) + tuple(x.shape[1:])
    # and the graph lowers: slice and broadcast are views, the multiply by a one-element constant one kernel
    run_llh_pipeline(g)
    kinds = [s.kind for s in make_plan(g) if s.kind not in ("view", "constant")]
    assert kinds == ["ew"]


def test_printer_round_trip_of_an_imported_model():
    from llcompiler_amd.compiler.aot import compile_module
    from llcompiler_amd.test_models import MLP, make_mlp_inputs
    g = compile_module(MLP().eval(), make_mlp_inputs(), weights="npy").engine.graph
    text = print_llh(g)
    assert '"llh.weight"() <{weight_file = "' in text and '"llh.matmul"' in text
    g2 = parse_llh(text)
    assert g2.op_names() == g.op_names()
    for a, b in zip(g.ops, g2.ops):
        assert tuple(a.results[0].shape) == tuple(b.results[0].shape) and a.results[0].dtype == b.results[0].dtype
        assert {k: v for k, v in a.attrs.items() if k != "cast_dims"} == {k: v for k, v in b.attrs.items() if k != "cast_dims"}
    assert print_llh(g2).replace("%arg", "%x") .count("llh.") == text.count("llh.")


def test_syntax_errors_are_reported():
    with pytest.raises(LLHSyntaxError):
        parse_llh("module {}")
    with pytest.raises(LLHSyntaxError):
        parse_llh('func.func @main() -> () { %0 = "llh.abs"(%nope) : (tensor<2xf32>) -> tensor<2xf32> return }')
    with pytest.raises(NotImplementedError):
        parse_llh('func.func @main(%a: tensor<2xf32>) -> () { %0 = "stablehlo.abs"(%a) : (tensor<2xf32>) -> tensor<2xf32> return }')


LINEAR_RELU = '''
func.func @main(%x: tensor<8x784xf32>, %w: tensor<512x784xf32>, %b: tensor<512xf32>, %w2: tensor<10x512xf32>) -> tensor<8x10xf32> attributes {entrance} {
  %wt = "llh.transpose"(%w) <{perms = array<i64: 1, 0>}> : (tensor<512x784xf32>) -> tensor<784x512xf32>
  %0 = "llh.matmul"(%x, %wt) : (tensor<8x784xf32>, tensor<784x512xf32>) -> tensor<8x512xf32>
  %c1 = "llh.constant"() <{value = 1 : i64}> : () -> i64
  %c512 = "llh.constant"() <{value = 512 : i64}> : () -> i64
  %br = "llh.reshape"(%b, %c1, %c512) : (tensor<512xf32>, i64, i64) -> tensor<1x512xf32>
  %1 = "llh.add"(%0, %br) : (tensor<8x512xf32>, tensor<1x512xf32>) -> tensor<8x512xf32>
  %2 = "llh.relu"(%1) : (tensor<8x512xf32>) -> tensor<8x512xf32>
  %w2t = "llh.transpose"(%w2) <{perms = array<i64: 1, 0>}> : (tensor<10x512xf32>) -> tensor<512x10xf32>
  %3 = "llh.matmul"(%2, %w2t) : (tensor<8x512xf32>, tensor<512x10xf32>) -> tensor<8x10xf32>
  %4 = "llh.exp"(%3) : (tensor<8x10xf32>) -> tensor<8x10xf32>
  %5 = "llh.abs"(%4) : (tensor<8x10xf32>) -> tensor<8x10xf32>
  return %5 : tensor<8x10xf32>
}
'''


def test_llh_plan_tool_prints_the_fused_plan(tmp_path, capsys):
    """The stand-in for `llc-opt ... | FileCheck`: text in, kernel plan out, checked line by line."""
    from llcompiler_amd.llh import plan_tool
    f = tmp_path / "linear.mlir"
    f.write_text(LINEAR_RELU)
    assert plan_tool.main([str(f)]) == 0
    lines = [l.strip() for l in capsys.readouterr().out.splitlines()]
    assert lines[0] == "plan(%x: tensor<8x784xf32>, %w: tensor<512x784xf32>, %b: tensor<512xf32>, %w2: tensor<10x512xf32>) {"
    mm = [l for l in lines if "= matmul(" in l]
    assert len(mm) == 2 and mm[0].endswith("{bias=%b, act=relu} : tensor<8x512xf32>") and mm[0].split("(")[1].startswith("%x, ")
    assert mm[1].endswith(": tensor<8x10xf32>") and "{" not in mm[1]
    assert any(l.split(" = ")[1].startswith("ew[exp abs](") for l in lines if " = " in l)
    assert not any("= ew[add" in l or "= ew[relu" in l for l in lines)      # both went into the first product
    assert lines[-2].startswith("return %") and lines[-1] == "}"
    # --emit llh prints the graph back in the input syntax, and that text plans the same way
    assert plan_tool.main([str(f), "--emit", "llh"]) == 0
    again = tmp_path / "again.mlir"
    again.write_text(capsys.readouterr().out)
    assert plan_tool.main([str(again)]) == 0
    assert [l.strip() for l in capsys.readouterr().out.splitlines()] == lines
    # one of several functions, as in the reference's split test files
    multi = tmp_path / "multi.mlir"
    multi.write_text(CONV_AND_SHAPES)
    assert plan_tool.main([str(multi), "--func", "conv_nchw_fchw"]) == 0
    out = capsys.readouterr().out
    assert "= conv(%arg1, %arg0) : tensor<?x4x?x?xf32>" in out


NHWC_CONV = '''func.func @main(%x: tensor<2x9x9x64xf32>, %w: tensor<8x3x3x64xf32>) -> tensor<2x9x9x8xf32> attributes {entrance} {
  %y = "llh.conv"(%x, %w) <{dilation = array<i64: 1, 1>, group = 1 : i64, kernel_shape = array<i64: 3, 3>, layout = #llh.Layout<NHWC>, weight_layout = #llh.Layout<FHWC>, pad = array<i64: 1, 1, 1, 1>, stride = array<i64: 1, 1>}> : (tensor<2x9x9x64xf32>, tensor<8x3x3x64xf32>) -> tensor<2x9x9x8xf32>
  return %y : tensor<2x9x9x8xf32>
}
'''


def test_conv_in_the_nhwc_layout_is_read_printed_and_read_again():
    """layout = #llh.Layout<NHWC> (include/llcompiler/Dialect/LLH/IR/LLHEnums.td:61-75): operands and result are
    [N,H,W,C] / [F,KH,KW,C] / [N,OH,OW,F]."""
    g = parse_llh(NHWC_CONV)
    (conv,) = g.ops
    assert conv.attrs["layout"] == "NHWC" and conv.results[0].shape == (2, 9, 9, 8)
    again = parse_llh(print_llh(g))
    assert again.ops[0].attrs["layout"] == "NHWC" and again.ops[0].results[0].shape == (2, 9, 9, 8)
    with pytest.raises(NotImplementedError):
        parse_llh(NHWC_CONV.replace("weight_layout = #llh.Layout<FHWC>", "weight_layout = #llh.Layout<HWCF>"))
