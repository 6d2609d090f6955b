"""The reference's own lit test inputs, read where they lie (nothing of them is copied into this repository), fed to
the LLH text reader and to this build's shape inference.  The reference tree is only present on the build machine:
without it these tests skip.

test/Dialect/LLH/symbol_infer/infer_symbol_shape.mlir gives every op an unranked result type (tensor<*xf32>) and
holds, in its CHECK-SAME lines, the type the reference's --infer-symbol-shape pass must produce: those are known
answers for llh/infer.py, including which extents are static and which dynamic extents are the same symbol."""
import glob
import os
import re

import pytest

from llcompiler_amd.llh.expr import Expr
from llcompiler_amd.llh.graph import Value
from llcompiler_amd.llh.text import LLHSyntaxError, parse_llh

REF_TESTS = "/root/reference/test"
pytestmark = pytest.mark.skipif(not os.path.isdir(REF_TESTS), reason="the reference tree is not on this machine")


def _functions(path):
    """(function name, text of its split) for every func.func of a lit file (splits are separated by // -----)."""
    for chunk in re.split(r"//\s*-----", open(path).read()):
        for name in re.findall(r"func\.func\s+@([\w\-.]+)", chunk):
            yield name, chunk


def test_reader_takes_the_reference_lit_inputs():
    """Every function of every lit file either parses or is refused for a stated reason (ops of other dialects in
    custom syntax, ops the backend has no counterpart for, NHWC convolutions): never a crash, and the LLH dialect's
    own test files parse almost completely."""
    parsed, refused = [], []
    for path in sorted(glob.glob(REF_TESTS + "/**/*.mlir", recursive=True)):
        for name, chunk in _functions(path):
            where = "%s:@%s" % (path[len(REF_TESTS) + 1:], name)
            try:
                parse_llh(chunk, func=name)
                parsed.append(where)
            except (LLHSyntaxError, NotImplementedError) as e:
                refused.append((where, str(e)))
    assert len(parsed) >= 85, "only %d of %d functions parsed" % (len(parsed), len(parsed) + len(refused))
    llh_dialect = [w for w in parsed if w.startswith("Dialect/LLH/") and "/symbol_infer/" not in w]
    llh_refused = [w for w, _ in refused if w.startswith("Dialect/LLH/") and "/symbol_infer/" not in w]
    assert len(llh_dialect) >= 30 and len(llh_refused) <= 3, (llh_refused,)
    for where, why in refused:
        assert why, where


def _expected_types(chunk):
    """SSA name -> (op, dims, symbols) from `// CHECK: llh.<op>` / `// CHECK-SAME: [->] tensor<...>` pairs: the type
    belongs to the next statement of that op."""
    lines = chunk.splitlines()
    out = {}
    for i, line in enumerate(lines):
        m = re.match(r"\s*//\s*CHECK-SAME:\s*(?:->\s*)?tensor<([^,>]*)(?:,\s*#llh\.encoding<shapes\s*=\s*([^>]*)>)?>\s*$", line)
        if not m or i == 0:
            continue
        op = re.match(r"\s*//\s*CHECK:\s*llh\.(\w+)", lines[i - 1])
        if not op:
            continue
        for later in lines[i + 1:]:
            st = re.match(r'\s*%([\w.$-]+)\s*=\s*"llh\.(\w+)"', later)
            if st and st.group(2) == op.group(1) and st.group(1) not in out:
                dims = m.group(1).split("x")[:-1]
                syms = [t.strip().lstrip("@") for t in m.group(2).split(",")] if m.group(2) else None
                out[st.group(1)] = (op.group(1), dims, syms)
                break
    return out


def test_shape_inference_agrees_with_the_reference_known_answers():
    path = REF_TESTS + "/Dialect/LLH/symbol_infer/infer_symbol_shape.mlir"
    checked, ops_seen = 0, set()
    for name, chunk in _functions(path):
        ssa = {}
        try:
            parse_llh(chunk, func=name, ssa=ssa)
        except NotImplementedError:
            continue          # llh.empty, llh.batch_norm (training form): no counterpart here
        expected = _expected_types(chunk)
        by_symbol = {}
        for ssa_name, (op, dims, syms) in expected.items():
            v = ssa.get(ssa_name)
            assert isinstance(v, Value), "@%s %%%s (%s): not a tensor here" % (name, ssa_name, op)
            mine = ["?" if isinstance(d, Expr) else str(d) for d in v.shape]
            assert mine == dims, "@%s %%%s = llh.%s: the reference infers %s, this build %s" % (name, ssa_name, op, dims, v.shape)
            checked += 1
            ops_seen.add(op)
            # extents the reference gives the same symbol must be the same expression here
            for d, s in zip(v.shape, syms or []):
                if isinstance(d, Expr) and re.fullmatch(r"s\d+", s):
                    by_symbol.setdefault(s, []).append((ssa_name, d))
        for s, uses in by_symbol.items():
            first = uses[0][1]
            for ssa_name, d in uses[1:]:
                assert str(d) == str(first), "@%s: the reference calls both extents @%s; here %s vs %s (%%%s)" % (name, s, first, d, ssa_name)
    assert checked >= 20, checked
    assert {"transpose", "max_pool", "reshape", "adaptive_average_pool", "matmul", "batch_matmul", "stride_slice", "conv",
            "broadcast_to", "extract", "where", "reduce_max"} <= ops_seen, ops_seen


def _filecheck_lite(printed, directives):
    """The reference's CHECK / CHECK-NOT / CHECK-COUNT-n / CHECK-SAME lines, restricted to those that name an
    llh op, against the printed graph: CHECK finds the next line with the pattern, CHECK-SAME looks at the same
    line, CHECK-NOT forbids the pattern between its neighbours' matches (or up to the end)."""
    lines = printed.splitlines()
    pos, pending_not = 0, []
    for kind, pat in directives:
        if kind == "CHECK-NOT":
            pending_not.append(pat)
            continue
        if kind == "CHECK-SAME":
            assert pos > 0 and pat in lines[pos - 1], "CHECK-SAME %r not on line %r" % (pat, lines[pos - 1] if pos else None)
            continue
        count = int(kind.split("-")[-1]) if kind.startswith("CHECK-COUNT") else 1
        for _ in range(count):
            hit = next((k for k in range(pos, len(lines)) if pat in lines[k]), None)
            assert hit is not None, "CHECK %r not found after line %d of:\n%s" % (pat, pos, printed)
            for bad in pending_not:
                assert not any(bad in l for l in lines[pos:hit]), "CHECK-NOT %r violated in:\n%s" % (bad, printed)
            pending_not = []
            pos = hit + 1
    for bad in pending_not:
        assert not any(bad in l for l in lines[pos:]), "CHECK-NOT %r violated in:\n%s" % (bad, printed)


# (file, function, which of its directives apply here: all those naming these op spellings)
_PASS_LEVEL = [
    ("Dialect/LLH/canonicalize.mlir", "fold_two_abs", ("llh.abs",)),
    ("Dialect/LLH/canonicalize.mlir", "fold_reshape", ("llh.reshape",)),
    ("Dialect/LLH/canonicalize.mlir", "fold_broadcast", ("llh.broadcast_to",)),
    ("Dialect/LLH/canonicalize.mlir", "fold_convert_to", ("llh.convert_to",)),
    ("Dialect/LLH/fold.mlir", "add_zore_fold", ("llh.add",)),
    ("Dialect/LLH/fold.mlir", "sub_same_fold", ("llh.sub",)),
    ("Dialect/LLH/fold.mlir", "mul_fold", ("llh.mul",)),
    ("Dialect/LLH/decompose_ops.mlir", "batch_norm", ("llh.add", "llh.sqrt", "llh.reshape", "llh.broadcast_to", "llh.sub", "llh.mul",
                                                      "llh.div", "llh.batch_norm_inference")),
    ("Dialect/LLH/operation-legalization.mlir", "extract", ("llh.extract", "-> tensor<1xf32>")),
    ("Dialect/LLH/operation-legalization.mlir", "weight_refine", ("llh.weight", "-> tensor<1xf32>")),
]


@pytest.mark.parametrize("path,func,patterns", _PASS_LEVEL)
def test_rewrites_satisfy_the_reference_check_lines(path, func, patterns):
    """The reference's pass-level expectations (its FileCheck lines) hold for this build's rewrites of the same input,
    for the passes it has a counterpart of: canonicalisation and folding, batch-norm decomposition, and the
    refinement of one-element results to tensor<1xT>."""
    from llcompiler_amd.llh.passes import run_llh_pipeline
    from llcompiler_amd.llh.text import _type_str

    def listing(g):   # one line per op: name and result type, in the reference's spelling
        return "\n".join('%%%s = "llh.%s"(%s) -> %s' % (op.results[0].name, op.name, ", ".join("%" + o.name for o in op.operands),
                                                      _type_str(op.results[0])) for op in g.ops)
    ran = 0
    for name, chunk in _functions(REF_TESTS + "/" + path):
        if name != func:
            continue
        body = chunk[chunk.index("@" + func):]
        directives = []
        for kind, pat in re.findall(r"//\s*(CHECK(?:-NOT|-COUNT-\d+|-SAME)?):\s*(.*)", body):
            pat = pat.strip()
            if any(pat == p or (p.startswith("->") and pat == p) for p in patterns):
                directives.append((kind, pat))
        try:
            g = parse_llh(chunk, func=func)
        except NotImplementedError:
            continue          # (a second function of the same name with scalar-only content)
        if not any(op.results[0].rank >= 0 for op in g.ops) and not directives:
            continue
        run_llh_pipeline(g)
        _filecheck_lite(listing(g), directives)
        ran += 1
    assert ran >= 1, "no function @%s in %s" % (func, path)


def test_operator_support_and_decompositions_cover_the_reference_tables():
    """llcompiler/compiler/torch_compile_config.py, read as text: every tensor op the reference's LLC_SUPPORT_DICT
    names has a translator here, its two symbol-arithmetic entries are handled as symbolic extents, and the
    decomposition set differs from the reference's exactly by the documented entries (ops that are translated
    directly instead: addmm, add / sub / mul / div, _softmax)."""
    import operator
    import torch
    from llcompiler_amd.compiler.torch_compile_config import LLC_DECOMPOSITIONS
    from llcompiler_amd.importer import fx_importer
    text = open("/root/reference/llcompiler/compiler/torch_compile_config.py").read()

    def table(name):
        body = text[text.index(name + " = {"):]
        return body[:body.index("\n}")]

    def resolve(dotted):
        obj = {"torch": torch, "_operator": operator}[dotted.split(".")[0]]
        for part in dotted.split(".")[1:]:
            obj = getattr(obj, part)
        return obj

    keys = re.findall(r'^\s*"([\w.]+)":\s*None', table("LLC_SUPPORT_DICT"), re.M)
    assert len(keys) >= 25
    symbolic = {"torch._sym_sqrt", "_operator.mul"}
    for key in keys:
        target = resolve(key)
        if key in symbolic:
            assert target in fx_importer._SYMBOLIC_TARGETS or target in fx_importer.TORCH_FUNCTION_TRANSLATE, key
        else:
            assert target in fx_importer.TORCH_FUNCTION_TRANSLATE, "the reference compiles %s, this build has no translator" % key
    theirs = set()
    for name in re.findall(r"^\s*(?:torch\.ops\.)?aten\.([\w.]+),", table("LLC_DECOMPOSITIONS"), re.M):
        op = torch.ops.aten
        for part in name.split("."):
            op = getattr(op, part)
        theirs.add(op)
    aten = torch.ops.aten
    translated_directly = {aten.addmm, aten.add, aten.sub, aten.mul, aten.div, aten._softmax}
    assert theirs - set(LLC_DECOMPOSITIONS) == translated_directly
    for packet in translated_directly:   # each of them reaches a translator through one of its overloads
        assert any(getattr(t, "overloadpacket", None) is packet for t in fx_importer.TORCH_FUNCTION_TRANSLATE), packet


def test_every_aten_target_the_reference_translates_has_a_translator():
    """The ATen / prims names registered by llcompiler/importer/fx_op_translate/*.py (read as text) all have a
    translator here, but for three that the reference itself cannot lower or that only exist in training graphs:
    native_dropout (llh.drop has no lowering), _native_batch_norm_legit_functional (training batch norm) and
    empty.memory_format (an uninitialised buffer); such nodes stay in torch eager."""
    from llcompiler_amd.importer import fx_importer
    names = set()
    for path in glob.glob("/root/reference/llcompiler/importer/fx_op_translate/*.py"):
        for m in re.finditer(r"@TORCH_FUNCTION_TRANSLATE\((.*?)\)\s*\n", open(path).read(), re.S):
            names |= set(re.findall(r'"((?:aten|prims)::[\w.]+)"', m.group(1)))
    assert len(names) >= 50
    have = set()
    for t in list(fx_importer.TORCH_FUNCTION_TRANSLATE) + list(fx_importer._SYMBOLIC_TARGETS):
        schema = getattr(t, "_schema", None)
        if schema is not None:
            have.add(schema.name + ("." + schema.overload_name if schema.overload_name else ""))
    import torch
    if "inductor_force_stride_order" not in dir(torch.ops.prims):
        names.discard("prims::inductor_force_stride_order")   # the op is defined by importing torch._inductor
    missing = sorted(n for n in names if not any(h == n or h.startswith(n + ".") for h in have))
    assert missing == ["aten::_native_batch_norm_legit_functional", "aten::empty.memory_format", "aten::native_dropout"], missing


def test_every_declared_llh_op_is_accounted_for():
    """include/llcompiler/Dialect/LLH/IR/LLHOps.td, read as text: each of the dialect's ops is either read and
    executed by this build, or part of the symbol bookkeeping that becomes symbolic extents here, or left out
    for a stated reason."""
    from llcompiler_amd.llh import graph
    from llcompiler_amd.llh.text import _SKIPPED
    text = open("/root/reference/include/llcompiler/Dialect/LLH/IR/LLHOps.td").read()
    # (LLH_Op<"name", ...> for most ops; llh.print is declared with the dialect spelt out: Op<LLH_Dialect, "print", ...>)
    declared = set(re.findall(r'def\s+LLH_\w+\s*:\s*\w+<\s*(?:LLH_Dialect\s*,\s*)?"([\w.]+)"', text))
    assert "print" in declared and "scalar_cast" in declared
    assert len(declared) >= 50
    executed = set(graph.UNARY_OPS) | set(graph.BINARY_OPS) | {
        "constant", "weight", "dim", "extract", "stride_slice", "reshape", "flatten", "broadcast_to", "convert_to",
        "adaptive_average_pool", "transpose", "compare", "conv", "conv_bias", "matmul", "batch_matmul", "layer_norm",
        "batch_norm_inference", "max_pool", "where", "softmax", "reduce_max", "reduce_min", "reduce_sum", "torch_symbolic_int",
        "scalar_cast",   # a symbol's value as a one-element tensor: an immediate of the consuming kernel, per binding
        "print"}         # the reader returns the printed tensors of a function without results
    bookkeeping = {"symbolic_bind", "encoding_bind", "symbol_bind", "symbolic_int", "symbolic_cast", "symbol_relation_map",
                   "symbol_binary_relation", "symbol_relation"}
    left_out = {
        "aot": "marks a function for the reference's ahead-of-time driver",
        "shape_of": "declared, no lowering and no importer use in the reference",
        "slice": "declared, no lowering in the reference (stride_slice is what its importer emits)",
        "cat": "declared, no lowering in the reference",
        "expand": "declared, no lowering in the reference (decomposed to broadcast_to before import)",
        "empty": "an uninitialised buffer: only meaningful as an out-parameter",
        "drop": "dropout, declared, no lowering in the reference; inference graphs have none",
        "batch_norm": "training-mode batch norm (updates running statistics)",
    }
    assert bookkeeping <= set(_SKIPPED)          # the reader drops them: extents are expressions here
    unaccounted = declared - executed - bookkeeping - set(left_out)
    assert not unaccounted, sorted(unaccounted)
    assert not (set(left_out) & executed)
