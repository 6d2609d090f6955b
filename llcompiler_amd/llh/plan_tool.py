"""llh-plan: reads an LLH graph in MLIR generic op syntax and prints what this backend makes of it.

The reference drives its pass-level tests with `llc-opt` (tools/llc-opt/llc-opt.cpp:37-60: an mlir-opt with the LLH
dialect registered) piped into FileCheck (test/Conversion/LLHToHLO/llh_to_hlo.mlir:1).  Here the counterpart of a
pass pipeline's output is the kernel plan: which ops were fused into which call.  Usage:

    python -m llcompiler_amd.llh.plan_tool [--func NAME] [--emit plan|llh|both] [--no-pipeline] FILE|-

`--emit llh` prints the graph after the LLH-level rewrites (the same text syntax), `--emit plan` one line per
kernel step:

    %7 = conv(%arg0, %w) {bias=%b, residual=%3, act=relu} : tensor<16x64x56x56xf32>
    %9 = ew[add relu](%7, %8) : tensor<16x64x56x56xf32>
    %10 = view.reshape(%9) : tensor<16x200704xf32>

Needs no GPU and no HIP library: planning is host logic.
"""
import argparse
import sys

from ..executor.planner import make_plan
from .passes import run_llh_pipeline
from .text import _type_str, parse_llh, print_llh


def _name(v):
    return "%" + v.name


def step_text(st):
    """One line for a planned step: result, kind with what was fused into it, operands, result type."""
    a = st.attrs if isinstance(st.attrs, dict) else {}
    kind = st.kind
    extra = ""
    if kind == "ew":
        kind = "ew[%s]" % " ".join(i[0] for i in a["insts"])
    elif kind == "view":
        kind = "view.%s" % a["op"]
    elif kind == "reduce":
        kind = "reduce.%s" % a["kind"]
        extra = " {axis=%s}" % list(a["axis"])
    elif kind in ("matmul", "batch_matmul", "conv"):
        e = a["epilogue"]
        parts = []
        if e.get("alpha", 1.0) != 1.0:
            parts.append("alpha=%g" % e["alpha"])
        for k in ("bias", "residual"):
            if e.get(k) is not None:
                parts.append("%s=%s" % (k, _name(e[k])))
        if e.get("act"):
            parts.append("act=%s" % e["act"])
        extra = " {%s}" % ", ".join(parts) if parts else ""
    elif kind == "constant":
        v = a["value"]
        extra = " {value=%s}" % ("dense of %d" % len(v) if isinstance(v, (list, tuple)) else repr(v))
    return "%s = %s(%s)%s : %s" % (_name(st.output), kind, ", ".join(_name(v) for v in st.inputs), extra, _type_str(st.output))


def plan_text(graph):
    lines = ["plan(%s) {" % ", ".join("%s: %s" % (_name(v), _type_str(v)) for v in graph.inputs)]
    lines += ["  " + step_text(st) for st in make_plan(graph)]
    outs = [o for o in graph.outputs if hasattr(o, "name")]
    lines.append("  return %s" % ", ".join(_name(o) for o in outs))
    lines.append("}")
    return "\n".join(lines) + "\n"


def main(argv=None):
    ap = argparse.ArgumentParser(prog="llh-plan", description=__doc__.split("\n\n")[0])
    ap.add_argument("file", help="LLH text file, or - for stdin")
    ap.add_argument("--func", default=None, help="function to read when the file holds several (default: the entrance)")
    ap.add_argument("--emit", choices=("plan", "llh", "both"), default="plan")
    ap.add_argument("--no-pipeline", action="store_true", help="plan the graph as written, without the LLH-level rewrites")
    ap.add_argument("--target-layout", choices=("NCHW", "NHWC"), default="NCHW",
                    help="layout the convolutions are rewritten to (the reference's --transform-layout option)")
    args = ap.parse_args(argv)
    text = sys.stdin.read() if args.file == "-" else open(args.file).read()
    graph = parse_llh(text, func=args.func)
    if not args.no_pipeline:
        run_llh_pipeline(graph, args.target_layout)
    out = ""
    if args.emit in ("llh", "both"):
        out += print_llh(graph)
    if args.emit in ("plan", "both"):
        out += plan_text(graph)
    sys.stdout.write(out)
    return 0


if __name__ == "__main__":
    sys.exit(main())
