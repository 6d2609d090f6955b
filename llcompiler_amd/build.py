"""Builds libllc_hip.so (the gfx950 kernel library) in-tree with hipcc.

    python -m llcompiler_amd.build [--force]

hipcc cross-compiles for gfx950 without a GPU, so this runs anywhere the ROCm toolchain is
installed.  Objects go to llcompiler_amd/csrc/build/, the library to llcompiler_amd/lib/.
"""
import concurrent.futures
import glob
import os
import subprocess
import sys

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
CSRC = os.path.join(PKG, "csrc")
OBJ = os.path.join(CSRC, "build")
LIB_DIR = os.path.join(PKG, "lib")
LIB = os.path.join(LIB_DIR, "libllc_hip.so")
# exports `main(void**)`, the symbol the reference's loader resolves, forwarding to libllc_hip.so
ENTRY_LIB = os.path.join(LIB_DIR, "libllc_entry.so")
ENTRY_SRC = os.path.join(CSRC, "entry_main.c")
# a host in plain C that loads a plan file and runs it through the C-ABI alone
RUN_PLAN = os.path.join(LIB_DIR, "llc_run_plan")
RUN_PLAN_SRC = os.path.join(CSRC, "run_plan_main.c")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "-O3", "--offload-arch=gfx950", "-std=c++17", "-fPIC",
    # hipcc -O3 forms packed fp32 ops by itself; some forms misbehave on this hardware pool
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    "-I", os.path.join(ROOT, "include"), "-I", CSRC,
]


def sources():
    return sorted(glob.glob(os.path.join(CSRC, "*.hip")))


def _compile(src):
    obj = os.path.join(OBJ, os.path.basename(src)[:-4] + ".o")
    cmd = [HIPCC] + FLAGS + ["-c", src, "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "is not a recognized feature for this target" not in l)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, err))
    return obj, err


def build(force=True, jobs=None, verbose=False):
    """Compile every HIP source and link the shared library.  Returns its path."""
    os.makedirs(OBJ, exist_ok=True)
    os.makedirs(LIB_DIR, exist_ok=True)
    srcs = sources()
    if not srcs:
        raise RuntimeError("no HIP sources under %s" % CSRC)
    deps = srcs + [ENTRY_SRC, RUN_PLAN_SRC] + glob.glob(os.path.join(CSRC, "*.hpp")) + glob.glob(os.path.join(ROOT, "include", "*.h"))
    if not force and os.path.exists(LIB) and os.path.exists(ENTRY_LIB) and os.path.exists(RUN_PLAN) and all(os.path.getmtime(LIB) >= os.path.getmtime(d) for d in deps):
        return LIB
    jobs = jobs or min(8, os.cpu_count() or 1, len(srcs))
    with concurrent.futures.ThreadPoolExecutor(jobs) as ex:
        results = list(ex.map(_compile, srcs))
    objs = [o for o, _ in results]
    if verbose:
        for _, err in results:
            if err.strip():
                print(err, file=sys.stderr)
    cmd = [HIPCC, "-shared", "-fPIC", "--offload-arch=gfx950", "-o", LIB] + objs
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stderr)
    cmd = ["gcc", "-O2", "-shared", "-fPIC", "-Wno-main", "-I", os.path.join(ROOT, "include"), ENTRY_SRC, "-o", ENTRY_LIB,
           "-L", LIB_DIR, "-lllc_hip", "-Wl,-rpath,$ORIGIN"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("building %s failed:\n%s" % (ENTRY_LIB, r.stderr))
    cmd = ["gcc", "-O2", "-std=c11", "-Wall", "-I", os.path.join(ROOT, "include"), RUN_PLAN_SRC, "-o", RUN_PLAN,
           "-L", LIB_DIR, "-lllc_hip", "-Wl,-rpath,$ORIGIN"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("building %s failed:\n%s" % (RUN_PLAN, r.stderr))
    return LIB


if __name__ == "__main__":
    print(build(force="--force" in sys.argv or True, verbose=True))
