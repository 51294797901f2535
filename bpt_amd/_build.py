"""Compiles the three native libraries in-tree:

  bpt_amd/csrc/libbptgraph.so  host C++ (g++)            <- bptgraph.cpp
  bpt_amd/csrc/libbptattn.so   gfx950 HIP (hipcc)        <- bptattn.hip
  bpt_amd/csrc/libbptplan.so   gfx950 HIP (hipcc)        <- bptplan.hip  (plans built on the GPU; rocPRIM headers)

hipcc cross-compiles for gfx950 without a GPU.  Run `python -m bpt_amd._build`.
"""
import os
import subprocess
import sys

CSRC = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc")
GRAPH_SO = os.path.join(CSRC, "libbptgraph.so")
ATTN_SO = os.path.join(CSRC, "libbptattn.so")
PLAN_SO = os.path.join(CSRC, "libbptplan.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
HIP_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    # packed FP32 forms (v_pk_*_f32) are kept out of the generated code on purpose
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-variable", "-Wno-unused-but-set-variable",
]


# The target feature above only exists for the GPU; hipcc also hands it to its host pass, which reports it once per
# internal step with exactly this line and ignores it.  The line is dropped so that real diagnostics stand out.
_HOST_PASS_NOTE = "'-packed-fp32-ops' is not a recognized feature for this target (ignoring feature)"


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(line for line in proc.stdout.splitlines() if line.strip() != _HOST_PASS_NOTE)
    if out.strip():
        print(out, flush=True)
    if proc.returncode != 0:
        raise subprocess.CalledProcessError(proc.returncode, cmd)


def build_graph(verbose=True):
    _run(["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-Wextra",
          os.path.join(CSRC, "bptgraph.cpp"), "-o", GRAPH_SO], verbose)
    return GRAPH_SO


def build_attn(verbose=True):
    _run([HIPCC] + HIP_FLAGS + [os.path.join(CSRC, "bptattn.hip"), "-o", ATTN_SO], verbose)
    return ATTN_SO


def build_plan(verbose=True):
    _run([HIPCC] + HIP_FLAGS + [os.path.join(CSRC, "bptplan.hip"), "-o", PLAN_SO], verbose)
    return PLAN_SO


def build_all(verbose=True):
    return build_graph(verbose), build_attn(verbose), build_plan(verbose)


if __name__ == "__main__":
    build_all()
    sys.exit(0)
