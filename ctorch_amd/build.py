"""Builds the HIP launch layer (ctorch_amd/csrc/*.hip -> ctorch_amd/libctorch_amd.so) for gfx950.

hipcc cross-compiles without a GPU.  Flags that matter for results:
  -ffp-contract=off            the kernels restate the reference's fp32 operation order; a fused
                               multiply-add would change bits (fusions that the reference build
                               does have are written out as explicit fma calls)
  -target-feature -packed-fp32-ops   no packed-fp32 VALU instructions
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libctorch_amd.so")
SOURCES = ["runtime.hip", "elementwise.hip", "reduce.hip", "softmax_ce.hip", "matmul.hip", "dataset.hip", "expr.hip", "typed.hip"]
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-ffp-contract=off", "-fPIC",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wall", "-Wno-unused-function"]


def _hipcc():
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    raise RuntimeError("hipcc not found")


def _run(cmd):
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # the host pass does not know the packed-fp32 feature and says so: harmless
    out = "\n".join(l for l in p.stdout.splitlines() if "packed-fp32-ops' is not a recognized feature" not in l)
    if p.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    return out


def build(verbose=False, jobs=4):
    """Compiles every source and links the shared library; always recompiles."""
    hipcc = _hipcc()
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    objs = [os.path.join(objdir, s.replace(".hip", ".o")) for s in SOURCES]

    def one(pair):
        src, obj = pair
        return _run([hipcc] + FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj])

    with ThreadPoolExecutor(max_workers=jobs) as ex:
        for out in ex.map(one, zip(SOURCES, objs)):
            if verbose and out.strip():
                print(out)
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs)
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
