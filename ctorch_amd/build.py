"""Builds the HIP launch layer (ctorch_amd/csrc/*.hip -> ctorch_amd/libctorch_amd.so) for gfx950.

hipcc cross-compiles without a GPU.  Flags that matter for results:
  -ffp-contract=off            the kernels restate the reference's fp32 operation order; a fused
                               multiply-add would change bits (fusions that the reference build
                               does have are written out as explicit fma calls)
  -target-feature -packed-fp32-ops   no packed-fp32 VALU instructions
"""
import json
import os
import re
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
RESOURCES = os.path.join(os.path.dirname(os.path.abspath(__file__)), "kernel_resources.json")
LIB = os.path.join(HERE, "libctorch_amd.so")
SOURCES = ["runtime.hip", "elementwise.hip", "reduce.hip", "softmax_ce.hip", "matmul.hip", "dataset.hip", "expr.hip", "expr_jit.hip", "typed.hip", "stats.hip", "head.hip"]
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
    _write_jit_text(os.path.join(objdir, "jit_text.inc"))

    def one(pair):
        src, obj = pair
        return _run([hipcc] + FLAGS + ["-Rpass-analysis=kernel-resource-usage", "-I", objdir, "-c", os.path.join(CSRC, src), "-o", obj])

    resources = {}
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        for src, out in zip(SOURCES, ex.map(one, zip(SOURCES, objs))):
            rest = _kernel_resources(src, out, resources)
            if verbose and rest.strip():
                print(rest)
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs + ["-lhiprtc"])
    # what every kernel needs (registers, spills, LDS), next to the library: a spilled register costs a
    # kernel its overlap of loads and arithmetic, so tests/test_abi_and_devmath.py refuses a build that has one
    with open(RESOURCES, "w") as f:
        json.dump(resources, f, indent=0, sort_keys=True)
    return LIB


def _write_jit_text(path):
    """devmath.h and expr_ops.h as one C++ string literal (their #include lines removed): the text that
    expr_jit.hip hands to the run-time compiler in front of every kernel it generates."""
    text = ""
    for name in ("devmath.h", "expr_ops.h"):
        for line in open(os.path.join(CSRC, name)):
            if not line.lstrip().startswith("#include"):
                text += line
    chunks = [text[i:i + 8000] for i in range(0, len(text), 8000)]      # below the compilers' limit on one literal
    with open(path, "w") as f:
        for c in chunks:
            assert ')jit"' not in c
            f.write('R"jit(' + c + ')jit"\n')


def _kernel_resources(src, out, table):
    """Moves the compiler's per-kernel resource remarks from `out` into `table`; returns the rest."""
    rest, name, after_remark = [], None, False
    for line in out.splitlines():
        if after_remark and re.match(r"\s+(\d+ )?\|", line):      # the source excerpt under a remark
            continue
        after_remark = "[-Rpass-analysis=kernel-resource-usage]" in line
        m = re.search(r"remark: (?:\s*)(Function Name|VGPRs|VGPRs Spill|SGPRs Spill|LDS Size \[bytes/block\]|Occupancy \[waves/SIMD\]|"
                      r"ScratchSize \[bytes/lane\]|AGPRs|SGPRs|Dynamic Stack|TotalSGPRs): (\S+)", line)
        if not m:
            if "-Rpass-analysis=kernel-resource-usage" not in line:
                rest.append(line)
            continue
        key, val = m.group(1), m.group(2)
        if key == "Function Name":
            name = "%s:%s" % (src, val)
            table[name] = {}
        elif name and key in ("VGPRs", "VGPRs Spill", "LDS Size [bytes/block]", "Occupancy [waves/SIMD]", "ScratchSize [bytes/lane]"):
            table[name][key] = int(val) if val.isdigit() else val
    return "\n".join(rest)


if __name__ == "__main__":
    print(build(verbose=True))
