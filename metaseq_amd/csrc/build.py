"""Builds libmetaseq_amd.so for gfx950 with hipcc (no GPU needed: hipcc cross-compiles).

Usage: python -m metaseq_amd.csrc.build [--force]
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "libmetaseq_amd.so")
SOURCES = ["capi.hip", "layernorm.hip", "embed.hip", "gemm.hip", "attention.hip", "attention_prefill.hip",
           "sampling.hip", "probe.hip", "decoder_step.hip"]
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17", "-Wall", "-Wno-unused-function",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


# per-source extras.  The prefill attention kernel keeps its MFMA results in ordinary vector
# registers (its softmax reads every score; by default hipcc parks them in the accumulator bank
# and copies each one out)
EXTRA_FLAGS = {"attention_prefill.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form=1"]}


def _hipcc():
    for c in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if c and (os.path.sep not in c or os.path.exists(c)):
            return c
    raise RuntimeError("hipcc not found")


def needs_build():
    if not os.path.exists(LIB):
        return True
    t = os.path.getmtime(LIB)
    deps = SOURCES + ["common.h", os.path.join("..", "..", "include", "metaseq_amd.h")]
    return any(os.path.getmtime(os.path.join(HERE, d)) > t for d in deps)


def build(force=True, verbose=True):
    """Compiles every kernel source and links the shared library in-tree."""
    if not force and not needs_build():
        return LIB
    hipcc = _hipcc()
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)

    def compile_one(src):
        obj = os.path.join(objdir, src.replace(".hip", ".o"))
        cmd = [hipcc] + FLAGS + EXTRA_FLAGS.get(src, []) + ["-c", os.path.join(HERE, src), "-o", obj]
        r = subprocess.run(cmd, capture_output=True, text=True)
        err = "\n".join(l for l in r.stderr.splitlines()
                        if "packed-fp32-ops" not in l)  # host pass does not know the feature
        if r.returncode != 0:
            raise RuntimeError("hipcc failed for %s:\n%s" % (src, err))
        if verbose and err.strip():
            print(err, file=sys.stderr)
        return obj

    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as ex:
        objs = list(ex.map(compile_one, SOURCES))
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stderr)
    if verbose:
        print("built", LIB)
    return LIB


if __name__ == "__main__":
    build(force=True)
