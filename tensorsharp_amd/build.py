"""Build libTsHipOps.so (gfx950 only) with hipcc, in-tree next to this file."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libTsHipOps.so")
SOURCES = ["abi.hip", "dequant.hip", "gemv.hip", "gemm.hip", "moe.hip", "fused.hip", "layer.hip"]

# packed-fp32 VALU forms stay off: the compiler must not form v_pk_{add,mul,fma}_f32.
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
    # the leading scalar arguments of every kernel (up to 14 dwords) arrive preloaded in SGPRs at wave launch; the code
    # objects keep a loading prologue for firmware without the feature
    "-mllvm", "-amdgpu-kernarg-preload-count=14",
]
# per-source additions
EXTRA_FLAGS = {}


def build(verbose=False, jobs=8):
    """Compile every source and link the shared library."""
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    lib = LIB
    objdir = os.path.join(HERE, "build", os.path.basename(lib))
    os.makedirs(objdir, exist_ok=True)
    procs = []
    objs = []
    for src in SOURCES:
        obj = os.path.join(objdir, src + ".o")
        objs.append(obj)
        cmd = [hipcc] + FLAGS + EXTRA_FLAGS.get(src, []) + ["-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        if len(procs) >= jobs:
            _drain(procs)
    _drain(procs)
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", lib] + objs
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    return lib


def _drain(procs):
    failed = []
    for src, p in procs:
        out, _ = p.communicate()
        # hipcc's host pass does not know the packed-fp32 feature name; that warning is harmless
        out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l)
        if out.strip():
            print(out)
        if p.returncode != 0:
            failed.append(src)
    procs.clear()
    if failed:
        raise RuntimeError("hipcc failed for: " + ", ".join(failed))


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
