"""Builds sage_amd/libsage_hip.so (the C-ABI library declared in include/sage_hip.h) for gfx950."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libsage_hip.so")
SOURCES = ["runtime.cpp", "pool.cpp", "map_jit.cpp", "reduce.hip", "index.hip", "gemm.hip", "attention.hip", "rand.hip", "optim.hip"]
# -packed-fp32-ops is switched off: hipcc would otherwise form v_pk_*_f32 from plain float code.
FLAGS = ["-O3", "-std=c++17", "-fPIC", "--offload-arch=gfx950", "-Wall", "-Wno-unused-function",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


# Per-source additions.  attention.hip: accumulators in ordinary vector registers; the compiler's default put
# the output accumulators into the accumulation file and copied them out and back for every rescaling.
# optim.hip: the fused optimizer step must round like the generated map kernels it stands for (no contraction).
EXTRA = {"attention.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form=1"], "optim.hip": ["-ffp-contract=off"]}


def build(verbose=True):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    objs = []
    procs = []
    for src in SOURCES:
        obj = os.path.join(CSRC, os.path.splitext(src)[0] + ".o")
        cmd = [hipcc, *FLAGS, *EXTRA.get(src, []), "-x", "hip", "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        objs.append(obj)
    failed = False
    for src, p in procs:
        out, _ = p.communicate()
        out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l)
        if out.strip() and verbose:
            print(out)
        if p.returncode:
            print(f"compiling {src} failed", file=sys.stderr)
            failed = True
    if failed:
        raise RuntimeError("hipcc failed")
    cmd = [hipcc, "-shared", "-fPIC", "--offload-arch=gfx950", *objs, "-o", LIB, "-lhiprtc"]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return LIB


if __name__ == "__main__":
    build()
