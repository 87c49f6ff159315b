"""Builds libllama_cu_amd.so (HIP kernels + C ABI + C++ host layer) for gfx950 with hipcc."""
import os
import subprocess
import sys

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
LIB = os.path.join(PKG, "libllama_cu_amd.so")
# diagnostic build: the same library with the phase timelines of the fused decode launch and of the
# W2 + norm launch compiled in (csrc/attention.hip, csrc/gemv.hip, -DLCU_PHASE_TIMELINE), read by timeline.py
TIMELINE_LIB = os.path.join(PKG, "libllama_cu_amd_timeline.so")

HIP_SOURCES = ["csrc/runtime.hip", "csrc/elementwise.hip", "csrc/gemv.hip", "csrc/gemm.hip", "csrc/attention.hip"]
HOST_SOURCES = ["host/buffers.cpp", "host/params.cpp", "host/model.cpp", "host/batch.cpp", "host/tokenizer.cpp", "host/capi.cpp"]
# command line programs linked against the library (found at run time next to bin/ through $ORIGIN)
APPS = {"transform": "apps/transform.cpp", "llama_cu": "apps/llama_cu.cpp"}
BIN = os.path.join(PKG, "bin")

COMMON = ["-O3", "-std=c++17", "-fPIC", "-I" + os.path.join(ROOT, "include"), "-I" + os.path.join(PKG, "csrc"),
          "-I" + os.path.join(PKG, "host"), "-Wall", "-Wno-unused-function"]
# no fast-math, no implicit fma contraction (the kernels write their fused multiply-adds out), and
# no packed-fp32 instructions
DEVICE = ["--offload-arch=gfx950", "-ffp-contract=off", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def build(verbose=False):
    objs = []
    os.makedirs(os.path.join(PKG, "build"), exist_ok=True)
    procs = []
    for src in HIP_SOURCES + HOST_SOURCES:
        obj = os.path.join(PKG, "build", os.path.basename(src) + ".o")
        objs.append(obj)
        cmd = ["hipcc"] + COMMON + (DEVICE if src.endswith(".hip") else ["-x", "c++"]) + ["-c", os.path.join(PKG, src), "-o", obj]
        if verbose:
            print(" ".join(cmd))
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
    failed = False
    for src, p in procs:
        out, _ = p.communicate()
        out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l and "unknown target feature" not in l)
        if p.returncode != 0:
            failed = True
            sys.stderr.write("FAILED %s\n%s\n" % (src, out))
        elif verbose and out.strip():
            print(out)
    if failed:
        raise RuntimeError("hipcc failed")
    cmd = ["hipcc", "--offload-arch=gfx950", "-shared", "-o", LIB] + objs
    subprocess.check_call(cmd)
    os.makedirs(BIN, exist_ok=True)
    for name, src in APPS.items():
        cmd = ["hipcc"] + COMMON + ["-x", "c++", os.path.join(PKG, src), "-o", os.path.join(BIN, name),
               "-L" + PKG, "-lllama_cu_amd", "-Wl,-rpath,$ORIGIN/.."]
        if verbose:
            print(" ".join(cmd))
        subprocess.check_call(cmd)
    return LIB


def build_timeline():
    """libllama_cu_amd_timeline.so: attention.hip and gemv.hip recompiled with -DLCU_PHASE_TIMELINE, every
    other object taken from the last ordinary build (build() first)."""
    instrumented = {}
    for name in ("attention.hip", "gemv.hip"):
        obj = os.path.join(PKG, "build", name + ".timeline.o")
        subprocess.check_call(["hipcc"] + COMMON + DEVICE + ["-DLCU_PHASE_TIMELINE", "-c", os.path.join(PKG, "csrc", name),
                               "-o", obj], stderr=subprocess.DEVNULL)
        instrumented[name] = obj
    objs = [instrumented.get(os.path.basename(src), os.path.join(PKG, "build", os.path.basename(src) + ".o"))
            for src in HIP_SOURCES + HOST_SOURCES]
    subprocess.check_call(["hipcc", "--offload-arch=gfx950", "-shared", "-o", TIMELINE_LIB] + objs)
    return TIMELINE_LIB


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
    if "--timeline" in sys.argv:
        print(build_timeline())
