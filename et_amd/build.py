"""Builds libet_amd.so (HIP kernels + C ABI) for gfx950 with hipcc, in-tree."""
from __future__ import annotations

import os
import shutil
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libet_amd.so")

SOURCES = ["runtime.hip", "formats.cpp", "skip_layernorm.hip", "tile_linear.hip", "tile_tail.hip", "dense_gemm.hip", "attention.hip",
           "encoder_capi.cpp"]

# packed fp32 ops stay off: some of their forms have produced wrong results on
# this hardware pool
HIP_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
             # keep MFMA accumulators in VGPRs: the softmax / epilogue VALU work
             # reads them directly instead of copying from AGPRs
             "-mllvm", "-amdgpu-mfma-vgpr-form=1"]


def hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found")
    return exe


def build(verbose: bool = False) -> str:
    objs = []
    procs = []
    for src in SOURCES:
        path = os.path.join(CSRC, src)
        if not os.path.exists(path):
            continue
        obj = os.path.join(CSRC, os.path.splitext(src)[0] + ".o")
        cmd = [hipcc(), "-x", "hip", "-c", path, "-o", obj, "-I", os.path.join(HERE, "..", "include"),
               "-I", HERE] + HIP_FLAGS + os.environ.get("ET_AMD_EXTRA_HIPFLAGS", "").split()
        if verbose:
            print(" ".join(cmd))
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        objs.append(obj)
    failed = []
    for src, p in procs:
        out, _ = p.communicate()
        out = "\n".join(l for l in out.splitlines() if "is not a recognized feature" not in l)
        if p.returncode != 0:
            failed.append((src, out))
        elif verbose and out.strip():
            print(out)
    if failed:
        raise RuntimeError("\n".join(f"--- {s} ---\n{o}" for s, o in failed))
    cmd = [hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs
    subprocess.check_call(cmd)
    build_examples(verbose)
    build_microbench(verbose)
    return LIB


MICROBENCH_LIB = os.path.join(HERE, "bench", "libet_microbench.so")


def build_microbench(verbose: bool = False) -> str:
    """The delivery-path microbenchmarks of bench.py --micro: a library of their own (they are a measuring tool,
    not part of the encoder's C ABI), linked against libet_amd.so for its error plumbing."""
    src = os.path.join(HERE, "bench", "microbench.hip")
    cmd = [hipcc(), "-x", "hip", src, "-shared", "-o", MICROBENCH_LIB, "-I", os.path.join(HERE, "..", "include"),
           "-I", HERE] + HIP_FLAGS + ["-L", HERE, "-let_amd", "-Wl,-rpath,$ORIGIN/.."]
    if verbose:
        print(" ".join(cmd))
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in p.stdout.splitlines() if "is not a recognized feature" not in l)
    if p.returncode != 0:
        raise RuntimeError(out)
    if verbose and out.strip():
        print(out)
    return MICROBENCH_LIB


def build_examples(verbose: bool = False) -> str:
    """The C++ callers of et_amd/examples (the reference's three test programs on this library): host C++
    only, compiled with the ROCm clang++ (half is _Float16) and linked against the library above."""
    cxx = os.path.join(os.path.dirname(os.path.realpath(hipcc())), "..", "lib", "llvm", "bin", "clang++")
    if not os.path.exists(cxx):
        cxx = "/opt/rocm/lib/llvm/bin/clang++"
    exe = ""
    for name in ("tile_test", "prune_test", "length_test"):
        src = os.path.join(HERE, "examples", name + ".cpp")
        exe = os.path.join(HERE, "examples", name)
        cmd = [cxx, "-std=c++17", "-O2", "-Wall", "-o", exe, src, "-L", HERE, "-let_amd", "-Wl,-rpath,$ORIGIN/.."]
        if verbose:
            print(" ".join(cmd))
        subprocess.check_call(cmd)
    return os.path.dirname(exe)


if __name__ == "__main__":
    print(build(verbose=True))
