"""Compiles the HIP sources into project-maya_amd/libmaya_moe.so for gfx950 (hipcc cross-compiles without a GPU)."""
import os
import subprocess
import sys

PKG = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(PKG, "csrc")
LIB = os.path.join(PKG, "libmaya_moe.so")
SOURCES = ["maya_kernels.hip", "maya_exl3.hip", "maya_prefill.hip"]
# -packed-fp32-ops off: the compiler then forms no v_pk_*_f32 from scalar float code.  amdgpu-kernarg-preload-count: the
# first 16 dwords of a kernel's arguments arrive in scalar registers with the dispatch instead of by a load (one memory
# round trip less at the start of every kernel: the decode layer 37.55 -> 37.15 us).
FLAGS = ["-O3", "-std=c++17", "--offload-arch=gfx950", "-fPIC", "-shared", "-ffp-contract=off",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-mllvm", "-amdgpu-kernarg-preload-count=16",
         "-Wall", "-Wno-unused-function"]


def _run(cmd, verbose):
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + " ".join(cmd) + "\n" + err)
    if verbose and err.strip():
        print(err, file=sys.stderr)


def build(verbose=False):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    _run([hipcc] + FLAGS + ["-o", LIB] + [os.path.join(CSRC, s) for s in SOURCES], verbose)
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
