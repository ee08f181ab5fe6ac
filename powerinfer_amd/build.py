"""Builds libpowerinfer_hip.so in-tree with hipcc for gfx950 (cross-compiles without a GPU).

    python -m powerinfer_amd.build
"""
import glob
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libpowerinfer_hip.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "-O3", "--offload-arch=gfx950", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden", "-pthread",
    # packed-FP32 instructions are not to be generated on this hardware pool
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # a product and a sum fuse into one FMA only where the source writes them as one expression: hipcc's default ("fast") also
    # fuses across statements and through __fmul_rn / __fadd_rn (plain * and + in the HIP headers), which moves results by one
    # unit in the last place where the CPU path rounds twice (norm weight then bias, the RoPE rotation)
    "-ffp-contract=on",
    "-Wno-unused-command-line-argument",
    # host code of the cold path uses the x86 vector extensions every MI355X host CPU has
    "-Xarch_host", "-mavx2", "-Xarch_host", "-mfma", "-Xarch_host", "-mf16c",
]
# dense mat-muls of long prompt chunks go to the library the reference's cuBLAS calls correspond to
LIBS = ["-L/opt/rocm/lib", "-lhipblaslt", "-Wl,-rpath,/opt/rocm/lib"]


def sources():
    return sorted(glob.glob(os.path.join(CSRC, "*.hip")) + glob.glob(os.path.join(CSRC, "*.cpp")))


def build(verbose=True):
    cmd = [HIPCC] + FLAGS + ["-o", LIB] + sources() + LIBS
    if verbose:
        print(" ".join(cmd), flush=True)
    p = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in p.stderr.splitlines() if "is not a recognized feature for this target" not in l)
    if p.returncode != 0:
        sys.stderr.write(err + "\n")
        raise RuntimeError("hipcc failed")
    if verbose and err.strip():
        print(err)
    return LIB


if __name__ == "__main__":
    build()
