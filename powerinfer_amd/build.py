"""Builds libpowerinfer_hip.so in-tree with hipcc for gfx950 (cross-compiles without a GPU).

    python -m powerinfer_amd.build            # recompiles the sources that changed (objects under csrc/.obj), then links
    python -m powerinfer_amd.build --force    # recompiles everything
"""
import concurrent.futures
import glob
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(CSRC, ".obj")
LIB = os.path.join(HERE, "libpowerinfer_hip.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "-O3", "--offload-arch=gfx950", "-std=c++17", "-fPIC", "-fvisibility=hidden", "-pthread",
    # packed-FP32 instructions are not to be generated on this hardware pool
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # a product and a sum fuse into one FMA only where the source writes them as one expression: hipcc's default ("fast") also
    # fuses across statements and through __fmul_rn / __fadd_rn (plain * and + in the HIP headers), which moves results by one
    # unit in the last place where the CPU path rounds twice (norm weight then bias, the RoPE rotation)
    "-ffp-contract=on",
    "-Wno-unused-command-line-argument",
    # the helpers of kernels_common.hpp sit in an unnamed namespace; a kernel file uses the ones it needs
    "-Wno-unused-function",
    # host code of the cold path uses the x86 vector extensions every MI355X host CPU has
    "-Xarch_host", "-mavx2", "-Xarch_host", "-mfma", "-Xarch_host", "-mf16c",
]
# dense mat-muls of long prompt chunks go to the library the reference's cuBLAS calls correspond to
LIBS = ["-L/opt/rocm/lib", "-lhipblaslt", "-Wl,-rpath,/opt/rocm/lib"]


def sources():
    return sorted(glob.glob(os.path.join(CSRC, "*.hip")) + glob.glob(os.path.join(CSRC, "*.cpp")))


def _headers_mtime():
    hs = glob.glob(os.path.join(CSRC, "*.hpp")) + glob.glob(os.path.join(HERE, "..", "include", "*.h"))
    return max(os.path.getmtime(h) for h in hs)


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    p = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in p.stderr.splitlines() if "is not a recognized feature for this target" not in l)
    return p.returncode, err


def build(verbose=True, force=False, jobs=None):
    """One object per source (a change to one kernel file recompiles that file), compiled side by side, then one link."""
    os.makedirs(OBJ, exist_ok=True)
    newest_header = _headers_mtime()
    todo, objs = [], []
    for src in sources():
        obj = os.path.join(OBJ, os.path.basename(src) + ".o")
        objs.append(obj)
        if force or not os.path.exists(obj) or os.path.getmtime(obj) < max(os.path.getmtime(src), newest_header):
            todo.append((src, obj))
    jobs = jobs or min(8, os.cpu_count() or 1)
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as ex:
        results = list(ex.map(lambda so: (so[0],) + _run([HIPCC] + FLAGS + ["-c", so[0], "-o", so[1]], verbose), todo))
    failed = False
    for src, rc, err in results:
        if rc != 0:
            sys.stderr.write("%s:\n%s\n" % (src, err))
            if os.path.exists(os.path.join(OBJ, os.path.basename(src) + ".o")):
                os.remove(os.path.join(OBJ, os.path.basename(src) + ".o"))
            failed = True
        elif verbose and err.strip():
            print(err)
    if failed:
        raise RuntimeError("hipcc failed")
    rc, err = _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-pthread", "-o", LIB] + objs + LIBS, verbose)
    if rc != 0:
        sys.stderr.write(err + "\n")
        raise RuntimeError("link failed")
    return LIB


if __name__ == "__main__":
    build(force="--force" in sys.argv[1:])
