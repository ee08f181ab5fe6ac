"""TEST INFRASTRUCTURE ONLY.  Times one sparse FFN block at the 7B layer shape (d 4096, ff 11008, predictor rank 1024, F16
weights, every neuron on the CPU) on the reference's own ggml.c (oracle/_ref/libpi_ref.so, built where /root/reference exists)
and on this repository's restatement (oracle/libpi_oracle.so), at 1 and 8 threads, and prints the ratio: how far the "port"
CPU baseline that bench.py reports is from the reference's real CPU kernels on the same machine.

    python oracle/calibrate_cpu.py
"""
import ctypes as C
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))
import oracle_lib as ol  # noqa: E402
from powerinfer_amd import synth  # noqa: E402


def main():
    d, ff, r = 4096, 11008, 1024
    Ly = synth.make_ffn_layer(seed=5, d=d, ff=ff, r=r, wtype=ol.F16, has_gate=True, T=1)
    gpu_idx = np.zeros(ff, np.int32)
    libs = [("restatement (pi_oracle.c)", ol.oracle())]
    if ol.ref() is not None:
        libs.insert(0, ("reference (ggml.c)", ol.ref()))
    res = {}
    for name, lib in libs:
        for nth in (1, 8):
            args = (lib, d, ff, r, 1, ol.F16, True, Ly["up"], Ly["gate"], Ly["down_t"], Ly["fc1"], Ly["fc2"], Ly["x"], Ly["x"], gpu_idx, 0.0, nth)
            if name.startswith("reference"):
                # the harness copies the weights into a fresh ggml context on every call: let it repeat the graph alone and time that
                lib.ref_set_repeat.argtypes = [C.c_int]
                lib.ref_last_compute_ms.restype = C.c_double
                lib.ref_set_repeat(200 if nth == 1 else 1000)
                o = ol.ffn_sparse(*args)
                lib.ref_set_repeat(1)
                ms = lib.ref_last_compute_ms()
            else:
                ol.ffn_sparse(*args)
                n, t0 = 0, time.perf_counter()
                while time.perf_counter() - t0 < 3.0:
                    o = ol.ffn_sparse(*args)
                    n += 1
                ms = (time.perf_counter() - t0) / n * 1e3
            res[(name, nth)] = ms
            print(f"{name:28s} threads {nth}: {ms:7.3f} ms per FFN block   active {int((o['logits'] >= 0).sum())} of {ff}", flush=True)
    if len(libs) == 2:
        for nth in (1, 8):
            print(f"threads {nth}: restatement / reference = {res[(libs[1][0], nth)] / res[(libs[0][0], nth)]:.2f}")


if __name__ == "__main__":
    main()
