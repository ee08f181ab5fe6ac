"""Writes tests/golden/ggml_abi.json: field offsets, sizes and enumerator values of the reference's ggml.h ABI
(the part its accelerator backend reads), obtained by compiling a probe against /root/reference/ggml.h.
Only runs where the reference tree exists; the JSON it writes is committed.

    python tests/golden/make_abi_fixture.py
"""
import json
import os
import subprocess
import tempfile

HERE = os.path.dirname(os.path.abspath(__file__))

PROBE = r'''
#include <stdio.h>
#include <stddef.h>
#include "%(header)s"
#define OFF(f) printf("\"off_" #f "\": %%zu,\n", offsetof(struct ggml_tensor, f))
#define VAL(v) printf("\"" #v "\": %%d,\n", (int)(v))
int main(void) {
    printf("{\n");
    OFF(type); OFF(backend); OFF(buffer); OFF(n_dims); OFF(ne); OFF(nb); OFF(op); OFF(op_params); OFF(is_param); OFF(grad);
    OFF(src); OFF(is_finish); OFF(perf_runs); OFF(view_src); OFF(view_offs); OFF(data); OFF(name); OFF(extra);
    printf("\"sizeof_tensor\": %%zu,\n", sizeof(struct ggml_tensor));
    printf("\"sizeof_params\": %%zu,\n", sizeof(struct ggml_compute_params));
    printf("\"off_params_wdata\": %%zu,\n", offsetof(struct ggml_compute_params, wdata));
    printf("\"off_params_aic\": %%zu,\n", offsetof(struct ggml_compute_params, aic));
    VAL(GGML_TYPE_F32); VAL(GGML_TYPE_F16); VAL(GGML_TYPE_Q4_0); VAL(GGML_TYPE_Q8_0); VAL(GGML_TYPE_I32);
    VAL(GGML_BACKEND_CPU); VAL(GGML_BACKEND_GPU); VAL(GGML_BACKEND_GPU_SPLIT);
    VAL(GGML_OP_DUP); VAL(GGML_OP_ADD); VAL(GGML_OP_MUL); VAL(GGML_OP_NORM); VAL(GGML_OP_RMS_NORM);
    VAL(GGML_OP_MUL_MAT); VAL(GGML_OP_MUL_MAT_SPARSE); VAL(GGML_OP_AXPY); VAL(GGML_OP_SCALE); VAL(GGML_OP_CPY); VAL(GGML_OP_CONT);
    VAL(GGML_OP_RESHAPE); VAL(GGML_OP_VIEW); VAL(GGML_OP_PERMUTE); VAL(GGML_OP_TRANSPOSE); VAL(GGML_OP_GET_ROWS);
    VAL(GGML_OP_SOFT_MAX); VAL(GGML_OP_ROPE); VAL(GGML_OP_UNARY); VAL(GGML_UNARY_OP_RELU);
    VAL(GGML_TASK_INIT); VAL(GGML_TASK_COMPUTE); VAL(GGML_TASK_FINALIZE);
    VAL(GGML_MAX_DIMS); VAL(GGML_MAX_SRC); VAL(GGML_MAX_NAME); VAL(GGML_MAX_OP_PARAMS);
    printf("\"end\": 0\n}\n");
    return 0;
}
'''


def probe(header, include_dir):
    with tempfile.TemporaryDirectory() as td:
        src = os.path.join(td, "probe.c")
        with open(src, "w") as f:
            f.write(PROBE % {"header": header})
        exe = os.path.join(td, "probe")
        subprocess.check_call(["gcc", "-std=c11", "-D_GNU_SOURCE", "-I", include_dir, "-o", exe, src])
        return json.loads(subprocess.check_output([exe]).decode())


if __name__ == "__main__":
    ref = probe("ggml.h", "/root/reference")
    with open(os.path.join(HERE, "ggml_abi.json"), "w") as f:
        json.dump(ref, f, indent=1, sort_keys=True)
    print("wrote", len(ref), "entries")
