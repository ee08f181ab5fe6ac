"""ctypes binding of libpowerinfer_hip.so (the C ABI declared in include/powerinfer_hip.h).

The library is loaded from this directory (built by `python -m powerinfer_amd.build`).  There is no CPU
fallback: without the shared object, or without a HIP device, everything here raises.
"""
import ctypes as C
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libpowerinfer_hip.so")

F32, F16, Q4_0, I32 = 0, 1, 2, 18
EPI_NONE, EPI_RELU, EPI_ADD, EPI_ADD2 = 0, 1, 2, 3
NORM_NONE, NORM_RMS, NORM_LAYER = 0, 1, 2

_vp, _i, _f, _sz, _u64 = C.c_void_p, C.c_int, C.c_float, C.c_size_t, C.c_uint64


class Norm(C.Structure):
    _fields_ = [("kind", C.c_int32), ("eps", C.c_float), ("w", C.c_void_p), ("b", C.c_void_p)]


class PiError(RuntimeError):
    pass


_lib = None
_inited = False

_SIGS = {
    "pi_init": (_i, [_i]),
    "pi_last_error": (C.c_char_p, []),
    "pi_device_name": (_i, [C.c_char_p, _sz]),
    "pi_malloc": (_vp, [_sz]),
    "pi_free": (_i, [_vp]),
    "pi_malloc_host": (_vp, [_sz]),
    "pi_free_host": (_i, [_vp]),
    "pi_memset": (_i, [_vp, _i, _sz]),
    "pi_memcpy_h2d": (_i, [_vp, _vp, _sz]),
    "pi_memcpy_d2h": (_i, [_vp, _vp, _sz]),
    "pi_memcpy_d2d": (_i, [_vp, _vp, _sz]),
    "pi_sync": (_i, []),
    "pi_fill_normal_f16": (_i, [_vp, _sz, _u64, _f, _vp, _i, _vp]),
    "pi_fill_normal_q4_0": (_i, [_vp, _sz, _u64, _f, _vp]),
    "pi_event_create": (_vp, []),
    "pi_event_record": (_i, [_vp, _vp]),
    "pi_event_elapsed_ms": (_i, [_vp, _vp, C.POINTER(_f)]),
    "pi_event_destroy": (_i, [_vp]),
    "pi_k_gemv": (_i, [_i, _vp, _i, _i, _vp, C.POINTER(Norm), _i, _vp, _vp, _vp, _vp]),
    "pi_k_gemv_multi_f16": (_i, [_vp, _vp, _i, _i, _vp, C.POINTER(Norm), _vp, _vp]),
    "pi_workspace_create": (_vp, [_i, _i]),
    "pi_workspace_destroy": (_i, [_vp]),
    "pi_k_predictor_fc2": (_i, [_vp, _i, _i, _vp, _f, _vp, _i, _vp, _vp, _vp, _vp, _vp, _vp]),
    "pi_k_compact_active": (_i, [_vp, _i, _f, _vp, _i, _vp, _vp, _vp, _vp]),
    "pi_k_sparse_upgate": (_i, [_i, _vp, _vp, _i, _i, _vp, C.POINTER(Norm), _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "pi_k_sparse_axpy": (_i, [_i, _vp, _i, _i, _vp, _vp, _vp, _vp, _vp, _i, _vp, _vp, _vp, _vp, _vp]),
    "pi_k_sparse_ffn_supported": (_i, [_i, _i, _i]),
    "pi_k_sparse_ffn_hot_supported": (_i, [_i, _i, _i]),
    "pi_k_sparse_ffn_workgroups": (_i, [_i, _i, _i]),
    "pi_k_sparse_ffn": (_i, [_vp, _i, _i, _vp, _f, _vp, _vp, _vp, _i, _vp, C.POINTER(Norm), _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "pi_k_sparse_ffn_noalloc_scratch_bytes": (_sz, []),
    "pi_k_sparse_ffn_noalloc_supported": (_i, [_i, _i, _i]),
    "pi_k_sparse_ffn_noalloc": (_i, [_vp, _i, _i, _vp, _f, _vp, _vp, _vp, _i, _vp, C.POINTER(Norm), _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "pi_k_pred_upgate_q4_supported": (_i, [_i, _i, _i]),
    "pi_k_pred_upgate_q4": (_i, [_vp, _i, _i, _vp, _f, _vp, _vp, _i, _vp, C.POINTER(Norm), _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "pi_k_axpy_q4_partials": (_i, [_vp, _i, _i, _vp, _vp, _vp, _vp, _vp]),
    "pi_k_pred_upgate_q4_split": (_i, [_vp, _i, _i, _vp, _f, _vp, _vp, _vp, _vp, _i, _vp, C.POINTER(Norm), _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "pi_k_axpy_q4_partials_split": (_i, [_vp, _vp, _i, _i, _vp, _vp, _vp, _vp, _vp]),
    "pi_k_axpy_q4_reduce": (_i, [_i, _i, _i, _vp, _vp, _vp, _vp, _vp, _vp]),
    "pi_k_k_shift": (_i, [_vp, _i, _i, _i, _i, _f, _f, _vp, _i, _vp]),
    "pi_k_k_shift_cells": (_i, [_vp, _i, _i, _i, _i, _i, _f, _f, _vp, _vp]),
    "pi_k_kv_compact": (_i, [_vp, _vp, _i, _i, _i, _vp, _i, _vp]),
    "pi_k_sparse_ffn_partials": (_i, [_vp, _i, _i, _vp, _f, _vp, _vp, _vp, _i, _vp, C.POINTER(Norm), _vp, _vp, _vp, _vp]),
    "pi_k_sparse_ffn_partials_hot": (_i, [_vp, _i, _i, _vp, _f, _vp, _vp, _vp, _i, _vp, C.POINTER(Norm), _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "pi_k_sparse_ffn_reduce_hot": (_i, [_i, _i, _i, _vp, _vp, _vp, _vp, _vp, _vp]),
    "pi_k_sparse_ffn_reduce": (_i, [_i, _i, _i, _vp, _vp, _vp, _vp, _vp, _vp]),
    "pi_k_pred_upgate_supported": (_i, [_i, _i, _i]),
    "pi_k_pred_upgate": (_i, [_vp, _i, _i, _vp, _f, _vp, _vp, _i, _vp, C.POINTER(Norm), _vp, _vp, _vp, _vp]),
    "pi_k_sparse_axpy_dense": (_i, [_vp, _i, _i, _vp, _vp, _i, _vp, _vp, _vp, _vp, _vp]),
    "pi_k_norm_round_f16": (_i, [_vp, _i, _i, C.POINTER(Norm), _vp, _vp, _vp]),
    "pi_k_gemm_f16": (_i, [_vp, _i, _i, _vp, _i, _i, _vp, _vp, _vp, _vp, _vp]),
    "pi_k_batch_predictor_fc2": (_i, [_vp, _i, _i, _vp, _i, _f, _vp, _vp, _vp]),
    "pi_k_batch_sparse_ffn": (_i, [_vp, _i, _i, _f, _vp, _vp, _vp, _i, _vp, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "pi_k_norm_round_f16_ol": (_i, [_vp, _i, _i, C.POINTER(Norm), _vp, _vp, _vp]),
    "pi_k_gemm_f16_ol": (_i, [_vp, _i, _i, _vp, _i, _i, _vp, _vp, _vp, _vp, _vp]),
    "pi_k_batch_predictor_fc2_ol": (_i, [_vp, _i, _i, _vp, _i, _f, _vp, _vp, _vp]),
    "pi_k_batch_sparse_ffn_ol": (_i, [_vp, _i, _i, _f, _vp, _vp, _vp, _i, _vp, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "pi_k_batch_union_count": (_i, [_i, _vp, _vp, _vp, _vp]),
    "pi_k_q4_split": (_i, [_vp, _i, _i, _vp, _vp, _vp]),
    "pi_k_norm_q8_blocks": (_i, [_vp, _i, _i, C.POINTER(Norm), _vp, _vp, _vp, _vp, _vp]),
    "pi_k_norm_q8_blocks_ol": (_i, [_vp, _i, _i, C.POINTER(Norm), _vp, _vp, _vp, _vp, _vp]),
    "pi_k_gemm_q4_t16": (_i, [_vp, _vp, _i, _i, _vp, _vp, _vp, _i, _i, _vp, _vp, _vp, _vp]),
    "pi_k_batch_sparse_ffn_q4": (_i, [_vp, _i, _i, _f, _vp, _vp, _vp, _vp, _vp, _vp, _i, _vp, _vp, _vp, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "pi_k_gemm_tile_f16": (_i, [_vp, _i, _i, _vp, _i, _i, _vp, _vp, _vp, _vp, _i, _vp]),
    "pi_k_ffn_h_f16": (_i, [_vp, _vp, _vp, _f, _i, _i, _vp, _vp]),
    "pi_k_transpose_f16": (_i, [_vp, _i, _i, _vp, _vp]),
    "pi_k_norm_q8_round_f16": (_i, [_vp, _i, _i, C.POINTER(Norm), _vp, _vp, _vp]),
    "pi_k_ffn_h_q8_f16": (_i, [_vp, _vp, _vp, _f, _i, _i, _vp, _vp]),
    "pi_k_dequant_q4_f16": (_i, [_vp, _vp, _vp, _vp, _i, _i, _vp, _vp]),
    "pi_k_assemble_rows_f16": (_i, [_vp, _vp, _vp, _vp, _i, _i, _vp, _vp]),
    "pi_k_embed_batch_q4": (_i, [_vp, _i, _vp, _i, _vp, _vp]),
    "pi_k_host_signal": (_i, [_vp, _vp, _i, _i, _vp]),
    "pi_k_sparse_ffn_two_phase_supported": (_i, [_i, _i, _i]),
    "pi_k_sparse_ffn_logits_hot": (_i, [_vp, _i, _i, _vp, _f, _i, _vp, C.POINTER(Norm), _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "pi_k_sparse_ffn_rows_hot": (_i, [_i, _f, _vp, _vp, _vp, _i, _vp, C.POINTER(Norm), _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "pi_k_sparse_ffn_q4_partials": (_i, [_vp, _i, _i, _vp, _f, _vp, _vp, _vp, _vp, _vp, _vp, _i, _vp, C.POINTER(Norm), _vp, _vp, _vp, _vp, _vp, _vp]),
    "pi_k_sparse_ffn_q4_reduce": (_i, [_i, _i, _i, _vp, _vp, _vp, _vp, _vp, _vp]),
    "pi_k_pred_q4_logits": (_i, [_vp, _i, _i, _vp, _f, _i, _vp, C.POINTER(Norm), _vp, _vp, _vp, _vp, _vp, _vp]),
    "pi_k_upgate_q4_hot_rows": (_i, [_i, _f, _vp, _vp, _i, _vp, C.POINTER(Norm), _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "pi_k_host_wait": (_i, [_vp, _vp, _i, _vp, C.c_double, _vp]),
    "pi_k_host_signal_wait": (_i, [_vp, _vp, _i, _i, _vp, C.c_double, _vp]),
    "pi_ggml_backend_get_stats": (None, [_vp]),
    "pi_ggml_backend_set_fusion": (None, [_i]),
    "pi_gemm_lib_create": (_vp, [C.c_size_t]),
    "pi_gemm_lib_destroy": (_i, [_vp]),
    "pi_gemm_lib_f16": (_i, [_vp, _vp, _i, _i, _vp, _i, _i, _vp, _vp, _vp, _vp, _vp]),
    "pi_k_batch_sparse_mul_mat": (_i, [_vp, _i, _i, _vp, _i, _vp, _f, _vp, _vp, _vp, _vp, _vp]),
    "pi_k_batch_sparse_axpy": (_i, [_vp, _i, _i, _vp, _vp, _i, _f, _vp, _vp, _vp, _vp, _vp]),
    "pi_k_attn_split_supported": (_i, [_i, _i, _i]),
    "pi_k_attn_ggml_supported": (_i, [_i, _i, _i]),
    "pi_k_attn_ggml": (_i, [_vp, _vp, _vp, _vp, _i, _f, _f, _f, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp, _vp, _vp, _vp]),
    "pi_k_attn_ggml_step": (_i, [_vp, _i, _vp, _i, _f, _f, _f, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _vp, _vp, _i, _vp, _i, _vp]),
    "pi_k_attn_split_scratch_floats": (_sz, [_i, _i, _i, _i]),
    "pi_k_attn_split": (_i, [_vp, _i, _vp, _vp, _vp, _sz, _i, _i, _i, _i, _i, _i, _i, _vp, _vp, _vp, _i, _vp, _vp]),
    "pi_k_attn_chunk_supported": (_i, [_i, _i, _i]),
    "pi_k_attn_chunk_long": (_i, [_vp, _i, _i, _i, _i, _i, _i, _f, _f, _vp, _i, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "pi_k_attn_split_cached": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _vp, _vp, _vp, _vp]),
    "pi_k_attn_fused_batch": (_i, [_vp, _i, _vp, _vp, _vp, _sz, _i, _i, _i, _i, _i, _i, _vp, _vp, _i, _vp, _vp]),
    "pi_k_attn_fused_batch_ol": (_i, [_vp, _i, _vp, _vp, _vp, _sz, _i, _i, _i, _i, _i, _i, _vp, _vp, _i, _vp, _vp]),
    "pi_k_attn_fused_batch_q8": (_i, [_vp, _i, _vp, _vp, _vp, _sz, _i, _i, _i, _i, _i, _i, _vp, _vp, _i, _vp, _vp, _vp, _vp]),
    "pi_k_attn_chunk": (_i, [_vp, _i, _i, _i, _i, _i, _i, _f, _f, _vp, _i, _i, _vp, _vp, _vp, _vp, _i, _vp, _vp]),
    "pi_k_embed_batch": (_i, [_vp, _i, _vp, _i, _vp, _vp]),
    "pi_k_argmax_batch": (_i, [_vp, _i, _i, _vp, _vp, _vp, _vp, _i, _vp]),
    "pi_k_step_advance": (_i, [_vp, _vp]),
    "pi_k_rope_kv_store": (_i, [_vp, _i, _i, _i, _i, _f, _f, _vp, _i, _vp, _vp, _vp, _vp]),
    "pi_k_attn_decode": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _vp, _vp, _vp]),
    "pi_k_rope_table": (_i, [_vp, _i, _i, _i, _f, _f, _vp]),
    "pi_k_attn_fused_supported": (_i, [_i, _i]),
    "pi_k_attn_decode_supported": (_i, [_i, _i]),
    "pi_k_attn_fused": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp, _vp, _vp]),
    "pi_k_embed": (_i, [_i, _vp, _i, _vp, _vp, _vp]),
    "pi_k_argmax": (_i, [_vp, _i, _vp, _vp]),
}


def load():
    """dlopen the library and declare signatures (no device call)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise PiError(f"{LIB_PATH} is missing: run `python -m powerinfer_amd.build` (no CPU fallback exists)")
        L = C.CDLL(LIB_PATH)
        for name, (res, args) in _SIGS.items():
            fn = getattr(L, name)
            fn.restype, fn.argtypes = res, args
        _lib = L
    return _lib


def declared_symbols():
    from .model import ENGINE_SYMBOLS
    return sorted(list(_SIGS) + ENGINE_SYMBOLS)


def check(rc, what=""):
    if rc != 0:
        raise PiError(f"{what} failed ({rc}): {load().pi_last_error().decode()}")


def init(device=0):
    global _inited
    L = load()
    if not _inited:
        check(L.pi_init(device), "pi_init")
        _inited = True
    return L


def device_name():
    buf = C.create_string_buffer(256)
    check(init().pi_device_name(buf, 256), "pi_device_name")
    return buf.value.decode()


class DevBuf:
    """A device allocation with numpy upload/download helpers."""

    def __init__(self, nbytes=None, host=None):
        L = init()
        if host is not None:
            host = np.ascontiguousarray(host)
            nbytes = host.nbytes
        self.nbytes = int(nbytes)
        self.ptr = L.pi_malloc(max(self.nbytes, 1))
        if not self.ptr:
            raise PiError("pi_malloc: " + L.pi_last_error().decode())
        if host is not None and self.nbytes:
            check(L.pi_memcpy_h2d(self.ptr, host.ctypes.data_as(_vp), self.nbytes), "h2d")

    @classmethod
    def zeros(cls, nbytes):
        b = cls(nbytes)
        check(load().pi_memset(b.ptr, 0, b.nbytes), "memset")
        return b

    def upload(self, host, offset=0):
        host = np.ascontiguousarray(host)
        assert offset + host.nbytes <= self.nbytes
        check(load().pi_memcpy_h2d(self.ptr + offset, host.ctypes.data_as(_vp), host.nbytes), "h2d")

    def download(self, dtype, count=None, offset=0):
        dt = np.dtype(dtype)
        count = (self.nbytes - offset) // dt.itemsize if count is None else count
        out = np.empty(count, dt)
        if count:
            check(load().pi_memcpy_d2h(out.ctypes.data_as(_vp), self.ptr + offset, out.nbytes), "d2h")
        return out

    def free(self):
        if self.ptr:
            load().pi_free(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def norm_arg(kind=NORM_NONE, eps=0.0, w=None, b=None):
    if kind == NORM_NONE:
        return None
    return C.byref(Norm(kind, eps, w.ptr if w is not None else None, b.ptr if b is not None else None))


def sync():
    check(init().pi_sync(), "pi_sync")
