"""Test-side stand-in for the reference's host: ggml tensors as ctypes structs laid out per
include/ggml_backend_abi.h, the op constructors llm_build_ffn_sparse uses (ggml.c:4100-4190 and friends), and an
executor that walks the nodes the way ggml_graph_compute does: every node is offered to
ggml_cuda_compute_forward first and computed by the CPU oracle only when the backend answers "not mine"
(ggml.c:14791-14798)."""
import ctypes as C

import numpy as np

import oracle_lib as ol
from oracle_lib import _ptr as P

F32, F16, Q4_0, I32 = 0, 1, 2, 18
CPU, GPU = 0, 10
OP = dict(NONE=0, DUP=1, ADD=2, MUL=6, NORM=19, RMS_NORM=20, MUL_MAT=23, MUL_MAT_SPARSE=24, AXPY=25, SCALE=27, CPY=29, CONT=30,
          RESHAPE=31, VIEW=32, PERMUTE=33, TRANSPOSE=34, GET_ROWS=35, SOFT_MAX=40, ROPE=42, UNARY=59)
UNARY_RELU = 6


class Tensor(C.Structure):
    pass


Tensor._fields_ = [
    ("type", C.c_int), ("backend", C.c_int), ("buffer", C.c_void_p), ("n_dims", C.c_int),
    ("ne", C.c_int64 * 4), ("nb", C.c_size_t * 4), ("op", C.c_int), ("op_params", C.c_int32 * 16),
    ("is_param", C.c_bool), ("grad", C.c_void_p), ("src", C.POINTER(Tensor) * 6),
    ("is_finish", C.c_int), ("perf_runs", C.c_int), ("perf_cycles", C.c_int64), ("perf_time_us", C.c_int64),
    ("view_src", C.POINTER(Tensor)), ("view_offs", C.c_size_t), ("data", C.c_void_p), ("name", C.c_char * 64),
    ("extra", C.c_void_p), ("padding", C.c_char * 12),
]


class Params(C.Structure):
    _fields_ = [("type", C.c_int), ("ith", C.c_int), ("nth", C.c_int), ("wsize", C.c_size_t), ("wdata", C.c_void_p), ("aic", C.c_void_p)]


def _tsize(t):
    return {F32: 4, I32: 4, F16: 2, Q4_0: 18}[t]


def _blck(t):
    return 32 if t == Q4_0 else 1


class Graph:
    def __init__(self, lib):
        self.L = lib
        lib.ggml_cuda_compute_forward.restype = C.c_bool
        lib.ggml_cuda_compute_forward.argtypes = [C.POINTER(Params), C.POINTER(Tensor)]
        for n in ("ggml_cuda_transform_tensor",):
            getattr(lib, n).argtypes = [C.c_void_p, C.POINTER(Tensor)]
        for n in ("ggml_cuda_assign_buffers", "ggml_cuda_assign_buffers_no_scratch", "ggml_cuda_copy_to_host", "ggml_cuda_copy_to_device",
                  "ggml_cuda_free_data", "ggml_cuda_alloc_tensor"):
            getattr(lib, n).argtypes = [C.POINTER(Tensor)]
        lib.ggml_cuda_set_device_constants.argtypes = [C.c_float]
        lib.ggml_cublas_loaded.restype = C.c_bool
        lib.ggml_init_cublas()
        assert lib.ggml_cublas_loaded()
        self.nodes, self.keep, self.gpu_run, self.cpu_run = [], [], [], []

    # ---- tensors -------------------------------------------------------------------------------------
    def new(self, type_, ne, host=None, name=""):
        t = Tensor()
        t.type, t.backend, t.n_dims = type_, CPU, len(ne)
        ne = list(ne) + [1] * (4 - len(ne))
        for i in range(4):
            t.ne[i] = ne[i]
        t.nb[0] = _tsize(type_)
        t.nb[1] = t.nb[0] * (ne[0] // _blck(type_))
        t.nb[2] = t.nb[1] * ne[1]
        t.nb[3] = t.nb[2] * ne[2]
        t.name = name.encode()[:63]
        nbytes = t.nb[3] * ne[3]
        if host is None:
            host = np.zeros(nbytes, np.uint8)
        host = np.ascontiguousarray(host)
        assert host.nbytes == nbytes, (name, host.nbytes, nbytes)
        t.data = host.ctypes.data
        self.keep.append(host)
        t._host = host
        return t

    def weight_to_gpu(self, t):
        """ggml_cuda_transform_tensor: the tensor becomes GPU-resident (llama.cpp:2192)."""
        t.backend = GPU
        self.L.ggml_cuda_transform_tensor(t.data, C.byref(t))
        return t

    def _node(self, op, type_, ne, srcs, name, params=()):
        t = self.new(type_, ne, name=name)
        t.op = OP[op]
        for i, s in enumerate(srcs):
            if s is not None:
                t.src[i] = C.pointer(s)
        for i, p in enumerate(params):
            t.op_params[i] = p
        t._srcs = srcs
        self.nodes.append(t)
        return t

    def on_gpu(self, t):
        self.L.ggml_cuda_assign_buffers_no_scratch(C.byref(t))
        return t

    # ---- op constructors (shapes as ggml.c builds them) -----------------------------------------------------
    def mul_mat(self, a, b, name="mul_mat"):
        return self._node("MUL_MAT", F32, [a.ne[1], b.ne[1], b.ne[2], b.ne[3]], [a, b], name)

    def relu(self, a, name="relu"):
        return self._node("UNARY", F32, list(a.ne), [a], name, params=(UNARY_RELU,))

    def mul(self, a, b, name="mul"):
        return self._node("MUL", F32, list(a.ne), [a, b], name)

    def add(self, a, b, name="add"):
        return self._node("ADD", F32, list(a.ne), [a, b], name)

    def mul_mat_idx(self, a, b, idx, gpu_idx, name="mul_mat_idx"):            # ggml.c:4126
        return self._node("MUL_MAT_SPARSE", F32, [a.ne[1], b.ne[1], b.ne[2], b.ne[3]], [a, b, idx, gpu_idx], name, params=(0 if gpu_idx is not None else 1,))

    def mul_mat_idx_upscale(self, a, b, idx, gpu_bucket, result_ne0, name="mul_mat_idx_upscale"):   # ggml.c:4100
        return self._node("MUL_MAT_SPARSE", F32, [result_ne0, b.ne[1], b.ne[2], b.ne[3]], [a, b, idx, gpu_bucket], name)

    def axpy(self, a, b, idx, aux, name="axpy"):                                # ggml.c:4158
        return self._node("AXPY", F32, [a.ne[0], b.ne[1], b.ne[2], b.ne[3]], [a, b, idx, aux], name, params=(0 if aux is not None else 1,))

    def _f32(self, v):
        return int(np.float32(v).view(np.int32))

    def rms_norm(self, a, eps, name="rms_norm"):                                # ggml.c:4553
        return self._node("RMS_NORM", F32, list(a.ne), [a], name, params=(self._f32(eps),))

    def norm(self, a, eps, name="norm"):                                        # ggml.c:4521
        return self._node("NORM", F32, list(a.ne), [a], name, params=(self._f32(eps),))

    def scale(self, a, s, name="scale"):                                        # ggml.c:4712 (the factor is a 1-element tensor)
        return self._node("SCALE", F32, list(a.ne), [a, s], name)

    def soft_max(self, a, name="soft_max"):                                     # ggml.c:5171
        return self._node("SOFT_MAX", F32, list(a.ne), [a], name)

    def rope(self, a, pos, n_dims, mode, freq_base=10000.0, freq_scale=1.0, name="rope", n_orig_ctx=0, ext_factor=0.0, attn_factor=1.0,
             beta_fast=32.0, beta_slow=1.0):                                                     # ggml_rope_impl, ggml.c:5222-5262
        params = [0, n_dims, mode, 0, n_orig_ctx, self._f32(freq_base), self._f32(freq_scale), self._f32(ext_factor), self._f32(attn_factor),
                  self._f32(beta_fast), self._f32(beta_slow)]
        return self._node("ROPE", F32, list(a.ne), [a, pos], name, params=params)

    def rope_inplace(self, a, pos, n_dims, mode, freq_base=10000.0, freq_scale=1.0, name="rope_inplace"):
        """ggml_rope_custom_inplace (ggml.c:5222-5262 with inplace = true): the result is a view of a, so the rotation overwrites it."""
        t = self.view(a, [a.ne[i] for i in range(4)], [a.nb[i] for i in range(1, 4)], 0, name)
        self.nodes.pop()
        t.op = OP["ROPE"]
        t.src[0], t.src[1] = C.pointer(a), C.pointer(pos)
        params = [0, n_dims, mode, 0, 0, self._f32(freq_base), self._f32(freq_scale), self._f32(0.0), self._f32(1.0), self._f32(32.0), self._f32(1.0)]
        for i, v in enumerate(params):
            t.op_params[i] = v
        t._srcs = [a, pos]
        self.nodes.append(t)
        return t

    def get_rows(self, a, ids, name="get_rows"):                                # ggml.c:4925
        return self._node("GET_ROWS", F32, [a.ne[0], ids.ne[0]], [a, ids], name)

    def view(self, a, ne, nb, offset, name="view"):
        """ggml_view_nd (ggml.c:4791-4900): a tensor over a's buffer with its own shape, byte strides nb[1..] and byte offset."""
        t = Tensor()
        t.type, t.backend, t.n_dims = a.type, CPU, len(ne)
        ne = list(ne) + [1] * (4 - len(ne))
        nb = [_tsize(a.type)] + list(nb)
        while len(nb) < 4:
            nb.append(nb[-1] * ne[len(nb) - 1])
        for i in range(4):
            t.ne[i], t.nb[i] = ne[i], nb[i]
        t.op = OP["VIEW"]
        t.src[0] = C.pointer(a)
        t.view_src = C.pointer(a)
        t.view_offs = offset
        t.op_params[0] = offset & 0xFFFFFFFF
        t.op_params[1] = offset >> 32
        t.data = a.data + offset
        t.name = name.encode()[:63]
        t._host, t._srcs = a._host, [a]
        self.nodes.append(t)
        return t

    def permute(self, a, axes, name="permute"):                                 # ggml_permute, ggml.c:4960-5010
        t = Tensor()
        t.type, t.backend, t.n_dims = a.type, CPU, 4
        for i in range(4):
            t.ne[axes[i]], t.nb[axes[i]] = a.ne[i], a.nb[i]
        t.op = OP["PERMUTE"]
        t.src[0] = C.pointer(a)
        t.view_src = a.view_src if a.view_src else C.pointer(a)
        t.view_offs = a.view_offs
        t.data = a.data
        t.name = name.encode()[:63]
        t._host, t._srcs = a._host, [a]
        self.nodes.append(t)
        return t

    def cpy(self, a, b, name="cpy"):                                            # ggml_cpy, ggml.c:4740: result is a view of b
        t = self.view(b, [b.ne[i] for i in range(4)], [b.nb[i] for i in range(1, 4)], 0, name)
        self.nodes.pop()
        t.op = OP["CPY"]
        t.src[0], t.src[1] = C.pointer(a), C.pointer(b)
        t._srcs = [a, b]
        self.nodes.append(t)
        return t

    def cont(self, a, name="cont"):                                             # ggml_cont, ggml.c:4766
        return self._node("CONT", a.type, [a.ne[i] for i in range(4)], [a], name)

    # ---- executor --------------------------------------------------------------------------------------
    def compute(self, threshold=0.0):
        self.L.ggml_cuda_set_device_constants(threshold)
        for t in self.nodes:
            handled = True
            for phase in (0, 1, 2):
                p = Params(phase, 0, 1, 0, None, None)
                handled = self.L.ggml_cuda_compute_forward(C.byref(p), C.byref(t)) and handled
            if handled:
                self.gpu_run.append(t.name.decode())
            else:
                self.cpu_run.append(t.name.decode())
                self._cpu(t, threshold)

    def host(self, t, dtype=np.float32):
        if t.backend == GPU:
            self.L.ggml_cuda_copy_to_host(C.byref(t))
        return t._host.view(dtype).reshape([t.ne[i] for i in (3, 2, 1, 0)]).squeeze()

    def _np(self, t, dtype=np.float32):
        if t.backend == GPU and t.extra:
            self.L.ggml_cuda_copy_to_host(C.byref(t))           # ggml_ensure_tensor_data_at_memory, ggml.c:14766
        return t._host.view(dtype)

    def _cpu(self, t, thr):
        """The reference's CPU kernels for nodes the backend declines (restated by the oracle)."""
        O = ol.oracle()
        s = t._srcs
        op = {v: k for k, v in OP.items()}[t.op]
        if op in ("VIEW", "PERMUTE", "RESHAPE", "TRANSPOSE"):
            return                                               # no computation (ggml.c:16508-16520)
        out = t._host.view(np.float32)
        T = int(t.ne[1] * t.ne[2] * t.ne[3])
        if op == "MUL_MAT":
            assert O.pio_mul_mat(s[0].type, P(s[0]._host), s[0].ne[1], s[0].ne[0], P(self._np(s[1])), T, P(out), 4) == 0
        elif op == "MUL_MAT_SPARSE":
            assert O.pio_mul_mat_sparse(s[0].type, P(s[0]._host), s[0].ne[1], s[0].ne[0], P(self._np(s[1])), T, P(self._np(s[2])),
                                        P(self._np(s[3], np.int32)), thr, P(out), 4) == 0
        elif op == "AXPY":
            assert O.pio_axpy(s[0].type, P(s[0]._host), s[0].ne[1], s[0].ne[0], P(self._np(s[1])), T, P(self._np(s[2])),
                              P(self._np(s[3], np.int32)), thr, P(out), 4) == 0
        elif op == "UNARY":
            out[:] = np.maximum(self._np(s[0]), 0)
        elif op == "MUL":
            out[:] = self._np(s[0]) * self._np(s[1])
        elif op == "ADD":
            out[:] = self._np(s[0]) + self._np(s[1])
        else:
            raise NotImplementedError(op)
