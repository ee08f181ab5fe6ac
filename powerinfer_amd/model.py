"""Python face of the decode engine (pi_model_* in include/powerinfer_hip.h): mirrors the slice of llama.h a
greedy batch-1 run uses -- load, llama_decode, llama_get_logits, greedy sampling, the token loop."""
import ctypes as C

import numpy as np

from . import lib as pl
from .lib import check

ARCH = {"llama": 0, "falcon": 1}

# tensor roles, same order as the enum in include/powerinfer_hip.h
KINDS = ["tok_embd", "output_norm", "output_norm_b", "output",
         "attn_norm", "attn_norm_b", "attn_norm_2", "attn_norm_2_b",
         "wq", "wk", "wv", "wqkv", "wo",
         "ffn_norm", "ffn_gate", "ffn_up", "ffn_down_t",
         "fc1", "fc2", "gpu_idx", "gpu_bucket", "neuron_rate"]
KIND = {k: i for i, k in enumerate(KINDS)}


class HParamsC(C.Structure):
    _fields_ = [("arch", C.c_int32), ("n_embd", C.c_int32), ("n_ff", C.c_int32), ("n_head", C.c_int32),
                ("n_head_kv", C.c_int32), ("n_layer", C.c_int32), ("n_vocab", C.c_int32), ("n_ctx", C.c_int32),
                ("norm_eps", C.c_float), ("rope_freq_base", C.c_float), ("sparse_threshold", C.c_float), ("rope_freq_scale", C.c_float)]


def _declare(L):
    vp, i = C.c_void_p, C.c_int
    L.pi_model_create.restype, L.pi_model_create.argtypes = vp, [C.POINTER(HParamsC)]
    L.pi_model_free.restype, L.pi_model_free.argtypes = None, [vp]
    L.pi_model_set_tensor.restype, L.pi_model_set_tensor.argtypes = i, [vp, i, i, i, vp, C.c_int64, C.c_int64, i]
    L.pi_model_finalize.restype, L.pi_model_finalize.argtypes = i, [vp]
    L.pi_model_kv_clear.restype, L.pi_model_kv_clear.argtypes = i, [vp]
    L.pi_model_kv_seq_rm.restype, L.pi_model_kv_seq_rm.argtypes = i, [vp, i, i]
    L.pi_model_kv_seq_shift.restype, L.pi_model_kv_seq_shift.argtypes = i, [vp, i, i, i]
    L.pi_model_decode.restype, L.pi_model_decode.argtypes = i, [vp, vp, i, i, vp]
    L.pi_model_generate.restype, L.pi_model_generate.argtypes = i, [vp, i, vp, C.POINTER(C.c_float)]
    L.pi_model_set_capture.restype, L.pi_model_set_capture.argtypes = i, [vp, i]
    L.pi_model_set_rest_on_gpu.restype, L.pi_model_set_rest_on_gpu.argtypes = i, [vp, i]
    L.pi_model_get_capture.restype, L.pi_model_get_capture.argtypes = i, [vp, vp, vp, vp, vp]
    L.pi_model_step_active.restype, L.pi_model_step_active.argtypes = i, [vp, vp, i]
    L.pi_model_batch_init.restype, L.pi_model_batch_init.argtypes = i, [vp, i]
    L.pi_model_batch_decode.restype, L.pi_model_batch_decode.argtypes = i, [vp, vp, vp, vp, vp]
    L.pi_model_batch_generate.restype, L.pi_model_batch_generate.argtypes = i, [vp, i, vp, C.POINTER(C.c_float)]
    L.pi_model_batch_kv_seq_rm.restype, L.pi_model_batch_kv_seq_rm.argtypes = i, [vp, i, i, i]
    L.pi_model_batch_kv_seq_shift.restype, L.pi_model_batch_kv_seq_shift.argtypes = i, [vp, i, i, i, i]
    L.pi_model_batch_kv_seq_cp.restype, L.pi_model_batch_kv_seq_cp.argtypes = i, [vp, i, i, i, i]
    L.pi_model_batch_union.restype, L.pi_model_batch_union.argtypes = i, [vp, vp]
    L.pi_model_batch_set_dense_above.restype, L.pi_model_batch_set_dense_above.argtypes = i, [vp, C.c_float]
    L.pi_model_batch_dense_layers.restype, L.pi_model_batch_dense_layers.argtypes = i, [vp]
    L.pi_model_kv_cells_init.restype, L.pi_model_kv_cells_init.argtypes = i, [vp, i]
    L.pi_model_kv_cells_decode.restype, L.pi_model_kv_cells_decode.argtypes = i, [vp, vp, vp, vp, i, vp, vp]
    L.pi_model_kv_cells_seq_rm.restype, L.pi_model_kv_cells_seq_rm.argtypes = i, [vp, i, i, i]
    L.pi_model_kv_cells_seq_cp.restype, L.pi_model_kv_cells_seq_cp.argtypes = i, [vp, i, i, i, i]
    L.pi_model_kv_cells_seq_keep.restype, L.pi_model_kv_cells_seq_keep.argtypes = i, [vp, i]
    L.pi_model_kv_cells_seq_shift.restype, L.pi_model_kv_cells_seq_shift.argtypes = i, [vp, i, i, i, i]
    L.pi_model_kv_cells_clear.restype, L.pi_model_kv_cells_clear.argtypes = i, [vp]
    L.pi_model_kv_cells_state.restype, L.pi_model_kv_cells_state.argtypes = i, [vp, vp, vp, vp]
    L.pi_model_time_section.restype, L.pi_model_time_section.argtypes = i, [vp, i, i, C.POINTER(C.c_float), C.POINTER(C.c_int)]


ENGINE_SYMBOLS = ["pi_model_create", "pi_model_free", "pi_model_set_tensor", "pi_model_finalize", "pi_model_kv_clear",
                  "pi_model_kv_seq_rm", "pi_model_kv_seq_shift",
                  "pi_model_decode", "pi_model_generate", "pi_model_set_capture", "pi_model_get_capture", "pi_model_set_rest_on_gpu",
                  "pi_model_step_active", "pi_model_time_section",
                  "pi_model_batch_init", "pi_model_batch_decode", "pi_model_batch_generate", "pi_model_batch_union",
                  "pi_model_batch_set_dense_above", "pi_model_batch_dense_layers",
                  "pi_model_batch_kv_seq_rm", "pi_model_batch_kv_seq_shift", "pi_model_batch_kv_seq_cp",
                  "pi_model_kv_cells_init", "pi_model_kv_cells_decode", "pi_model_kv_cells_seq_rm", "pi_model_kv_cells_seq_cp",
                  "pi_model_kv_cells_seq_keep", "pi_model_kv_cells_seq_shift", "pi_model_kv_cells_clear", "pi_model_kv_cells_state"]


def _type_of(a, hint):
    if a.dtype == np.float32:
        return pl.F32
    if a.dtype == np.float16:
        return pl.F16
    if a.dtype == np.int32:
        return pl.I32
    if a.dtype == np.uint8:
        return pl.Q4_0
    raise TypeError(f"{hint}: unsupported dtype {a.dtype}")


def _ne(a, t):
    """(ne0, ne1) of a 1-D or 2-D numpy array holding a tensor of ggml type t."""
    rows = a.shape[0] if a.ndim == 2 else 1
    inner = a.shape[-1]
    return (inner // 18 * 32 if t == pl.Q4_0 else inner), rows


class Model:
    def __init__(self, hp):
        self.L = pl.init()
        _declare(self.L)
        self.hp = hp
        c = HParamsC(ARCH[hp.arch], hp.n_embd, hp.n_ff, hp.n_head, hp.n_head_kv, hp.n_layer, hp.n_vocab, hp.n_ctx,
                     hp.norm_eps, hp.rope_freq_base, hp.sparse_threshold, hp.get("rope_freq_scale", 1.0))
        self.h = self.L.pi_model_create(C.byref(c))
        if not self.h:
            raise pl.PiError("pi_model_create: " + self.L.pi_last_error().decode())
        if hp.get("rest_on_gpu"):      # non-resident rows stay in pinned host memory and the GPU reads the active ones itself
            check(self.L.pi_model_set_rest_on_gpu(self.h, 1), "set_rest_on_gpu")
        self._keep = []        # host arrays the engine borrows (hybrid layers)
        self.n_seq = 0         # sequences of batched decoding (batch_init)

    def set_tensor(self, layer, kind, arr):
        arr = np.ascontiguousarray(arr)
        t = _type_of(arr, kind)
        ne0, ne1 = _ne(arr, t)
        self._keep.append(arr)
        check(self.L.pi_model_set_tensor(self.h, layer, KIND[kind], t, arr.ctypes.data_as(C.c_void_p), ne0, ne1, 0), f"set_tensor {kind}")

    def set_tensor_device(self, layer, kind, ptr, t, ne0, ne1):
        check(self.L.pi_model_set_tensor(self.h, layer, KIND[kind], t, ptr, ne0, ne1, 1), f"set_tensor {kind}")

    def load(self, model):
        """model: the dict powerinfer_amd.synth.make_model returns."""
        for k, a in model["glob"].items():
            self.set_tensor(-1, k, a)
        for il, Lr in enumerate(model["layers"]):
            for k, a in Lr.items():
                if k in KIND and a is not None:
                    self.set_tensor(il, k, a)
            if Lr.get("p") is not None and self.hp.get("use_rates", True):
                # the neurons' firing rates (the activation statistics the reference's solver works from): the engine deals the
                # neurons of a fully resident F16 layer out by rate over the groups of its fused kernel
                self.set_tensor(il, "neuron_rate", np.asarray(Lr["p"], np.float32))
        self.finalize()
        return self

    def finalize(self):
        check(self.L.pi_model_finalize(self.h), "pi_model_finalize")

    def kv_clear(self):
        check(self.L.pi_model_kv_clear(self.h), "pi_model_kv_clear")

    def kv_seq_rm(self, p0, p1):
        """llama_kv_cache_seq_rm for the model's own sequence; returns the number of live cells."""
        n = self.L.pi_model_kv_seq_rm(self.h, p0, p1)
        check(min(n, 0), "pi_model_kv_seq_rm")
        return n

    def kv_seq_shift(self, p0, p1, delta):
        """llama_kv_cache_seq_shift (positions in [p0, p1) move by delta, their K rows are rotated); returns the live cells."""
        n = self.L.pi_model_kv_seq_shift(self.h, p0, p1, delta)
        check(min(n, 0), "pi_model_kv_seq_shift")
        return n

    def decode(self, tokens, n_past, want_logits=True):
        tokens = np.ascontiguousarray(tokens, np.int32)
        logits = np.empty(self.hp.n_vocab, np.float32) if want_logits else None
        tok = self.L.pi_model_decode(self.h, tokens.ctypes.data_as(C.c_void_p), tokens.size, n_past,
                                     logits.ctypes.data_as(C.c_void_p) if want_logits else None)
        if tok < 0:
            raise pl.PiError(f"pi_model_decode ({tok}): " + self.L.pi_last_error().decode())
        return tok, logits

    def generate(self, n_steps):
        out = np.empty(n_steps, np.int32)
        ms = C.c_float(0)
        check(self.L.pi_model_generate(self.h, n_steps, out.ctypes.data_as(C.c_void_p), C.byref(ms)), "pi_model_generate")
        return out, float(ms.value)

    def set_capture(self, on):
        check(self.L.pi_model_set_capture(self.h, int(on)), "set_capture")

    def get_capture(self):
        hp = self.hp
        ffn = np.empty((hp.n_layer, hp.n_embd), np.float32)
        lg = np.empty((hp.n_layer, hp.n_ff), np.float32)
        na = np.empty(hp.n_layer, np.int32)
        src = np.empty((hp.n_layer, hp.n_embd), np.float32)
        check(self.L.pi_model_get_capture(self.h, ffn.ctypes.data_as(C.c_void_p), lg.ctypes.data_as(C.c_void_p),
                                          na.ctypes.data_as(C.c_void_p), src.ctypes.data_as(C.c_void_p)), "get_capture")
        return ffn, lg, na, src

    def step_active(self, n_steps):
        out = np.empty(n_steps, np.int32)
        check(self.L.pi_model_step_active(self.h, out.ctypes.data_as(C.c_void_p), n_steps), "step_active")
        return out

    def time_section(self, section, rounds):
        """(ms per instance, instances) of a replayed section: 0 qkv mat-vec, 1 sparse FFN block, 2 lm-head."""
        ms, n = C.c_float(0), C.c_int(0)
        check(self.L.pi_model_time_section(self.h, section, rounds, C.byref(ms), C.byref(n)), "time_section")
        return float(ms.value) / n.value, n.value

    # ---- batched greedy decoding: n_seq independent sequences, one token each per step ----------------------
    def batch_init(self, n_seq):
        check(self.L.pi_model_batch_init(self.h, n_seq), "pi_model_batch_init")
        self.n_seq = n_seq

    def batch_decode(self, tokens, positions, want_logits=True):
        if self.n_seq <= 0:
            raise pl.PiError("batch_decode: batch_init first")
        tokens = np.ascontiguousarray(tokens, np.int32)
        positions = np.ascontiguousarray(positions, np.int32)
        if tokens.size != self.n_seq or positions.size != self.n_seq:
            raise pl.PiError("batch_decode: one token and one position per sequence")
        nxt = np.empty(self.n_seq, np.int32)
        logits = np.empty((self.n_seq, self.hp.n_vocab), np.float32) if want_logits else None
        check(self.L.pi_model_batch_decode(self.h, tokens.ctypes.data_as(C.c_void_p), positions.ctypes.data_as(C.c_void_p),
                                           nxt.ctypes.data_as(C.c_void_p), logits.ctypes.data_as(C.c_void_p) if want_logits else None),
              "pi_model_batch_decode")
        return nxt, logits

    def batch_generate(self, n_steps):
        out = np.empty((n_steps, self.n_seq), np.int32)
        ms = C.c_float(0)
        check(self.L.pi_model_batch_generate(self.h, n_steps, out.ctypes.data_as(C.c_void_p), C.byref(ms)), "pi_model_batch_generate")
        return out, float(ms.value)

    def batch_kv_seq_rm(self, seq, p0, p1):
        n = self.L.pi_model_batch_kv_seq_rm(self.h, seq, p0, p1)
        check(min(n, 0), "pi_model_batch_kv_seq_rm")
        return n

    def batch_kv_seq_shift(self, seq, p0, p1, delta):
        n = self.L.pi_model_batch_kv_seq_shift(self.h, seq, p0, p1, delta)
        check(min(n, 0), "pi_model_batch_kv_seq_shift")
        return n

    def batch_kv_seq_cp(self, src, dst, p0, p1):
        """Cells [p0, p1) of sequence src become the same cells of dst (which must hold exactly p0 cells)."""
        n = self.L.pi_model_batch_kv_seq_cp(self.h, src, dst, p0, p1)
        check(min(n, 0), "pi_model_batch_kv_seq_cp")
        return n

    # ---- one KV cache with cells shared between sequences (llama_kv_cache) ----
    def kv_cells_init(self, n_cells):
        check(self.L.pi_model_kv_cells_init(self.h, int(n_cells)), "pi_model_kv_cells_init")
        self.n_cells = int(n_cells)

    def kv_cells_decode(self, tokens, positions, seqs, want_logits=True):
        """One step of up to 16 tokens.  seqs[t]: a sequence id, or a list of ids the token's cell belongs to with the lowest first
        (the token attends the cells of its first sequence, as the reference masks by seq_id[t][0]).  Returns (greedy next token per
        token, logits [n_tokens][n_vocab] or None)."""
        tokens = np.ascontiguousarray(tokens, np.int32)
        positions = np.ascontiguousarray(positions, np.int32)
        masks = np.zeros(tokens.size, np.uint32)
        for t, sq in enumerate(seqs):
            ids = [int(sq)] if np.isscalar(sq) else [int(v) for v in sq]
            if min(ids) != ids[0]:
                raise pl.PiError("kv_cells_decode: list a token's lowest sequence id first")
            for v in ids:
                masks[t] |= np.uint32(1 << v)
        nxt = np.empty(tokens.size, np.int32)
        logits = np.empty((tokens.size, self.hp.n_vocab), np.float32) if want_logits else None
        check(self.L.pi_model_kv_cells_decode(self.h, tokens.ctypes.data_as(C.c_void_p), positions.ctypes.data_as(C.c_void_p),
                                              masks.ctypes.data_as(C.c_void_p), int(tokens.size), nxt.ctypes.data_as(C.c_void_p),
                                              logits.ctypes.data_as(C.c_void_p) if want_logits else None), "pi_model_kv_cells_decode")
        return nxt, logits

    def kv_cells_seq_rm(self, seq, p0, p1):
        check(self.L.pi_model_kv_cells_seq_rm(self.h, seq, p0, p1), "pi_model_kv_cells_seq_rm")

    def kv_cells_seq_cp(self, src, dst, p0, p1):
        check(self.L.pi_model_kv_cells_seq_cp(self.h, src, dst, p0, p1), "pi_model_kv_cells_seq_cp")

    def kv_cells_seq_keep(self, seq):
        check(self.L.pi_model_kv_cells_seq_keep(self.h, seq), "pi_model_kv_cells_seq_keep")

    def kv_cells_seq_shift(self, seq, p0, p1, delta):
        check(self.L.pi_model_kv_cells_seq_shift(self.h, seq, p0, p1, delta), "pi_model_kv_cells_seq_shift")

    def kv_cells_clear(self):
        check(self.L.pi_model_kv_cells_clear(self.h), "pi_model_kv_cells_clear")

    def kv_cells_state(self):
        """(positions [n_cells] (-1: free), sequence bit sets [n_cells], head of the ring)"""
        pos, seq, head = np.empty(self.n_cells, np.int32), np.empty(self.n_cells, np.uint32), C.c_int32(0)
        n = self.L.pi_model_kv_cells_state(self.h, pos.ctypes.data_as(C.c_void_p), seq.ctypes.data_as(C.c_void_p), C.byref(head))
        check(min(n, 0), "pi_model_kv_cells_state")
        return pos, seq, int(head.value)

    def batch_union(self):
        out = np.empty(self.hp.n_layer, np.int32)
        check(self.L.pi_model_batch_union(self.h, out.ctypes.data_as(C.c_void_p)), "pi_model_batch_union")
        return out

    def batch_set_dense_above(self, fraction):
        """Layers whose union of active rows exceeded fraction * n_ff in the last step run their FFN dense (<= 0: always, >= 1: never)."""
        check(self.L.pi_model_batch_set_dense_above(self.h, float(fraction)), "pi_model_batch_set_dense_above")

    def batch_dense_layers(self):
        n = self.L.pi_model_batch_dense_layers(self.h)
        if n < 0:
            check(n, "pi_model_batch_dense_layers")
        return n

    def close(self):
        if self.h:
            self.L.pi_model_free(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
