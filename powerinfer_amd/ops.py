"""Host-side mirror of the reference's operator sequence for one sparse FFN block
(llm_build_ffn_sparse, llama.cpp:4652-4757), driving the HIP launchers through the C ABI.
Used by the parity tests and the layer-level benchmark; the fused decode loop lives in the C++ engine.
"""
import ctypes as C

import numpy as np

from . import lib as pl
from .lib import DevBuf, check


class SparseFFN:
    """Device-resident weights of one layer + the launch sequence
    fc1 -> relu -> fc2+threshold+compaction -> sparse up/gate -> sparse axpy.

    bucket (optional int32 array): the layer holds only the GPU-resident neurons (rows bucket[i] of the
    full matrices, compact, in bucket order) as llama.cpp's slice_ffn_mat_to_gpu does (llama.cpp:2898-2967).
    """

    def __init__(self, d, ff, r, wtype, up, gate, down_t, fc1, fc2, threshold=0.0, bucket=None,
                 norm_kind=pl.NORM_NONE, norm_w=None, norm_b=None, eps=1e-5):
        self.L = pl.init()
        self.d, self.ff, self.r, self.wtype, self.thr = d, ff, r, wtype, float(threshold)
        self.bucket_host = None if bucket is None else np.ascontiguousarray(bucket, np.int32)
        sel = (lambda a: a) if bucket is None else (lambda a: np.ascontiguousarray(a[self.bucket_host]))
        self.up = DevBuf(host=sel(up))
        self.gate = DevBuf(host=sel(gate)) if gate is not None else None
        self.down = DevBuf(host=sel(down_t))
        self.fc1, self.fc2 = DevBuf(host=fc1), DevBuf(host=fc2)
        self.bucket = DevBuf(host=self.bucket_host) if bucket is not None else None
        self.n_bucket = 0 if bucket is None else int(self.bucket_host.size)
        self.norm_kind, self.eps = norm_kind, eps
        self.norm_w = DevBuf(host=np.asarray(norm_w, np.float32)) if norm_w is not None else None
        self.norm_b = DevBuf(host=np.asarray(norm_b, np.float32)) if norm_b is not None else None
        self.ws = self.L.pi_workspace_create(ff, d)
        if not self.ws:
            raise pl.PiError(self.L.pi_last_error().decode())
        f4 = 4
        self.x, self.xp = DevBuf(d * f4), DevBuf(d * f4)
        self.hidden, self.logits = DevBuf(r * f4), DevBuf(ff * f4)
        self.list, self.n_active = DevBuf(ff * 4), DevBuf.zeros(4)
        self.h_c = DevBuf(ff * f4)
        self.h_dense, self.up_dense, self.gate_dense = DevBuf.zeros(ff * f4), DevBuf.zeros(ff * f4), DevBuf.zeros(ff * f4)
        self.out = DevBuf(d * f4)
        self.resid = DevBuf.zeros(d * f4)

    def launch(self, stream=None, dense_outputs=True, epilogue=pl.EPI_NONE):
        """dense_outputs: also scatter up/gate/h into neuron-indexed vectors (what GGML_OP_MUL_MAT_SPARSE returns);
        this takes the explicit-list route.  Without it (and without a bucket) the fused route runs: the up/gate
        kernel derives the active rows from the predictor's mask words itself."""
        L, p = self.L, (lambda b: b.ptr if b is not None else None)
        fused = not dense_outputs and self.bucket is None
        need_h_dense = dense_outputs or self.wtype == pl.Q4_0
        n_rows = self.n_bucket if self.bucket is not None else self.ff
        check(L.pi_k_gemv(pl.F16, self.fc1.ptr, self.r, self.d, self.xp.ptr, None, pl.EPI_RELU, None, None, self.hidden.ptr, stream), "fc1")
        check(L.pi_k_predictor_fc2(self.fc2.ptr, self.ff, self.r, self.hidden.ptr, self.thr, p(self.bucket), self.n_bucket,
                                   self.logits.ptr, None if fused else self.list.ptr, None if fused else self.n_active.ptr,
                                   self.h_dense.ptr if need_h_dense else None, self.ws, stream), "fc2")
        nrm = pl.norm_arg(self.norm_kind, self.eps, self.norm_w, self.norm_b)
        check(L.pi_k_sparse_upgate(self.wtype, self.up.ptr, p(self.gate), self.d, self.ff, self.x.ptr, nrm, int(fused),
                                   self.list.ptr, self.n_active.ptr, p(self.bucket), self.h_c.ptr,
                                   self.h_dense.ptr if need_h_dense else None,
                                   self.up_dense.ptr if dense_outputs else None,
                                   self.gate_dense.ptr if dense_outputs else None, self.ws, stream), "upgate")
        check(L.pi_k_sparse_axpy(self.wtype, self.down.ptr, self.d, n_rows, self.h_c.ptr,
                                 self.h_dense.ptr if self.wtype == pl.Q4_0 else None, p(self.bucket),
                                 self.list.ptr, self.n_active.ptr, epilogue, self.resid.ptr if epilogue else None, None,
                                 self.out.ptr, self.ws, stream), "axpy")

    def forward(self, x_ffn, x_pred, dense_outputs=True):
        """One token.  Returns dict(logits, active, up, gate, h, out) as numpy arrays (dense vectors are
        neuron-indexed; rows outside the GPU bucket stay zero; up/gate/h only with dense_outputs)."""
        self.x.upload(np.asarray(x_ffn, np.float32))
        self.xp.upload(np.asarray(x_pred, np.float32))
        for b in (self.up_dense, self.gate_dense, self.h_dense):
            check(self.L.pi_memset(b.ptr, 0, b.nbytes), "memset")
        self.launch(dense_outputs=dense_outputs)
        pl.sync()
        n = int(self.n_active.download(np.int32)[0])
        return dict(logits=self.logits.download(np.float32), active=self.list.download(np.int32, n),
                    up=self.up_dense.download(np.float32), gate=self.gate_dense.download(np.float32),
                    h=self.h_dense.download(np.float32), h_compact=self.h_c.download(np.float32, n),
                    out=self.out.download(np.float32))

    def forward_two_launch(self, x_ffn, x_pred, epilogue=pl.EPI_NONE, resid=None):
        """The full-GPU F16 fast route of the decode loop: fc1, then pi_k_pred_upgate (fc2 + mask + up/gate in one
        launch) and pi_k_sparse_axpy_dense (down projection from the dense h).  Returns dict(logits, mask_words,
        h, n_active, out)."""
        L = self.L
        if self.bucket is not None or self.wtype != pl.F16 or not L.pi_k_pred_upgate_supported(self.ff, self.r, self.d):
            raise pl.PiError("forward_two_launch: shape or placement outside the fused kernels")
        self.x.upload(np.asarray(x_ffn, np.float32))
        self.xp.upload(np.asarray(x_pred, np.float32))
        if resid is not None:
            self.resid.upload(np.asarray(resid, np.float32))
        check(L.pi_memset(self.h_dense.ptr, 0xFF, self.h_dense.nbytes), "memset")      # the kernel must write every entry
        nrm = pl.norm_arg(self.norm_kind, self.eps, self.norm_w, self.norm_b)
        check(L.pi_k_gemv(pl.F16, self.fc1.ptr, self.r, self.d, self.xp.ptr, None, pl.EPI_RELU, None, None, self.hidden.ptr, None), "fc1")
        check(L.pi_k_pred_upgate(self.fc2.ptr, self.ff, self.r, self.hidden.ptr, self.thr, self.up.ptr,
                                 self.gate.ptr if self.gate is not None else None, self.d, self.x.ptr, nrm,
                                 self.logits.ptr, self.h_dense.ptr, self.ws, None), "pred_upgate")
        check(L.pi_k_sparse_axpy_dense(self.down.ptr, self.d, self.ff, self.h_dense.ptr, self.n_active.ptr, epilogue,
                                       self.resid.ptr if epilogue else None, None, self.out.ptr, self.ws, None), "axpy_dense")
        pl.sync()
        return dict(logits=self.logits.download(np.float32), h=self.h_dense.download(np.float32),
                    n_active=int(self.n_active.download(np.int32)[0]), out=self.out.download(np.float32))

    def forward_one_launch(self, x_ffn, x_pred, epilogue=pl.EPI_NONE, resid=None, noalloc=False):
        """fc1, then pi_k_sparse_ffn: predictor fc2, mask, gate/up, h and the down projection in one launch plus the
        fixed-order reduction of the per-workgroup partial outputs.  Returns dict(logits, h, n_active, out).
        noalloc: go through pi_k_sparse_ffn_noalloc (scratch in the library's static device array, no workspace)."""
        L = self.L
        if self.bucket is not None or self.wtype != pl.F16 or not L.pi_k_sparse_ffn_supported(self.ff, self.r, self.d):
            raise pl.PiError("forward_one_launch: shape or placement outside the fused kernel")
        self.x.upload(np.asarray(x_ffn, np.float32))
        self.xp.upload(np.asarray(x_pred, np.float32))
        if resid is not None:
            self.resid.upload(np.asarray(resid, np.float32))
        check(L.pi_memset(self.h_dense.ptr, 0xFF, self.h_dense.nbytes), "memset")      # the kernel must write every entry
        nrm = pl.norm_arg(self.norm_kind, self.eps, self.norm_w, self.norm_b)
        check(L.pi_k_gemv(pl.F16, self.fc1.ptr, self.r, self.d, self.xp.ptr, None, pl.EPI_RELU, None, None, self.hidden.ptr, None), "fc1")
        args = (self.fc2.ptr, self.ff, self.r, self.hidden.ptr, self.thr, self.up.ptr,
                self.gate.ptr if self.gate is not None else None, self.down.ptr, self.d, self.x.ptr, nrm,
                epilogue, self.resid.ptr if epilogue else None, None, self.out.ptr,
                self.logits.ptr, self.h_dense.ptr, self.n_active.ptr)
        if noalloc:
            check(L.pi_k_sparse_ffn_noalloc(*args, None), "sparse_ffn_noalloc")
        else:
            check(L.pi_k_sparse_ffn(*args, self.ws, None), "sparse_ffn")
        pl.sync()
        return dict(logits=self.logits.download(np.float32), h=self.h_dense.download(np.float32),
                    n_active=int(self.n_active.download(np.int32)[0]), out=self.out.download(np.float32))

    def _hot_tables(self):
        """hot_words[g] bit j: neuron 32g+j is GPU-resident; hot_prefix[g]: resident neurons before group g."""
        if self.bucket_host is None:
            return None, None
        if not hasattr(self, "_hot"):
            bits = np.zeros(self.ff, np.uint8)
            bits[self.bucket_host] = 1
            words = (bits.reshape(-1, 32).astype(np.uint64) << np.arange(32, dtype=np.uint64)).sum(1).astype(np.uint32)
            prefix = np.concatenate([[0], np.cumsum(bits.reshape(-1, 32).sum(1))[:-1]]).astype(np.int32)
            self._hot = (DevBuf(host=words), DevBuf(host=prefix))
        return self._hot

    def forward_one_launch_hot(self, x_ffn, x_pred, epilogue=pl.EPI_NONE, resid=None):
        """The fused F16 route on a hot/cold split layer: pi_k_sparse_ffn_partials_hot + pi_k_sparse_ffn_reduce_hot over the
        bucket's compact matrices.  Returns dict(logits, h, xn16, n_active, out): out is the resident neurons' share."""
        L = self.L
        if self.bucket is None or self.wtype != pl.F16 or not L.pi_k_sparse_ffn_supported(self.ff, self.r, self.d):
            raise pl.PiError("forward_one_launch_hot: needs a bucket, F16 weights and a shape the fused kernel covers")
        hw, hp = self._hot_tables()
        self.x.upload(np.asarray(x_ffn, np.float32))
        self.xp.upload(np.asarray(x_pred, np.float32))
        if resid is not None:
            self.resid.upload(np.asarray(resid, np.float32))
        check(L.pi_memset(self.h_dense.ptr, 0xFF, self.h_dense.nbytes), "memset")      # the kernel must write every entry
        xn16 = DevBuf(self.d * 2)
        nrm = pl.norm_arg(self.norm_kind, self.eps, self.norm_w, self.norm_b)
        check(L.pi_k_gemv(pl.F16, self.fc1.ptr, self.r, self.d, self.xp.ptr, None, pl.EPI_RELU, None, None, self.hidden.ptr, None), "fc1")
        check(L.pi_k_sparse_ffn_partials_hot(self.fc2.ptr, self.ff, self.r, self.hidden.ptr, self.thr, self.up.ptr,
                                             self.gate.ptr if self.gate is not None else None, self.down.ptr, self.d, self.x.ptr, nrm,
                                             hw.ptr, hp.ptr, self.logits.ptr, self.h_dense.ptr, xn16.ptr, self.ws, None), "partials_hot")
        check(L.pi_k_sparse_ffn_reduce_hot(self.ff, self.d, epilogue, self.resid.ptr if epilogue else None, None, self.out.ptr,
                                           self.n_active.ptr, self.ws, None), "reduce_hot")
        pl.sync()
        return dict(logits=self.logits.download(np.float32), h=self.h_dense.download(np.float32), xn16=xn16.download(np.float16),
                    n_active=int(self.n_active.download(np.int32)[0]), out=self.out.download(np.float32))

    def forward_q4_fused(self, x_ffn, x_pred, epilogue=pl.EPI_NONE, resid=None, fill_h=None):
        """Q4_0 route of the decode loop at d = 4096: fc1, pi_k_pred_upgate_q4 (fc2 + mask + up/gate of the resident neurons),
        then pi_k_axpy_q4_partials + pi_k_axpy_q4_reduce.  fill_h(h) may return the vector with the host share's neurons
        filled in (hybrid layers) before the down projection.  Returns dict(logits, h, xq8, n_active, out)."""
        L = self.L
        if self.wtype != pl.Q4_0 or not L.pi_k_pred_upgate_q4_supported(self.ff, self.r, self.d):
            raise pl.PiError("forward_q4_fused: type or shape outside the fused kernels")
        hw, hp = self._hot_tables()
        p = lambda b: b.ptr if b is not None else None  # noqa: E731
        self.x.upload(np.asarray(x_ffn, np.float32))
        self.xp.upload(np.asarray(x_pred, np.float32))
        if resid is not None:
            self.resid.upload(np.asarray(resid, np.float32))
        check(L.pi_memset(self.h_dense.ptr, 0xFF, self.h_dense.nbytes), "memset")      # the kernel must write every entry
        xq8 = DevBuf(self.d // 32 * 34)
        nrm = pl.norm_arg(self.norm_kind, self.eps, self.norm_w, self.norm_b)
        check(L.pi_k_gemv(pl.F16, self.fc1.ptr, self.r, self.d, self.xp.ptr, None, pl.EPI_RELU, None, None, self.hidden.ptr, None), "fc1")
        check(L.pi_k_pred_upgate_q4(self.fc2.ptr, self.ff, self.r, self.hidden.ptr, self.thr, self.up.ptr, p(self.gate), self.d,
                                    self.x.ptr, nrm, p(hw), p(hp), self.logits.ptr, self.h_dense.ptr, xq8.ptr, self.ws, None), "pred_upgate_q4")
        pl.sync()
        h = self.h_dense.download(np.float32)
        if fill_h is not None:
            self.h_dense.upload(np.ascontiguousarray(fill_h(h.copy()), np.float32))
        check(L.pi_k_axpy_q4_partials(self.down.ptr, self.d, self.ff, self.h_dense.ptr, p(hw), p(hp), self.ws, None), "axpy_q4_partials")
        check(L.pi_k_axpy_q4_reduce(self.ff, self.d, epilogue, self.resid.ptr if epilogue else None, None, self.out.ptr,
                                    self.n_active.ptr, self.ws, None), "axpy_q4_reduce")
        pl.sync()
        return dict(logits=self.logits.download(np.float32), h=h, xq8=xq8.download(np.uint8),
                    n_active=int(self.n_active.download(np.int32)[0]), out=self.out.download(np.float32))

    def forward_q4_one_launch(self, x_ffn, x_pred, epilogue=pl.EPI_NONE, resid=None, rest=None):
        """The Q4_0 layer as the decode loop runs it when every active neuron is computed on the device: fc1, then
        pi_k_sparse_ffn_q4_partials (fc2 + mask + up/gate + down rows of each workgroup's 32 neurons) and pi_k_sparse_ffn_q4_reduce.
        With a bucket, `rest` = (up, gate, down_t) rows of the neurons outside it in ascending order (the split form: those rows may
        be pinned host memory in the engine).  Returns dict(logits, h, n_active, out)."""
        L = self.L
        if self.wtype != pl.Q4_0 or not L.pi_k_pred_upgate_q4_supported(self.ff, self.r, self.d):
            raise pl.PiError("forward_q4_one_launch: type or shape outside the fused kernels")
        hw, hp = self._hot_tables()
        if (hw is None) != (rest is None):
            raise pl.PiError("forward_q4_one_launch: a bucket and the other neurons' rows go together")
        p = lambda b: b.ptr if b is not None else None  # noqa: E731
        keep = [DevBuf(host=a) if a is not None else None for a in (rest or (None, None, None))]
        self.x.upload(np.asarray(x_ffn, np.float32))
        self.xp.upload(np.asarray(x_pred, np.float32))
        if resid is not None:
            self.resid.upload(np.asarray(resid, np.float32))
        check(L.pi_memset(self.h_dense.ptr, 0xFF, self.h_dense.nbytes), "memset")      # the kernel must write every entry
        nrm = pl.norm_arg(self.norm_kind, self.eps, self.norm_w, self.norm_b)
        check(L.pi_k_gemv(pl.F16, self.fc1.ptr, self.r, self.d, self.xp.ptr, None, pl.EPI_RELU, None, None, self.hidden.ptr, None), "fc1")
        check(L.pi_k_sparse_ffn_q4_partials(self.fc2.ptr, self.ff, self.r, self.hidden.ptr, self.thr, self.up.ptr, p(self.gate), self.down.ptr,
                                            p(keep[0]), p(keep[1]), p(keep[2]), self.d, self.x.ptr, nrm, p(hw), p(hp),
                                            self.logits.ptr, self.h_dense.ptr, self.ws, None), "sparse_ffn_q4_partials")
        check(L.pi_k_sparse_ffn_q4_reduce(self.ff, self.d, epilogue, self.resid.ptr if epilogue else None, None, self.out.ptr,
                                          self.n_active.ptr, self.ws, None), "sparse_ffn_q4_reduce")
        pl.sync()
        return dict(logits=self.logits.download(np.float32), h=self.h_dense.download(np.float32),
                    n_active=int(self.n_active.download(np.int32)[0]), out=self.out.download(np.float32))

    def forward_q4_handover(self, x_ffn, x_pred, host_h, host_out, limit_s=20.0):
        """The same layer with the host share computed while the stream runs, nothing launched in between (what the decode loop
        queues for a hybrid Q4_0 layer): pi_k_pred_q4_logits -> pi_k_upgate_q4_hot_rows (its first lane starts the hand-over) ->
        pi_k_host_signal_wait -> pi_k_axpy_q4_partials (h in pinned memory) -> pi_k_host_wait -> pi_k_axpy_q4_reduce (+ the host
        share's output from pinned memory).  Everything is queued first; then this thread plays the host side: once the logits have
        arrived host_h(logits, xq8) returns {neuron: h} for the host's neurons, and once the resident neurons' h has arrived
        host_out(h_full) returns the host share of the output.  Returns dict(logits, h, n_active, out, status)."""
        import ctypes as C
        import time
        L = self.L
        if self.wtype != pl.Q4_0 or not L.pi_k_pred_upgate_q4_supported(self.ff, self.r, self.d):
            raise pl.PiError("forward_q4_handover: type or shape outside the fused kernels")
        hw, hp = self._hot_tables()
        if hw is None:
            raise pl.PiError("forward_q4_handover: needs a hot/cold split")
        p = lambda b: b.ptr if b is not None else None  # noqa: E731

        def pinned(nbytes, dtype):
            ptr = L.pi_malloc_host(nbytes)
            if not ptr:
                raise pl.PiError("pi_malloc_host: " + L.pi_last_error().decode())
            arr = np.frombuffer((C.c_char * nbytes).from_address(ptr), dtype=dtype)
            arr[...] = 0
            return ptr, arr

        flags_p, flags = pinned(64 * 4, np.uint32)
        lg_p, lg = pinned(self.ff * 4, np.float32)
        h_p, h = pinned(self.ff * 4, np.float32)
        out_p, out_host = pinned(self.d * 4, np.float32)
        xq_p, xq = pinned(self.d // 32 * 34, np.uint8)
        words_p, words = pinned(self.ff // 32 * 4, np.uint32)
        seq, status, lg_dev = DevBuf.zeros(4), DevBuf.zeros(4), DevBuf(self.ff * 4)
        try:
            self.x.upload(np.asarray(x_ffn, np.float32))
            self.xp.upload(np.asarray(x_pred, np.float32))
            nrm = pl.norm_arg(self.norm_kind, self.eps, self.norm_w, self.norm_b)
            check(L.pi_k_gemv(pl.F16, self.fc1.ptr, self.r, self.d, self.xp.ptr, None, pl.EPI_RELU, None, None, self.hidden.ptr, None), "fc1")
            check(L.pi_k_pred_q4_logits(self.fc2.ptr, self.ff, self.r, self.hidden.ptr, self.thr, self.d, self.x.ptr, nrm, lg_p, lg_dev.ptr, xq_p, words_p, self.ws, None), "pred_q4_logits")
            check(L.pi_k_upgate_q4_hot_rows(self.ff, self.thr, self.up.ptr, p(self.gate), self.d, self.x.ptr, nrm, hw.ptr, hp.ptr, lg_dev.ptr, h_p,
                                            seq.ptr, flags_p, self.ws, None), "hot_rows")
            check(L.pi_k_host_signal_wait(seq.ptr, flags_p, 8, 16, status.ptr, limit_s, None), "signal_wait")
            check(L.pi_k_axpy_q4_partials(self.down.ptr, self.d, self.ff, h_p, hw.ptr, hp.ptr, self.ws, None), "axpy_q4_partials")
            check(L.pi_k_host_wait(seq.ptr, flags_p, 32, status.ptr, limit_s, None), "wait")
            check(L.pi_k_axpy_q4_reduce(self.ff, self.d, pl.EPI_ADD, out_p, None, self.out.ptr, self.n_active.ptr, self.ws, None), "axpy_q4_reduce")

            def wait_flag(word):
                t0 = time.time()
                while int(flags[word]) != 1:
                    if time.time() - t0 > limit_s:
                        flags[48] = 1
                        raise pl.PiError("forward_q4_handover: the device never signalled word %d" % word)
            wait_flag(0)
            for j, v in host_h(lg.copy(), xq.copy()).items():
                h[j] = v
            flags[16] = 1
            wait_flag(8)
            out_host[...] = host_out(h.copy())
            flags[32] = 1
            pl.sync()
            return dict(logits=lg.copy(), h=h.copy(), n_active=int(self.n_active.download(np.int32)[0]), out=self.out.download(np.float32),
                        status=int(status.download(np.uint32)[0]), words=words.copy())
        finally:
            pl.sync()
            del flags, lg, h, out_host, xq, words
            for ptr in (flags_p, lg_p, h_p, out_p, xq_p, words_p):
                L.pi_free_host(ptr)

    def close(self):
        if self.ws:
            self.L.pi_workspace_destroy(self.ws)
            self.ws = None
