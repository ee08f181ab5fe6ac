"""pi_k_sparse_ffn_noalloc (scratch in the library's static device array, no allocation) against pi_k_sparse_ffn on the same
inputs.  Both run the same kernels in the same order, so every output must be bit-identical.  Two calls in a row, the second
on a smaller layer, show that what the first call left in the shared scratch array does not leak into the second."""
import numpy as np
import pytest

import oracle_lib as ol
from powerinfer_amd import synth

pytestmark = pytest.mark.gpu


def test_noalloc_matches_workspace_entry_point_twice():
    from powerinfer_amd import lib as pl
    from powerinfer_amd.ops import SparseFFN
    L = pl.init()
    assert L.pi_k_sparse_ffn_noalloc_scratch_bytes() == (8 << 20) + 2 * 4 * 4096
    rng = np.random.default_rng(9)
    # first call: the full 7B layer shape (one partial vector of 4096 floats per compute unit); second: a smaller layer with LayerNorm, no gate
    for (d, ff, r, has_gate, norm) in ((4096, 11008, 1024, True, 1), (4096, 2048, 512, False, 2)):
        assert L.pi_k_sparse_ffn_noalloc_supported(ff, r, d) == 1
        Ly = synth.make_ffn_layer(seed=31 + ff, d=d, ff=ff, r=r, wtype=ol.F16, has_gate=has_gate, T=2)
        nw = (1 + 0.1 * rng.standard_normal(d)).astype(np.float32)
        nb = (0.1 * rng.standard_normal(d)).astype(np.float32) if norm == 2 else None
        ffn = SparseFFN(d, ff, r, ol.F16, Ly["up"], Ly["gate"], Ly["down_t"], Ly["fc1"], Ly["fc2"], norm_kind=norm, norm_w=nw, norm_b=nb)
        for t in range(2):
            resid = rng.standard_normal(d).astype(np.float32)
            a = ffn.forward_one_launch(Ly["x"][t], Ly["x"][t], epilogue=pl.EPI_ADD, resid=resid)
            b = ffn.forward_one_launch(Ly["x"][t], Ly["x"][t], epilogue=pl.EPI_ADD, resid=resid, noalloc=True)
            assert a["n_active"] == b["n_active"] and a["n_active"] > 0
            for k in ("logits", "h", "out"):
                assert np.array_equal(a[k], b[k]), k
            # and against the CPU oracle evaluated under the predictor logits the GPU produced
            o = ol.ffn_under_logits(ol.oracle(), d, ff, ol.F16, has_gate, Ly["up"], Ly["gate"], Ly["down_t"],
                                    ol.apply_norm(Ly["x"][t], norm, nw, nb, 1e-5), b["logits"], 0.0)
            assert np.abs(b["out"] - resid - o["out"]).max() <= 2e-3 * np.abs(o["out"]).max()
        ffn.close()


def test_noalloc_rejects_shapes_beyond_the_scratch():
    from powerinfer_amd import lib as pl
    L = pl.init()
    # 4096 columns: one partial vector per 32 neurons -> 8 MiB holds ff <= 16384
    assert L.pi_k_sparse_ffn_noalloc_supported(16384, 1024, 4096) == 1
    assert L.pi_k_sparse_ffn_noalloc_supported(16416, 1024, 4096) == 0
    assert L.pi_k_sparse_ffn_noalloc_supported(32768, 1024, 8192) == 1      # Falcon-40B layer: 256 partial vectors of 8192 floats
    assert L.pi_k_sparse_ffn_noalloc_supported(65536, 1024, 8192) == 0
    assert L.pi_k_sparse_ffn_noalloc_supported(11008, 1024, 5120) == 0      # a width the fused kernel does not cover
    buf = pl.DevBuf(64)
    rc = L.pi_k_sparse_ffn_noalloc(buf.ptr, 16416, 1024, buf.ptr, 0.0, buf.ptr, None, buf.ptr, 4096, buf.ptr, None, 0, None, None, buf.ptr,
                                   None, None, None, None)
    assert rc == -3 and b"static scratch" in L.pi_last_error()


def _hip():
    import ctypes as C
    hip = C.CDLL("libamdhip64.so")
    hip.hipMemGetInfo.argtypes = [C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)]
    vp, pvp = C.c_void_p, C.POINTER(C.c_void_p)
    hip.hipStreamCreate.argtypes = [pvp]
    hip.hipStreamBeginCapture.argtypes = [vp, C.c_int]
    hip.hipStreamEndCapture.argtypes = [vp, pvp]
    hip.hipGraphInstantiate.argtypes = [pvp, vp, vp, vp, C.c_size_t]
    hip.hipGraphLaunch.argtypes = [vp, vp]
    hip.hipStreamSynchronize.argtypes = [vp]
    hip.hipGraphExecDestroy.argtypes = [vp]
    hip.hipGraphDestroy.argtypes = [vp]
    hip.hipStreamDestroy.argtypes = [vp]
    return hip, C


def test_noalloc_allocates_nothing_and_replays_from_a_graph():
    """What the entry point is for: device memory in use does not move over many calls, and a call recorded into a HIP graph (stream
    capture, thread-local mode) replays with the eager call's bits - several replays, with eager launches and synchronisations of the
    program's own in between, every replay checked."""
    from powerinfer_amd import lib as pl
    from powerinfer_amd.ops import SparseFFN
    L = pl.init()
    hip, C = _hip()
    d, ff, r = 4096, 11008, 1024
    Ly = synth.make_ffn_layer(seed=5, d=d, ff=ff, r=r, wtype=ol.F16, has_gate=True, T=3)
    nw = np.ones(d, np.float32)
    ffn = SparseFFN(d, ff, r, ol.F16, Ly["up"], Ly["gate"], Ly["down_t"], Ly["fc1"], Ly["fc2"], norm_kind=1, norm_w=nw)
    eager = [ffn.forward_one_launch(Ly["x"][t], Ly["x"][t], noalloc=True) for t in range(3)]

    def mem_free():
        f, t = C.c_size_t(0), C.c_size_t(0)
        assert hip.hipMemGetInfo(C.byref(f), C.byref(t)) == 0
        return f.value
    free0 = mem_free()
    for i in range(24):
        ffn.forward_one_launch(Ly["x"][i % 3], Ly["x"][i % 3], noalloc=True)
    assert mem_free() == free0

    # record fc1 + the no-alloc entry point on a stream of the test's own, replay for each input
    stream, graph, gexec = C.c_void_p(), C.c_void_p(), C.c_void_p()
    assert hip.hipStreamCreate(C.byref(stream)) == 0
    nrm = pl.norm_arg(1, 1e-5, ffn.norm_w, None)
    assert hip.hipStreamBeginCapture(stream, 1) == 0                     # hipStreamCaptureModeThreadLocal
    pl.check(L.pi_k_gemv(pl.F16, ffn.fc1.ptr, r, d, ffn.xp.ptr, None, pl.EPI_RELU, None, None, ffn.hidden.ptr, stream), "fc1")
    pl.check(L.pi_k_sparse_ffn_noalloc(ffn.fc2.ptr, ff, r, ffn.hidden.ptr, 0.0, ffn.up.ptr, ffn.gate.ptr, ffn.down.ptr, d, ffn.x.ptr, nrm,
                                       pl.EPI_NONE, None, None, ffn.out.ptr, ffn.logits.ptr, ffn.h_dense.ptr, ffn.n_active.ptr, stream), "noalloc under capture")
    assert hip.hipStreamEndCapture(stream, C.byref(graph)) == 0
    assert hip.hipGraphInstantiate(C.byref(gexec), graph, None, None, 0) == 0
    for rep in range(2):
        for t in range(3):
            ffn.x.upload(np.asarray(Ly["x"][t], np.float32))
            ffn.xp.upload(np.asarray(Ly["x"][t], np.float32))
            pl.check(L.pi_memset(ffn.out.ptr, 0xFF, ffn.out.nbytes), "memset")
            pl.sync()
            assert hip.hipGraphLaunch(gexec, stream) == 0
            assert hip.hipStreamSynchronize(stream) == 0
            assert np.array_equal(ffn.out.download(np.float32).view(np.uint32), eager[t]["out"].view(np.uint32)), (rep, t)
            assert np.array_equal(ffn.logits.download(np.float32).view(np.uint32), eager[t]["logits"].view(np.uint32))
            assert int(ffn.n_active.download(np.int32)[0]) == eager[t]["n_active"]
            ffn.forward_one_launch(Ly["x"][(t + 1) % 3], Ly["x"][(t + 1) % 3])          # eager work of the program's own between replays
    hip.hipGraphExecDestroy(gexec); hip.hipGraphDestroy(graph); hip.hipStreamDestroy(stream)
    ffn.close()
