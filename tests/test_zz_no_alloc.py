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
    # first call: the full 7B layer shape (344 partial vectors of 4096 floats); second: a smaller layer with LayerNorm, no gate
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
