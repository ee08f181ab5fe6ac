"""Dense operators of the decode path (mat-vec with fused norm, RoPE + KV store, decode attention, embedding,
argmax) through the C ABI against the CPU oracle and the reference's golden vectors."""
import ctypes as C

import numpy as np
import pytest

import oracle_lib as ol
from oracle_lib import _ptr as P
from powerinfer_amd import synth

pytestmark = pytest.mark.gpu


def rel_err(a, b):
    return float(np.abs(a - b).max() / max(np.abs(b).max(), 1e-30))


def gpu_gemv(wtype, w, rows, cols, x, norm=None, epi=0, add1=None, add2=None):
    from powerinfer_amd import lib as pl
    L = pl.init()
    dw, dx, dy = pl.DevBuf(host=w), pl.DevBuf(host=x.astype(np.float32)), pl.DevBuf(rows * 4)
    d1 = pl.DevBuf(host=add1) if add1 is not None else None
    d2 = pl.DevBuf(host=add2) if add2 is not None else None
    na = None
    keep = []
    if norm is not None:
        kind, eps, nw, nb = norm
        bw = pl.DevBuf(host=nw) if nw is not None else None
        bb = pl.DevBuf(host=nb) if nb is not None else None
        keep += [bw, bb]
        na = pl.norm_arg(kind, eps, bw, bb)
    pl.check(L.pi_k_gemv(wtype, dw.ptr, rows, cols, dx.ptr, na, epi, d1.ptr if d1 else None, d2.ptr if d2 else None, dy.ptr, None), "gemv")
    pl.sync()
    return dy.download(np.float32)


@pytest.mark.parametrize("wtype", [ol.F16, ol.Q4_0])
@pytest.mark.parametrize("rows,cols", [(40, 256), (4096, 4096), (12288, 4096), (1024, 4096), (3000, 8192), (2050, 5120)])
def test_gemv_plain(wtype, rows, cols):
    rng = np.random.default_rng(rows + cols)
    w32 = (rng.standard_normal((rows, cols)) * 0.02).astype(np.float32)
    w = synth.encode(w32, wtype)
    x = rng.standard_normal(cols).astype(np.float32)
    want = np.zeros(rows, np.float32)
    assert ol.oracle().pio_mul_mat(wtype, P(w), rows, cols, P(x), 1, P(want), 8) == 0
    got = gpu_gemv(wtype, w, rows, cols, x)
    assert rel_err(got, want) < 2e-6


def test_gemv_golden_reference(golden):
    g = golden("ops")
    for tag, wt in (("mm_f16", ol.F16), ("mm_q4", ol.Q4_0)):
        w, x, y = g[tag + "_w"], g[tag + "_x"], g[tag + "_y"]
        for t in range(x.shape[0]):
            got = gpu_gemv(wt, w, y.shape[1], x.shape[1], x[t])
            assert rel_err(got, y[t]) < 2e-6


@pytest.mark.parametrize("wtype,cols,rows", [(ol.F16, 4096, 2048), (ol.Q4_0, 4096, 2048), (ol.F16, 5120, 2304), (ol.F16, 8192, 2304),
                                             (ol.F16, 8192, 120), (ol.Q4_0, 8192, 2048)])
@pytest.mark.parametrize("kind", [1, 2])
def test_gemv_fused_norm_and_epilogues(wtype, cols, rows, kind):
    """The register-resident mat-vecs with the fused RMSNorm / LayerNorm prologue at every width they are instantiated for:
    4096 (7B), 5120 (13B), 8192 (Falcon-40B: a row is split in two halves, LayerNorm with bias is what its q|k|v projection
    runs), with more rows than the grid has waves (2304 = 2048 + 256: a second, partial round), fewer (120) and Q4_0."""
    from powerinfer_amd import lib as pl
    rng = np.random.default_rng(kind * 7 + wtype + cols)
    w = synth.encode((rng.standard_normal((rows, cols)) * 0.02).astype(np.float32), wtype)
    x = (rng.standard_normal(cols) * 3 + 0.5).astype(np.float32)
    nw = (1 + 0.1 * rng.standard_normal(cols)).astype(np.float32)
    nb = (0.1 * rng.standard_normal(cols)).astype(np.float32) if kind == 2 else None
    a1, a2 = rng.standard_normal(rows).astype(np.float32), rng.standard_normal(rows).astype(np.float32)
    O = ol.oracle()
    xn = np.zeros_like(x)
    (O.pio_rms_norm if kind == 1 else O.pio_norm)(P(x), cols, 1, 1e-5, P(xn))
    xn = xn * nw
    if nb is not None:
        xn = xn + nb
    want = np.zeros(rows, np.float32)
    assert O.pio_mul_mat(wtype, P(w), rows, cols, P(np.ascontiguousarray(xn, np.float32)), 1, P(want), 8) == 0
    got = gpu_gemv(wtype, w, rows, cols, x, norm=(kind, 1e-5, nw, nb))
    assert rel_err(got, want) < 5e-6
    assert rel_err(gpu_gemv(wtype, w, rows, cols, x, norm=(kind, 1e-5, nw, nb), epi=pl.EPI_RELU), np.maximum(want, 0)) < 5e-6
    assert rel_err(gpu_gemv(wtype, w, rows, cols, x, norm=(kind, 1e-5, nw, nb), epi=pl.EPI_ADD, add1=a1), want + a1) < 5e-6
    assert rel_err(gpu_gemv(wtype, w, rows, cols, x, norm=(kind, 1e-5, nw, nb), epi=pl.EPI_ADD2, add1=a1, add2=a2), (want + a1) + a2) < 5e-6


def test_gemv_rejects_bad_shapes():
    from powerinfer_amd import lib as pl
    L = pl.init()
    b = pl.DevBuf(1024)
    assert L.pi_k_gemv(pl.F16, b.ptr, 4, 12, b.ptr, None, 0, None, None, b.ptr, None) == -1      # cols % 8
    assert L.pi_k_gemv(pl.Q4_0, b.ptr, 4, 48, b.ptr, None, 0, None, None, b.ptr, None) == -1     # cols % 32
    assert L.pi_k_gemv(7, b.ptr, 4, 64, b.ptr, None, 0, None, None, b.ptr, None) == -3           # unsupported type
    assert L.pi_k_gemv(pl.F16, None, 4, 64, b.ptr, None, 0, None, None, b.ptr, None) == -1
    assert L.pi_k_gemv(pl.F16, b.ptr, 4, 64, b.ptr, None, pl.EPI_ADD, None, None, b.ptr, None) == -1
    assert b"pi_k_gemv" in L.pi_last_error()


@pytest.mark.parametrize("mode,hd,nh,nkv,chunks,fs", [(0, 128, 4, 4, (37, 45), 1.0), (2, 64, 8, 2, (70, 17, 2), 1.0), (0, 128, 2, 1, (130,), 1.0),
                                                     (0, 64, 4, 4, (16, 33), 1.0), (0, 128, 4, 4, (37, 45), 0.25), (2, 64, 8, 2, (70, 17, 2), 0.5)])
def test_attention_of_prompt_chunks(mode, hd, nh, nkv, chunks, fs, monkeypatch):
    """Prompt chunks through pi_k_attn_chunk (RoPE + KV store of the whole chunk, then causal attention of every token over the cache)
    against the oracle's rope + attention: the route on the matrix cores (16 tokens per workgroup; chunk lengths on and off that
    tile, caches filled by earlier chunks, grouped query heads) and the one-token-per-workgroup route, which must agree with
    each other more closely than either has to agree with the CPU.  fs = linear RoPE scaling (freq_scale)."""
    from powerinfer_amd import lib as pl
    L = pl.init()
    O = ol.oracle()
    rng = np.random.default_rng(mode + hd + sum(chunks))
    n_ctx, gqa, d = 160, nkv * hd, nh * hd
    kc_o = np.zeros((n_ctx, gqa), np.uint16)
    vc_o = np.zeros((gqa, n_ctx), np.uint16)
    theta_scale = float(np.float32(10000.0) ** np.float32(-2.0 / hd))
    caches = {r: (pl.DevBuf.zeros(nkv * n_ctx * hd * 2), pl.DevBuf.zeros(nkv * n_ctx * hd * 2)) for r in ("mfma", "scalar")}
    for kc, vc in caches.values():                                    # cells never written must not leak into a result
        pl.check(L.pi_memset(kc.ptr, 0x7E, kc.nbytes), "memset")      # 0x7E7E is a NaN pattern in fp16
        pl.check(L.pi_memset(vc.ptr, 0x7E, vc.nbytes), "memset")
    n_past = 0
    for T in chunks:
        qkv = rng.standard_normal((T, d + 2 * gqa)).astype(np.float32)
        q, k, v = (np.ascontiguousarray(a) for a in (qkv[:, :d], qkv[:, d:d + gqa], qkv[:, d + gqa:]))
        pos = np.arange(n_past, n_past + T, dtype=np.int32)
        qr, kr = np.zeros_like(q), np.zeros_like(k)
        O.pio_rope(P(q), hd, nh, T, P(pos), hd, mode, 10000.0, fs, P(qr))
        O.pio_rope(P(k), hd, nkv, T, P(pos), hd, mode, 10000.0, fs, P(kr))
        n_kv = (n_past + T + 31) // 32 * 32
        mask = np.where(np.arange(n_kv)[None, :] > pos[:, None], -np.inf, 0).astype(np.float32)
        want = np.zeros((T, d), np.float32)
        assert O.pio_attention(hd, nh, nkv, n_ctx, n_kv, T, P(pos), P(mask), P(qr), P(kr), P(v), P(kc_o), P(vc_o), P(want)) == 0
        dq, dpos = pl.DevBuf(host=qkv), pl.DevBuf(host=pos)
        got = {}
        for route, (kc, vc) in caches.items():
            if route == "scalar":
                monkeypatch.setenv("PI_ATTN_CHUNK", "scalar")
            else:
                monkeypatch.delenv("PI_ATTN_CHUNK", raising=False)
            dqr, dout, dout16 = pl.DevBuf(T * d * 4), pl.DevBuf(T * d * 4), pl.DevBuf(T * d * 2)
            pl.check(L.pi_memset(dout.ptr, 0xFF, dout.nbytes), "memset")
            # the scores in LDS are sized for the cells the chunk attends (mfma) or for the whole cache (n_kv_max 0)
            pl.check(L.pi_k_attn_chunk(dq.ptr, d + 2 * gqa, T, nh, nkv, hd, mode, theta_scale, fs, dpos.ptr, n_ctx, n_past + T if route == "mfma" else 0,
                                       dqr.ptr, kc.ptr, vc.ptr, dout.ptr, d, dout16.ptr, None), "attn_chunk")
            pl.sync()
            got[route] = dout.download(np.float32).reshape(T, d)
            assert np.array_equal(dout16.download(np.float16).reshape(T, d), got[route].astype(np.float16))
            assert rel_err(got[route], want) < 2e-3, (route, T, rel_err(got[route], want))
        # the scores are summed in another order, so here and there fp16(s - max) lands on the neighbouring value and one p moves by a unit
        assert rel_err(got["mfma"], got["scalar"]) < 5e-4, rel_err(got["mfma"], got["scalar"])
        assert not np.array_equal(got["mfma"], got["scalar"])         # two routes, two summation orders
        n_past += T
    monkeypatch.delenv("PI_ATTN_CHUNK", raising=False)
    # which kernel a chunk gets depends on the cells it attends, not on the size of the cache
    assert L.pi_k_attn_chunk_supported(128, 32768, 0) == 0 and L.pi_k_attn_chunk_supported(128, 32768, 1800) == 1
    assert L.pi_k_attn_chunk_supported(128, 32768, 2400) == 0 and L.pi_k_attn_chunk_supported(128, 8192, 2400) == 1      # one token per workgroup


@pytest.mark.parametrize("mode,hd,nh,nkv,fs", [(0, 128, 4, 4, 1.0), (2, 64, 8, 2, 1.0), (0, 128, 4, 4, 0.25), (2, 64, 8, 2, 0.5)])
def test_rope_attention_sequence(mode, hd, nh, nkv, fs):
    """Six decode steps: RoPE + KV store + attention on the GPU against the oracle's rope + attention with
    the reference cache layout (K cell-major, V transposed).  fs = linear RoPE scaling (the oracle's rope is pinned against the
    compiled reference for fs != 1 too, NeoX mode's double product included)."""
    from powerinfer_amd import lib as pl
    L = pl.init()
    O = ol.oracle()
    rng = np.random.default_rng(mode + hd)
    n_ctx, gqa, d = 48, nkv * hd, nh * hd
    kc_o = np.zeros((n_ctx, gqa), np.uint16)
    vc_o = np.zeros((gqa, n_ctx), np.uint16)
    kc_g, vc_g = pl.DevBuf.zeros(nkv * n_ctx * hd * 2), pl.DevBuf.zeros(nkv * n_ctx * hd * 2)
    dq, dpos, dqr, dout = pl.DevBuf((d + 2 * gqa) * 4), pl.DevBuf(4), pl.DevBuf(d * 4), pl.DevBuf(d * 4)
    theta_scale = float(np.float32(10000.0) ** np.float32(-2.0 / hd))
    kc_f, vc_f = pl.DevBuf.zeros(nkv * n_ctx * hd * 2), pl.DevBuf.zeros(nkv * n_ctx * hd * 2)
    tab, dout_f = pl.DevBuf(n_ctx * hd * 4), pl.DevBuf(d * 4)
    pl.check(L.pi_k_rope_table(tab.ptr, n_ctx, hd, mode, theta_scale, fs, None), "rope_table")
    for pos in range(6):
        qkv = rng.standard_normal(d + 2 * gqa).astype(np.float32)
        q, k, v = qkv[:d], qkv[d:d + gqa], qkv[d + gqa:]
        p = np.array([pos], np.int32)
        qr, kr = np.zeros_like(q), np.zeros_like(k)
        O.pio_rope(P(q), hd, nh, 1, P(p), hd, mode, 10000.0, fs, P(qr))
        O.pio_rope(P(k), hd, nkv, 1, P(p), hd, mode, 10000.0, fs, P(kr))
        n_kv = max(32, pos + 1)
        mask = np.where(np.arange(n_kv)[None, :] > pos, -np.inf, 0).astype(np.float32)
        want = np.zeros(d, np.float32)
        assert O.pio_attention(hd, nh, nkv, n_ctx, n_kv, 1, P(p), P(mask), P(qr), P(kr), P(np.ascontiguousarray(v)), P(kc_o), P(vc_o), P(want)) == 0
        dq.upload(qkv)
        dpos.upload(p)
        pl.check(L.pi_k_rope_kv_store(dq.ptr, nh, nkv, hd, mode, theta_scale, fs, dpos.ptr, n_ctx, dqr.ptr, kc_g.ptr, vc_g.ptr, None), "rope")
        pl.check(L.pi_k_attn_decode(dqr.ptr, kc_g.ptr, vc_g.ptr, nh, nkv, hd, n_ctx, dpos.ptr, dout.ptr, None), "attn")
        pl.check(L.pi_k_attn_fused(dq.ptr, tab.ptr, kc_f.ptr, vc_f.ptr, nh, nkv, hd, mode, n_ctx, dpos.ptr, dout_f.ptr, None), "attn_fused")
        pl.sync()
        assert rel_err(dqr.download(np.float32), qr) < 1e-6
        got = dout.download(np.float32)
        assert rel_err(got, want) < 2e-3, (pos, rel_err(got, want))
        got_f = dout_f.download(np.float32)     # fused launch: same arithmetic; cos/sin come from a table kernel and
        assert rel_err(got_f, want) < 2e-3      # may differ from the inline ones in the last place before the fp16 rounding
        assert rel_err(got_f, got) < 1e-3
    # the caches hold the same fp16 values, in this library's [kv_head][cell][hd] layout
    kg = kc_g.download(np.uint16).reshape(nkv, n_ctx, hd)
    vg = vc_g.download(np.uint16).reshape(nkv, n_ctx, hd)
    ko = kc_o.reshape(n_ctx, nkv, hd).transpose(1, 0, 2)
    vo = vc_o.reshape(nkv, hd, n_ctx).transpose(0, 2, 1)
    assert (kg[:, :6] != ko[:, :6]).mean() < 2e-3          # cos/sin may differ in the last place before rounding
    assert np.array_equal(vg[:, :6], vo[:, :6])
    assert (kc_f.download(np.uint16) != kc_g.download(np.uint16)).mean() < 1e-3
    assert np.array_equal(vc_f.download(np.uint16), vc_g.download(np.uint16))


@pytest.mark.parametrize("mode,hd,nh,nkv", [(0, 128, 4, 4), (2, 64, 8, 2)])
def test_attention_long_context(mode, hd, nh, nkv):
    """One decode step over a cache that already holds several hundred cells: the fused kernel requests the K and V rows of its
    first four passes (256 cells at head size 128, 512 at 64) before its prologue and takes the rest in a loop; positions on both
    sides of that boundary are compared with the oracle, as is the two-launch form."""
    from powerinfer_amd import lib as pl
    L = pl.init()
    O = ol.oracle()
    rng = np.random.default_rng(3 * mode + hd)
    n_ctx, gqa, d = 768, nkv * hd, nh * hd
    theta_scale = float(np.float32(10000.0) ** np.float32(-2.0 / hd))
    tab = pl.DevBuf(n_ctx * hd * 4)
    pl.check(L.pi_k_rope_table(tab.ptr, n_ctx, hd, mode, theta_scale, 1.0, None), "rope_table")
    kfill = (rng.standard_normal((n_ctx, nkv, hd)) * 0.5).astype(np.float16)        # cell-major, as the oracle keeps K
    vfill = (rng.standard_normal((n_ctx, nkv, hd)) * 0.5).astype(np.float16)
    boundary = 4 * (1024 // (hd // 8))
    for pos in (boundary - 1, boundary, boundary + 1, boundary + 45, 700):
        kc_o = np.ascontiguousarray(kfill.reshape(n_ctx, gqa)).view(np.uint16).copy()
        vc_o = np.ascontiguousarray(vfill.reshape(n_ctx, gqa).T).view(np.uint16).copy()
        kg = np.ascontiguousarray(kfill.transpose(1, 0, 2))
        vg = np.ascontiguousarray(vfill.transpose(1, 0, 2))
        qkv = rng.standard_normal(d + 2 * gqa).astype(np.float32)
        q, k, v = qkv[:d], qkv[d:d + gqa], qkv[d + gqa:]
        p = np.array([pos], np.int32)
        qr, kr = np.zeros_like(q), np.zeros_like(k)
        O.pio_rope(P(q), hd, nh, 1, P(p), hd, mode, 10000.0, 1.0, P(qr))
        O.pio_rope(P(k), hd, nkv, 1, P(p), hd, mode, 10000.0, 1.0, P(kr))
        n_kv = pos + 1
        mask = np.zeros((1, n_kv), np.float32)
        want = np.zeros(d, np.float32)
        assert O.pio_attention(hd, nh, nkv, n_ctx, n_kv, 1, P(p), P(mask), P(qr), P(kr), P(np.ascontiguousarray(v)), P(kc_o), P(vc_o), P(want)) == 0
        dq, dpos = pl.DevBuf(host=qkv), pl.DevBuf(host=p)
        for fused in (True, False):
            kc, vc, dout, dqr = pl.DevBuf(host=kg), pl.DevBuf(host=vg), pl.DevBuf(d * 4), pl.DevBuf(d * 4)
            if fused:
                pl.check(L.pi_k_attn_fused(dq.ptr, tab.ptr, kc.ptr, vc.ptr, nh, nkv, hd, mode, n_ctx, dpos.ptr, dout.ptr, None), "attn_fused")
            else:
                pl.check(L.pi_k_rope_kv_store(dq.ptr, nh, nkv, hd, mode, theta_scale, 1.0, dpos.ptr, n_ctx, dqr.ptr, kc.ptr, vc.ptr, None), "rope")
                pl.check(L.pi_k_attn_decode(dqr.ptr, kc.ptr, vc.ptr, nh, nkv, hd, n_ctx, dpos.ptr, dout.ptr, None), "attn")
            pl.sync()
            assert rel_err(dout.download(np.float32), want) < 2e-3, (pos, fused)
            # only the new cell was written
            after = kc.download(np.float16).reshape(nkv, n_ctx, hd)
            untouched = np.ones(n_ctx, bool); untouched[pos] = False
            assert np.array_equal(after[:, untouched], kg[:, untouched])


@pytest.mark.parametrize("mode,hd,nh,nkv,n_ctx,parts", [(0, 128, 4, 4, 8192, 8), (2, 64, 8, 2, 32768, 4), (0, 128, 2, 1, 32768, 16)])
def test_attention_split_over_cells(mode, hd, nh, nkv, n_ctx, parts):
    """pi_k_attn_split: the cells of every head divided among `parts` workgroups and merged by a second launch, at contexts of 8 k and 32 k
    cells that one workgroup's LDS cannot hold.  Positions with fewer cells than parts (empty parts), around the prefetch boundary of a
    part and at the end of the context are compared with the oracle; where the single-workgroup kernel can run, the two agree to the
    last places of the fp16 roundings; and only the new cell is written.  The chunk form (K / V already stored, q already rotated)
    must return the same numbers as the decode form."""
    from powerinfer_amd import lib as pl
    L = pl.init()
    O = ol.oracle()
    rng = np.random.default_rng(7 * mode + hd + parts)
    gqa, d = nkv * hd, nh * hd
    assert L.pi_k_attn_split_supported(hd, n_ctx, parts) == 1 and L.pi_k_attn_fused_supported(hd, n_ctx) == 0
    theta_scale = float(np.float32(10000.0) ** np.float32(-2.0 / hd))
    tab = pl.DevBuf(n_ctx * hd * 4)
    pl.check(L.pi_k_rope_table(tab.ptr, n_ctx, hd, mode, theta_scale, 1.0, None), "rope_table")
    kfill = (rng.standard_normal((n_ctx, nkv, hd)) * 0.5).astype(np.float16)
    vfill = (rng.standard_normal((n_ctx, nkv, hd)) * 0.5).astype(np.float16)
    kg = np.ascontiguousarray(kfill.transpose(1, 0, 2))
    vg = np.ascontiguousarray(vfill.transpose(1, 0, 2))
    kc_o = np.ascontiguousarray(kfill.reshape(n_ctx, gqa)).view(np.uint16)
    vc_o = np.ascontiguousarray(vfill.reshape(n_ctx, gqa).T).view(np.uint16)
    scratch = pl.DevBuf(4 * L.pi_k_attn_split_scratch_floats(1, nh, hd, parts))
    per_pass = 512 // (hd // 8)
    for pos in (0, 1, parts - 1, parts + 3, 4 * per_pass * parts - 1, 4 * per_pass * parts + 77, 5000, n_ctx - 1):
        qkv = rng.standard_normal(d + 2 * gqa).astype(np.float32)
        q, k, v = qkv[:d], qkv[d:d + gqa], qkv[d + gqa:]
        p = np.array([pos], np.int32)
        qr, kr = np.zeros_like(q), np.zeros_like(k)
        O.pio_rope(P(q), hd, nh, 1, P(p), hd, mode, 10000.0, 1.0, P(qr))
        O.pio_rope(P(k), hd, nkv, 1, P(p), hd, mode, 10000.0, 1.0, P(kr))
        n_kv = pos + 1
        mask = np.zeros((1, n_kv), np.float32)
        want = np.zeros(d, np.float32)
        ko, vo = kc_o.copy(), vc_o.copy()
        assert O.pio_attention(hd, nh, nkv, n_ctx, n_kv, 1, P(p), P(mask), P(qr), P(kr), P(np.ascontiguousarray(v)), P(ko), P(vo), P(want)) == 0
        dq, dpos = pl.DevBuf(host=qkv), pl.DevBuf(host=p)
        kc, vc, dout = pl.DevBuf(host=kg), pl.DevBuf(host=vg), pl.DevBuf(d * 4)
        pl.check(L.pi_k_attn_split(dq.ptr, 0, tab.ptr, kc.ptr, vc.ptr, 0, 1, nh, nkv, hd, mode, n_ctx, parts, dpos.ptr, scratch.ptr, dout.ptr, 0, None, None), "attn_split")
        pl.sync()
        got = dout.download(np.float32)
        assert rel_err(got, want) < 2e-3, (pos, rel_err(got, want))
        after_k = kc.download(np.float16).reshape(nkv, n_ctx, hd)
        untouched = np.ones(n_ctx, bool); untouched[pos] = False
        assert np.array_equal(after_k[:, untouched], kg[:, untouched])
        assert np.array_equal(vc.download(np.float16).reshape(nkv, n_ctx, hd)[:, untouched], vg[:, untouched])
        # the chunk form on the cache the decode form left behind (the new cell is in it now)
        dqr, dout2 = pl.DevBuf(host=qr), pl.DevBuf(d * 4)
        pl.check(L.pi_k_attn_split_cached(dqr.ptr, kc.ptr, vc.ptr, 1, nh, nkv, hd, n_ctx, parts, dpos.ptr, scratch.ptr, dout2.ptr, None), "attn_split_cached")
        pl.sync()
        assert rel_err(dout2.download(np.float32), got) < 1e-5, pos
    # against the single-workgroup kernel, at a context both can run
    n_small = 2048
    tab2 = pl.DevBuf(n_small * hd * 4)
    pl.check(L.pi_k_rope_table(tab2.ptr, n_small, hd, mode, theta_scale, 1.0, None), "rope_table")
    kg2, vg2 = np.ascontiguousarray(kg[:, :n_small]), np.ascontiguousarray(vg[:, :n_small])
    for pos in (5, 700, n_small - 1):
        qkv = rng.standard_normal(d + 2 * gqa).astype(np.float32)
        dq, dpos = pl.DevBuf(host=qkv), pl.DevBuf(host=np.array([pos], np.int32))
        outs = []
        for split in (False, True):
            kc, vc, dout = pl.DevBuf(host=kg2), pl.DevBuf(host=vg2), pl.DevBuf(d * 4)
            if split:
                pl.check(L.pi_k_attn_split(dq.ptr, 0, tab2.ptr, kc.ptr, vc.ptr, 0, 1, nh, nkv, hd, mode, n_small, parts, dpos.ptr, scratch.ptr, dout.ptr, 0, None, None), "attn_split")
            else:
                pl.check(L.pi_k_attn_fused(dq.ptr, tab2.ptr, kc.ptr, vc.ptr, nh, nkv, hd, mode, n_small, dpos.ptr, dout.ptr, None), "attn_fused")
            pl.sync()
            outs.append(dout.download(np.float32))
        # each part rounds its exp arguments to fp16 relative to its own maximum, the single workgroup relative to the global one:
        # the two differ by those roundings (a few 2^-11 of a score), no more
        assert rel_err(outs[1], outs[0]) < 1.5e-3, (pos, rel_err(outs[1], outs[0]))
    assert L.pi_k_attn_split_supported(hd, n_ctx, 65) == 0 and L.pi_k_attn_split_supported(24, n_ctx, parts) == 0


@pytest.mark.parametrize("cols,kind", [(4096, 1), (5120, 0), (8192, 2)])
def test_gemv_of_three_matrices_in_one_launch(cols, kind):
    """pi_k_gemv_multi_f16: the q, k and v projections of a host that keeps them as three tensors, one launch against one normalised
    vector.  Every product is bit for bit the one pi_k_gemv computes for that matrix alone."""
    import ctypes as C
    from powerinfer_amd import lib as pl
    L = pl.init()
    rng = np.random.default_rng(cols + kind)
    rows = [cols, 1024, 520]
    Ws = [pl.DevBuf(host=(rng.standard_normal((r, cols)) * 0.02).astype(np.float16)) for r in rows]
    x = pl.DevBuf(host=rng.standard_normal(cols).astype(np.float32))
    nw = pl.DevBuf(host=(1 + 0.1 * rng.standard_normal(cols)).astype(np.float32)) if kind else None
    nb = pl.DevBuf(host=(0.1 * rng.standard_normal(cols)).astype(np.float32)) if kind == 2 else None
    nrm = pl.norm_arg(kind, 1e-5, nw, nb) if kind else None
    ys = [pl.DevBuf(r * 4) for r in rows]
    pl.check(L.pi_k_gemv_multi_f16((C.c_void_p * 3)(*[w.ptr for w in Ws]), (C.c_int * 3)(*rows), 3, cols, x.ptr, nrm, (C.c_void_p * 3)(*[y.ptr for y in ys]), None), "gemv_multi")
    pl.sync()
    for W, r, y in zip(Ws, rows, ys):
        one = pl.DevBuf(r * 4)
        pl.check(L.pi_k_gemv(pl.F16, W.ptr, r, cols, x.ptr, nrm, 0, None, None, one.ptr, None), "gemv")
        pl.sync()
        assert np.array_equal(y.download(np.float32), one.download(np.float32))
    assert L.pi_k_gemv_multi_f16((C.c_void_p * 3)(*[w.ptr for w in Ws]), (C.c_int * 3)(*rows), 3, 4000, x.ptr, nrm, (C.c_void_p * 3)(*[y.ptr for y in ys]), None) != 0


@pytest.mark.parametrize("mode,hd,nh,nkv", [(0, 128, 4, 4), (2, 64, 8, 2)])
def test_attention_on_the_reference_cache_layouts(mode, hd, nh, nkv):
    """pi_k_attn_ggml: one token's attention with K cells [cell][n_embd_gqa] and V transposed [n_embd_gqa][n_ctx], as the reference's
    llm_build_kv_store / llm_build_kqv lay the cache out, RoPE and both cache stores included.  Forty tokens one after the other
    against the oracle's rope + attention on the same layouts: outputs within 2e-3, the two caches identical up to the last bit of
    the rotated K values; cells are handed out in a scrambled order and hidden cells carry -inf in the mask, as a ring with holes does;
    the number of attended cells passes through values that are no multiple of 8."""
    from powerinfer_amd import lib as pl
    L = pl.init()
    O = ol.oracle()
    rng = np.random.default_rng(mode + hd)
    n_ctx, gqa, d = 64, nkv * hd, nh * hd
    assert L.pi_k_attn_ggml_supported(hd, n_ctx, 33) == 1 and L.pi_k_attn_ggml_supported(hd, 63, 33) == 0
    kc_o, vc_o = np.zeros((n_ctx, gqa), np.uint16), np.zeros((gqa, n_ctx), np.uint16)
    kc, vc = pl.DevBuf.zeros(n_ctx * gqa * 2), pl.DevBuf.zeros(n_ctx * gqa * 2)
    theta_scale = float(np.float32(10000.0) ** np.float32(-2.0 / hd))
    scale = pl.DevBuf(host=np.array([1.0 / np.sqrt(hd)], np.float32))
    cells = rng.permutation(40)                                  # token t lives in cell cells[t]
    used = np.zeros(n_ctx, bool)
    for t in range(40):
        cell = int(cells[t])
        used[cell] = True
        n_kv = max(int(np.flatnonzero(used).max()) + 1, 5)       # cells up to the highest one in use are attended, the unused ones masked
        q, k, v = (rng.standard_normal(n).astype(np.float32) for n in (d, gqa, gqa))
        pos = np.array([t], np.int32)
        mask = np.where(used[:n_kv], 0.0, -np.inf).astype(np.float32)
        qr, kr = np.zeros_like(q), np.zeros_like(k)
        O.pio_rope(P(q), hd, nh, 1, P(pos), hd, mode, 10000.0, 1.0, P(qr))
        O.pio_rope(P(k), hd, nkv, 1, P(pos), hd, mode, 10000.0, 1.0, P(kr))
        want = np.zeros(d, np.float32)
        slot = np.array([cell], np.int32)
        assert O.pio_attention(hd, nh, nkv, n_ctx, n_kv, 1, P(slot), P(mask), P(qr), P(kr), P(v), P(kc_o), P(vc_o), P(want)) == 0
        dq, dk, dv, dpos, dmask, dout = pl.DevBuf(host=q), pl.DevBuf(host=k), pl.DevBuf(host=v), pl.DevBuf(host=pos), pl.DevBuf(host=mask), pl.DevBuf(d * 4)
        pl.check(L.pi_k_attn_ggml(dq.ptr, dk.ptr, dv.ptr, dpos.ptr, mode, theta_scale, 1.0, 1.0, kc.ptr, vc.ptr, nh, nkv, hd, n_ctx, n_kv, cell,
                                  scale.ptr, dmask.ptr, dout.ptr, None), "attn_ggml")
        pl.sync()
        assert rel_err(dout.download(np.float32), want) < 2e-3, (t, rel_err(dout.download(np.float32), want))
    kg = kc.download(np.float16).reshape(n_ctx, gqa).astype(np.float32)
    vg = vc.download(np.uint16).reshape(gqa, n_ctx)
    assert np.array_equal(vg, vc_o)
    assert np.abs(kg - kc_o.view(np.float16).astype(np.float32)).max() <= 2e-3 * np.abs(kg).max()


@pytest.mark.parametrize("mode,hd,nh,nkv,T", [(0, 128, 4, 4, 16), (2, 64, 8, 2, 5), (0, 128, 8, 8, 1)])
def test_attention_of_a_step_on_the_reference_cache_layouts(mode, hd, nh, nkv, T):
    """pi_k_attn_ggml_step: T tokens whose rows go to a run of consecutive cells, each under its own mask row, in one launch, against
    the oracle's llm_build_kv_store + llm_build_kqv for the same batch (which stores every token's rows before anyone attends).
    Three steps into a cache that already holds cells: tokens of two interleaved sequences (a token does not see the other
    sequence's cells, old or new), causal inside the step, and in the last step the tokens come in descending positions, so that a
    token attends rows of tokens behind it in the batch."""
    from powerinfer_amd import lib as pl
    L = pl.init()
    O = ol.oracle()
    rng = np.random.default_rng(mode + hd + T)
    n_ctx, gqa, d = 96, nkv * hd, nh * hd
    stride = d + 2 * gqa + 8                                     # tokens' [q | k | v] rows with a gap between them
    kc_o, vc_o = np.zeros((n_ctx, gqa), np.uint16), np.zeros((gqa, n_ctx), np.uint16)
    kc, vc = pl.DevBuf.zeros(n_ctx * gqa * 2), pl.DevBuf.zeros(n_ctx * gqa * 2)
    theta_scale = float(np.float32(10000.0) ** np.float32(-2.0 / hd))
    scale = pl.DevBuf(host=np.array([1.0 / np.sqrt(hd)], np.float32))
    cell_seq, cell_pos = np.full(n_ctx, -1), np.full(n_ctx, -1)
    next_pos = [0, 0]
    cell0 = 3                                                    # the first run does not start at cell 0
    for step in range(3):
        seqs = rng.integers(0, 2, T)
        pos = np.zeros(T, np.int32)
        for t in range(T):
            pos[t] = next_pos[seqs[t]]
            next_pos[seqs[t]] += 1
        if step == 2:
            seqs, pos = seqs[::-1].copy(), pos[::-1].copy()
        cell_seq[cell0:cell0 + T], cell_pos[cell0:cell0 + T] = seqs, pos
        n_kv = cell0 + T + (3 if step == 1 else 0)               # a range that is no multiple of 8 and reaches past the cells in use
        mask = np.zeros((T, n_kv), np.float32)
        for t in range(T):
            hidden = (cell_seq[:n_kv] != seqs[t]) | (cell_pos[:n_kv] > pos[t]) | (cell_pos[:n_kv] < 0)
            mask[t, hidden] = -np.inf
        qkv = rng.standard_normal((T, stride)).astype(np.float32)
        q, k, v = (np.ascontiguousarray(qkv[:, a:b]) for a, b in ((0, d), (d, d + gqa), (d + gqa, d + 2 * gqa)))
        qr, kr = np.zeros_like(q), np.zeros_like(k)
        O.pio_rope(P(q), hd, nh, T, P(pos), hd, mode, 10000.0, 1.0, P(qr))
        O.pio_rope(P(k), hd, nkv, T, P(pos), hd, mode, 10000.0, 1.0, P(kr))
        want = np.zeros((T, d), np.float32)
        slots = np.arange(cell0, cell0 + T, dtype=np.int32)
        assert O.pio_attention(hd, nh, nkv, n_ctx, n_kv, T, P(slots), P(mask), P(qr), P(kr), P(v), P(kc_o), P(vc_o), P(want)) == 0
        dqkv, dpos, dmask, dout = pl.DevBuf(host=qkv), pl.DevBuf(host=pos), pl.DevBuf(host=mask), pl.DevBuf(T * (d + 4) * 4)
        pl.check(L.pi_k_attn_ggml_step(dqkv.ptr, stride, dpos.ptr, mode, theta_scale, 1.0, 1.0, kc.ptr, vc.ptr, nh, nkv, hd, n_ctx, n_kv, T, cell0,
                                       scale.ptr, dmask.ptr, n_kv, dout.ptr, d + 4, None), "attn_ggml_step")
        pl.sync()
        got = dout.download(np.float32).reshape(T, d + 4)[:, :d]
        for t in range(T):
            assert rel_err(got[t], want[t]) < 2e-3, (step, t, rel_err(got[t], want[t]))
        cell0 += T + (2 if step == 0 else 0)                     # a hole of two free cells behind the first run
    vg = vc.download(np.uint16).reshape(gqa, n_ctx)
    assert np.array_equal(vg, vc_o)
    kg = kc.download(np.float16).reshape(n_ctx, gqa).astype(np.float32)
    assert np.abs(kg - kc_o.view(np.float16).astype(np.float32)).max() <= 2e-3 * np.abs(kg).max()
    assert L.pi_k_attn_ggml_step(dqkv.ptr, stride, dpos.ptr, mode, theta_scale, 1.0, 1.0, kc.ptr, vc.ptr, nh, nkv, hd, n_ctx, 40, 17, 0,
                                 scale.ptr, dmask.ptr, 40, dout.ptr, d + 4, None) != 0                   # more than 16 tokens


@pytest.mark.parametrize("mode,fs", [(0, 1.0), (2, 0.5)])
def test_k_shift_on_the_reference_cache_layout(mode, fs):
    """pi_k_k_shift_cells rotates K cells laid out [layer][cell][kv head][hd] (the view llm_build_k_shift rotates): the same data
    permuted into [layer * kv head][cell][hd] and sent through pi_k_k_shift, which test_k_shift_and_compaction holds to the
    reference's fp16 RoPE, must come out bit for bit the same; cells with delta 0 keep their bits."""
    from powerinfer_amd import lib as pl
    L = pl.init()
    n_layer, n_cells, nkv, hd = 3, 40, 2, 64
    rng = np.random.default_rng(3 + mode)
    k = rng.standard_normal((n_layer, n_cells, nkv, hd)).astype(np.float16)
    delta = rng.integers(-9, 10, n_cells).astype(np.int32)
    delta[::3] = 0
    theta_scale = float(np.float32(10000.0) ** np.float32(-2.0 / hd))
    ka = pl.DevBuf(host=k)
    kb = pl.DevBuf(host=np.ascontiguousarray(k.transpose(0, 2, 1, 3)))          # [layer][kv head][cell][hd]
    dd = pl.DevBuf(host=delta)
    pl.check(L.pi_k_k_shift_cells(ka.ptr, n_layer, n_cells, nkv, hd, mode, theta_scale, fs, dd.ptr, None), "k_shift_cells")
    pl.check(L.pi_k_k_shift(kb.ptr, n_layer * nkv, n_cells, hd, mode, theta_scale, fs, dd.ptr, n_cells, None), "k_shift")
    pl.sync()
    got = ka.download(np.float16).reshape(n_layer, n_cells, nkv, hd)
    want = kb.download(np.float16).reshape(n_layer, nkv, n_cells, hd).transpose(0, 2, 1, 3)
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))
    assert np.array_equal(got[:, delta == 0].view(np.uint16), k[:, delta == 0].view(np.uint16))
    assert not np.array_equal(got[:, delta != 0].view(np.uint16), k[:, delta != 0].view(np.uint16))


def test_embed_and_argmax():
    from powerinfer_amd import lib as pl
    L = pl.init()
    rng = np.random.default_rng(0)
    tab32 = (rng.standard_normal((100, 256)) * 0.02).astype(np.float32)
    for wt in (ol.F16, ol.Q4_0):
        tab = synth.encode(tab32, wt)
        dt, dtok, dx = pl.DevBuf(host=tab), pl.DevBuf(host=np.array([37], np.int32)), pl.DevBuf(256 * 4)
        pl.check(L.pi_k_embed(wt, dt.ptr, 256, dtok.ptr, dx.ptr, None), "embed")
        pl.sync()
        want = tab[37].astype(np.float32) if wt == ol.F16 else synth.dequantize_q4_0(tab[37:38], 256)[0]
        assert np.array_equal(dx.download(np.float32), want)
    lg = rng.standard_normal(32000).astype(np.float32)
    lg[[123, 20000]] = lg.max() + 1          # tie: the first index wins
    dl, dtok = pl.DevBuf(host=lg), pl.DevBuf(4)
    pl.check(L.pi_k_argmax(dl.ptr, 32000, dtok.ptr, None), "argmax")
    pl.sync()
    assert dtok.download(np.int32)[0] == 123 == int(np.argmax(lg))


@pytest.mark.parametrize("mode,fs", [(0, 1.0), (2, 1.0), (0, 0.5), (2, 0.5)])
def test_k_shift_and_compaction(mode, fs):
    """pi_k_k_shift against the fp16 RoPE of the reference's K-shift restated in numpy (ggml.c:11327-11478: fp16 in, fp32
    rotation with theta advanced by repeated multiplication, fp16 out), and pi_k_kv_compact against a gather.  With linear
    scaling (fs) the model-level fixtures written by the compiled reference are the check proper (tests/test_gpu_model_golden.py);
    here the kernel is held to the same restatement."""
    from powerinfer_amd import lib as pl
    L = pl.init()
    rows, n_ctx, hd, n_cells = 6, 40, 64, 33
    rng = np.random.default_rng(11)
    k = rng.standard_normal((rows, n_ctx, hd)).astype(np.float16)
    delta = rng.integers(-9, 10, n_cells).astype(np.int32)
    delta[::4] = 0
    theta_scale = np.float32(10000.0) ** np.float32(-2.0 / hd)
    want = k.copy()
    for c in range(n_cells):
        if delta[c] == 0:
            continue
        th = np.float32(delta[c])
        if mode == 2:
            th = np.float32(th * np.float32(fs))
        for i in range(hd // 2):
            ang = np.float32(np.float32(fs) * th)
            cs, sn = np.float32(np.cos(ang)), np.float32(np.sin(ang))
            i0, i1 = (i, i + hd // 2) if mode == 2 else (2 * i, 2 * i + 1)
            x0, x1 = k[:, c, i0].astype(np.float32), k[:, c, i1].astype(np.float32)
            want[:, c, i0] = (x0 * cs - x1 * sn).astype(np.float16)
            want[:, c, i1] = (x0 * sn + x1 * cs).astype(np.float16)
            th = np.float32(th * theta_scale)
    kd, dd = pl.DevBuf(host=k), pl.DevBuf(host=delta)
    pl.check(L.pi_k_k_shift(kd.ptr, rows, n_ctx, hd, mode, float(theta_scale), fs, dd.ptr, n_cells, None), "k_shift")
    pl.sync()
    got = kd.download(np.float16).reshape(rows, n_ctx, hd)
    assert np.array_equal(got[:, n_cells:], k[:, n_cells:])                       # cells beyond the live range untouched
    assert np.array_equal(got[:, :n_cells][:, delta == 0], k[:, :n_cells][:, delta == 0])
    diff = np.abs(got.astype(np.float32) - want.astype(np.float32))
    assert diff.max() <= 2e-3 * np.abs(want.astype(np.float32)).max()             # cosf/sinf of the device vs numpy: a last-place fp16 step
    assert (got != want).mean() < 0.02
    # compaction: drop cells 3..8 and 20
    keep = np.array([c for c in range(n_cells) if not (3 <= c < 9 or c == 20)], np.int32)
    stage, md = pl.DevBuf(rows * n_ctx * hd * 2), pl.DevBuf(host=keep)
    pl.check(L.pi_k_kv_compact(kd.ptr, stage.ptr, rows, n_ctx, hd, md.ptr, keep.size, None), "kv_compact")
    pl.sync()
    after = kd.download(np.float16).reshape(rows, n_ctx, hd)
    assert np.array_equal(after[:, :keep.size], got[:, keep])


def test_host_signal_and_bounded_wait():
    """The hand-over kernels between the stream and host threads: a signal publishes the hand-over count in pinned memory once the
    work before it is complete; a wait returns when the host's word has reached that count, and gives up after its limit (here a
    millisecond, with a host that never answers) by recording the failure, after which later waits return at once - the stream
    always drains."""
    import ctypes as C
    import time
    from powerinfer_amd import lib as pl
    L = pl.init()
    fp = L.pi_malloc_host(64 * 4)
    assert fp
    flags = np.frombuffer((C.c_char * 256).from_address(fp), dtype=np.uint32)
    flags[...] = 0
    seq, status = pl.DevBuf.zeros(4), pl.DevBuf.zeros(4)
    try:
        pl.check(L.pi_k_host_signal(seq.ptr, fp, 0, 1, None), "signal")
        pl.sync()
        assert int(flags[0]) == 1 and int(flags[8]) == 0 and int(seq.download(np.uint32)[0]) == 1
        flags[16] = 1                                           # the host has already answered hand-over 1
        pl.check(L.pi_k_host_signal_wait(seq.ptr, fp, 8, 16, status.ptr, 5.0, None), "signal_wait")       # the second signal travels with the wait
        pl.sync()
        assert int(status.download(np.uint32)[0]) == 0 and int(flags[8]) == 1
        pl.check(L.pi_k_host_wait(seq.ptr, fp, 32, status.ptr, 5.0, None), "wait")      # answered while the kernel polls
        time.sleep(0.05)
        flags[32] = 1
        pl.sync()
        assert int(status.download(np.uint32)[0]) == 0
        pl.check(L.pi_k_host_signal(seq.ptr, fp, 0, 1, None), "signal")                 # hand-over 2, never answered
        t0 = time.time()
        pl.check(L.pi_k_host_wait(seq.ptr, fp, 16, status.ptr, 1e-3, None), "wait")
        pl.sync()
        assert int(status.download(np.uint32)[0]) == 1 and int(flags[0]) == 2
        pl.check(L.pi_k_host_wait(seq.ptr, fp, 32, status.ptr, 30.0, None), "wait")     # returns at once: the status word is set
        pl.sync()
        assert time.time() - t0 < 5.0
        assert L.pi_k_host_wait(seq.ptr, fp, 7, status.ptr, 1.0, None) != 0
        assert L.pi_k_host_signal_wait(seq.ptr, fp, 16, 32, status.ptr, 1.0, None) != 0                    # word 16 is the host's
        assert L.pi_k_host_wait(seq.ptr, fp, 16, status.ptr, 1e9, None) != 0
    finally:
        pl.sync()
        del flags
        L.pi_free_host(fp)
