"""Batched decode step kernels (T <= 16 tokens, one per sequence) through the C ABI against the CPU oracle:
dense mat-mul on the matrix cores, and the sparse FFN over the union of the tokens' active sets."""
import numpy as np
import pytest

import oracle_lib as ol
from oracle_lib import _ptr as P
from powerinfer_amd import synth

pytestmark = pytest.mark.gpu


def rel_err(a, b):
    return float(np.abs(a - b).max() / max(np.abs(b).max(), 1e-30))


def gpu_norm_round(pl, L, x, norm=None):
    T, cols = x.shape
    dx, dn = pl.DevBuf(host=np.ascontiguousarray(x, np.float32)), pl.DevBuf(T * cols * 2)
    keep, na = [], None
    if norm is not None:
        kind, eps, nw, nb = norm
        bw = pl.DevBuf(host=nw) if nw is not None else None
        bb = pl.DevBuf(host=nb) if nb is not None else None
        keep += [bw, bb]
        na = pl.norm_arg(kind, eps, bw, bb)
    pl.check(L.pi_k_norm_round_f16(dx.ptr, T, cols, na, dn.ptr, None, None), "norm_round")
    pl.sync()
    return dn


@pytest.mark.parametrize("rows,cols,T", [(3000, 5120, 16), (4096, 4096, 7), (13824, 1280, 16), (70, 128, 1)])
def test_gemm_matches_oracle(rows, cols, T):
    from powerinfer_amd import lib as pl
    L = pl.init()
    rng = np.random.default_rng(rows + cols + T)
    w = (rng.standard_normal((rows, cols)) * 0.02).astype(np.float16)
    x = rng.standard_normal((T, cols)).astype(np.float32)
    a1 = rng.standard_normal((T, rows)).astype(np.float32)
    want = np.zeros((T, rows), np.float32)
    assert ol.oracle().pio_mul_mat(ol.F16, P(w), rows, cols, P(x), T, P(want), 8) == 0
    dn = gpu_norm_round(pl, L, x)
    assert np.array_equal(dn.download(np.float16).reshape(T, cols), x.astype(np.float16))
    dw, dy, d1 = pl.DevBuf(host=w), pl.DevBuf(T * rows * 4), pl.DevBuf(host=a1)
    pl.check(L.pi_k_gemm_f16(dw.ptr, rows, cols, dn.ptr, T, pl.EPI_NONE, None, None, dy.ptr, None, None), "gemm")
    pl.sync()
    got = dy.download(np.float32).reshape(T, rows)
    assert rel_err(got, want) < 5e-6
    pl.check(L.pi_k_gemm_f16(dw.ptr, rows, cols, dn.ptr, T, pl.EPI_ADD, d1.ptr, None, dy.ptr, None, None), "gemm")
    pl.sync()
    assert rel_err(dy.download(np.float32).reshape(T, rows), want + a1) < 5e-6
    dy16 = pl.DevBuf(T * rows * 2)
    pl.check(L.pi_k_gemm_f16(dw.ptr, rows, cols, dn.ptr, T, pl.EPI_RELU, None, None, dy.ptr, dy16.ptr, None), "gemm")
    pl.sync()
    got = dy.download(np.float32).reshape(T, rows)
    assert rel_err(got, np.maximum(want, 0)) < 5e-6
    assert np.array_equal(dy16.download(np.float16).reshape(T, rows), got.astype(np.float16))


@pytest.mark.parametrize("tile", [0, 256128, 192128, 128128, 96128, 128064, 64128, 64064])
@pytest.mark.parametrize("rows,cols,T", [(3000, 5120, 300), (4104, 4096, 512), (1024, 11008, 130), (520, 512, 17), (64, 64, 1), (130, 192, 129),
                                         (2048, 1024, 40), (12288, 4096, 512)])
def test_gemm_tile_matches_oracle(rows, cols, T, tile):
    """This library's LDS-tiled mat-mul of prompt chunks against the reference's CPU mat-mul on the same fp16-rounded activations, on
    every output tile it is built for and on the one the library picks: token and row counts on and off the tile sizes (a single
    token, one past a tile, 512 tokens), a reduction dimension of one stage and of 172, every epilogue, the fp16 copy, and the
    transposition that feeds the down projection."""
    from powerinfer_amd import lib as pl
    L = pl.init()
    rng = np.random.default_rng(rows + cols + T)
    w = (rng.standard_normal((rows, cols)) * 0.02).astype(np.float16)
    x = rng.standard_normal((T, cols)).astype(np.float32)
    a1, a2 = rng.standard_normal((T, rows)).astype(np.float32), rng.standard_normal((T, rows)).astype(np.float32)
    want = np.zeros((T, rows), np.float32)
    assert ol.oracle().pio_mul_mat(ol.F16, P(w), rows, cols, P(x), T, P(want), 8) == 0
    dn = gpu_norm_round(pl, L, x)
    dw, dy, d1, d2 = pl.DevBuf(host=w), pl.DevBuf(T * rows * 4), pl.DevBuf(host=a1), pl.DevBuf(host=a2)
    pl.check(L.pi_memset(dy.ptr, 0xFF, dy.nbytes), "memset")
    pl.check(L.pi_k_gemm_tile_f16(dw.ptr, rows, cols, dn.ptr, T, pl.EPI_NONE, None, None, dy.ptr, None, tile, None), "gemm_tile")
    pl.sync()
    got = dy.download(np.float32).reshape(T, rows)
    assert rel_err(got, want) < 5e-6
    pl.check(L.pi_k_gemm_tile_f16(dw.ptr, rows, cols, dn.ptr, T, pl.EPI_ADD, d1.ptr, None, dy.ptr, None, tile, None), "gemm_tile")
    pl.sync()
    assert rel_err(dy.download(np.float32).reshape(T, rows), want + a1) < 5e-6
    pl.check(L.pi_k_gemm_tile_f16(dw.ptr, rows, cols, dn.ptr, T, pl.EPI_ADD2, d1.ptr, d2.ptr, dy.ptr, None, tile, None), "gemm_tile")
    pl.sync()
    assert rel_err(dy.download(np.float32).reshape(T, rows), (want + a1) + a2) < 5e-6
    dy16 = pl.DevBuf(T * rows * 2)
    pl.check(L.pi_k_gemm_tile_f16(dw.ptr, rows, cols, dn.ptr, T, pl.EPI_RELU, None, None, dy.ptr, dy16.ptr, tile, None), "gemm_tile")
    pl.sync()
    got = dy.download(np.float32).reshape(T, rows)
    assert rel_err(got, np.maximum(want, 0)) < 5e-6
    assert np.array_equal(dy16.download(np.float16).reshape(T, rows), got.astype(np.float16))
    if tile == 0:
        dt = pl.DevBuf(rows * cols * 2)
        pl.check(L.pi_k_transpose_f16(dw.ptr, rows, cols, dt.ptr, None), "transpose")
        pl.sync()
        assert np.array_equal(dt.download(np.float16).reshape(cols, rows), w.T)
        assert L.pi_k_gemm_tile_f16(dw.ptr, rows, cols, dn.ptr, T, pl.EPI_NONE, None, None, dy.ptr, None, 32032, None) != 0        # no such tile
        assert L.pi_k_gemm_tile_f16(dw.ptr, rows, cols - 8, dn.ptr, T, pl.EPI_NONE, None, None, dy.ptr, None, 0, None) != 0       # cols % 64
        assert L.pi_k_gemm_tile_f16(dw.ptr, rows, cols, dn.ptr, T, pl.EPI_ADD, None, None, dy.ptr, None, 0, None) != 0            # residual missing


@pytest.mark.parametrize("rows,cols,T", [(3000, 5120, 300), (4104, 4096, 512), (1024, 11008, 130), (520, 512, 17), (12288, 4096, 512)])
def test_gemm_lib_matches_oracle(rows, cols, T):
    """The library mat-mul of long prompt chunks (hipBLASLt plans, fp16 operands, fp32 accumulation) against the reference's CPU
    mat-mul on the same fp16-rounded activations: token and row counts on and off round numbers, the FFN-wide reduction, every
    epilogue (a residual as the C operand, the second residual / ReLU / fp16 copy in the pass behind it), a plan used twice."""
    from powerinfer_amd import lib as pl
    L = pl.init()
    rng = np.random.default_rng(rows + cols + T)
    w = (rng.standard_normal((rows, cols)) * 0.02).astype(np.float16)
    x = rng.standard_normal((T, cols)).astype(np.float32)
    a1, a2 = rng.standard_normal((T, rows)).astype(np.float32), rng.standard_normal((T, rows)).astype(np.float32)
    want = np.zeros((T, rows), np.float32)
    assert ol.oracle().pio_mul_mat(ol.F16, P(w), rows, cols, P(x), T, P(want), 8) == 0
    g = L.pi_gemm_lib_create(32 << 20)
    assert g, L.pi_last_error()
    dn = gpu_norm_round(pl, L, x)
    dw, dy, d1, d2 = pl.DevBuf(host=w), pl.DevBuf(T * rows * 4), pl.DevBuf(host=a1), pl.DevBuf(host=a2)
    for _ in range(2):
        pl.check(L.pi_memset(dy.ptr, 0xFF, dy.nbytes), "memset")
        pl.check(L.pi_gemm_lib_f16(g, dw.ptr, rows, cols, dn.ptr, T, pl.EPI_NONE, None, None, dy.ptr, None, None), "gemm_lib")
        pl.sync()
        assert rel_err(dy.download(np.float32).reshape(T, rows), want) < 2e-5
    pl.check(L.pi_gemm_lib_f16(g, dw.ptr, rows, cols, dn.ptr, T, pl.EPI_ADD, d1.ptr, None, dy.ptr, None, None), "gemm_lib")
    pl.sync()
    assert rel_err(dy.download(np.float32).reshape(T, rows), want + a1) < 2e-5
    pl.check(L.pi_gemm_lib_f16(g, dw.ptr, rows, cols, dn.ptr, T, pl.EPI_ADD2, d1.ptr, d2.ptr, dy.ptr, None, None), "gemm_lib")
    pl.sync()
    assert rel_err(dy.download(np.float32).reshape(T, rows), (want + a1) + a2) < 2e-5
    dy16 = pl.DevBuf(T * rows * 2)
    pl.check(L.pi_gemm_lib_f16(g, dw.ptr, rows, cols, dn.ptr, T, pl.EPI_RELU, None, None, dy.ptr, dy16.ptr, None), "gemm_lib")
    pl.sync()
    got = dy.download(np.float32).reshape(T, rows)
    assert rel_err(got, np.maximum(want, 0)) < 2e-5
    assert np.array_equal(dy16.download(np.float16).reshape(T, rows), got.astype(np.float16))
    assert L.pi_gemm_lib_f16(g, dw.ptr, rows, cols, dn.ptr, T, pl.EPI_ADD, None, None, dy.ptr, None, None) != 0      # residual missing
    pl.check(L.pi_gemm_lib_destroy(g), "destroy")


def test_ffn_h_from_dense_products():
    from powerinfer_amd import lib as pl
    L = pl.init()
    rng = np.random.default_rng(4)
    T, ff = 37, 1024
    up, gate, lg = (rng.standard_normal((T, ff)).astype(np.float32) for _ in range(3))
    du, dg, dl, dh = pl.DevBuf(host=up), pl.DevBuf(host=gate), pl.DevBuf(host=lg), pl.DevBuf(T * ff * 2)
    for g_ptr, want in ((dg.ptr, np.where(lg >= 0.1, np.maximum(gate, 0) * up, 0)), (None, np.where(lg >= 0.1, np.maximum(up, 0), 0))):
        pl.check(L.pi_k_ffn_h_f16(du.ptr, g_ptr, dl.ptr, 0.1, T, ff, dh.ptr, None), "ffn_h")
        pl.sync()
        assert np.array_equal(dh.download(np.float16).reshape(T, ff), want.astype(np.float32).astype(np.float16))


@pytest.mark.parametrize("kind", [1, 2])
def test_norm_round_matches_oracle(kind):
    from powerinfer_amd import lib as pl
    L = pl.init()
    rng = np.random.default_rng(kind)
    T, cols = 5, 5120
    x = (rng.standard_normal((T, cols)) * 2 + 0.3).astype(np.float32)
    nw = (1 + 0.1 * rng.standard_normal(cols)).astype(np.float32)
    nb = (0.1 * rng.standard_normal(cols)).astype(np.float32) if kind == 2 else None
    O = ol.oracle()
    xn = np.zeros_like(x)
    (O.pio_rms_norm if kind == 1 else O.pio_norm)(P(x), cols, T, 1e-5, P(xn))
    xn = xn * nw + (nb if nb is not None else 0)
    got = gpu_norm_round(pl, L, x, norm=(kind, 1e-5, nw, nb)).download(np.float16).reshape(T, cols).astype(np.float32)
    want = xn.astype(np.float32).astype(np.float16).astype(np.float32)
    # identical up to fp16 rounding ties on a handful of elements
    assert (got != want).mean() < 1e-3
    assert rel_err(got, want) < 1e-3


def q8_values(x):
    """What the CPU path's Q8_0 blocks keep of the rows of x (quantize_row_q8_0, ggml-quants.c:702-760): q * fp16(amax / 127) as float32."""
    O = ol.oracle()
    x = np.ascontiguousarray(x, np.float32)
    blocks = np.zeros(x.size // 32 * 34, np.uint8)
    O.pio_quantize_row_q8_0(P(x), P(blocks), x.size)
    blocks = blocks.reshape(-1, 34)
    d = blocks[:, :2].copy().view(np.float16).astype(np.float32)
    q = blocks[:, 2:].copy().view(np.int8).astype(np.float32)
    return (q * d).reshape(x.shape)


@pytest.mark.parametrize("kind,cols", [(0, 4096), (1, 4096), (2, 8192), (1, 1280)])
def test_norm_q8_round_matches_oracle(kind, cols):
    """The chunk input of a Q4_0 mat-mul: the normalised row as the values its Q8_0 blocks keep, then fp16.  Against the oracle's norm
    followed by the oracle's quantize_row_q8_0; the norm's last-bit differences move a handful of quantised values by one step."""
    from powerinfer_amd import lib as pl
    L = pl.init()
    rng = np.random.default_rng(10 + kind)
    T = 7
    x = (rng.standard_normal((T, cols)) * 2 + 0.3).astype(np.float32)
    nw = (1 + 0.1 * rng.standard_normal(cols)).astype(np.float32) if kind else None
    nb = (0.1 * rng.standard_normal(cols)).astype(np.float32) if kind == 2 else None
    O = ol.oracle()
    xn = x.copy()
    if kind:
        (O.pio_rms_norm if kind == 1 else O.pio_norm)(P(x), cols, T, 1e-5, P(xn))
        xn = (xn * nw + (nb if nb is not None else 0)).astype(np.float32)
    want = q8_values(xn).astype(np.float16).astype(np.float32)
    dx, dn, dp = pl.DevBuf(host=x), pl.DevBuf(T * cols * 2), pl.DevBuf(T * cols * 2)
    bw = pl.DevBuf(host=nw) if nw is not None else None
    bb = pl.DevBuf(host=nb) if nb is not None else None
    pl.check(L.pi_k_norm_q8_round_f16(dx.ptr, T, cols, pl.norm_arg(kind, 1e-5, bw, bb), dn.ptr, dp.ptr, None), "norm_q8_round")
    pl.sync()
    got = dn.download(np.float16).reshape(T, cols).astype(np.float32)
    assert np.array_equal(dp.download(np.float16).reshape(T, cols), x.astype(np.float16))
    if kind == 0:
        assert np.array_equal(got, want)
    else:
        assert (got != want).mean() < 2e-3
        step = np.abs(xn).reshape(T, -1, 32).max(-1, keepdims=True) / 127
        assert (np.abs(got - want).reshape(T, -1, 32) <= 1.01 * step + 1e-7).all()
    assert L.pi_k_norm_q8_round_f16(dx.ptr, T, cols - 16, pl.norm_arg(0, 0.0, None, None), dn.ptr, None, None) != 0


def test_ffn_h_q8_from_dense_products():
    """h of a prompt chunk for a Q4_0 down projection: masked relu(gate) * up through Q8_0 blocks of 32 neurons (ggml.c:14465-14618), then fp16."""
    from powerinfer_amd import lib as pl
    L = pl.init()
    rng = np.random.default_rng(5)
    T, ff = 19, 2048
    up, gate, lg = (rng.standard_normal((T, ff)).astype(np.float32) for _ in range(3))
    du, dg, dl, dh = pl.DevBuf(host=up), pl.DevBuf(host=gate), pl.DevBuf(host=lg), pl.DevBuf(T * ff * 2)
    for g_ptr, h in ((dg.ptr, np.where(lg >= 0.1, np.maximum(gate, 0) * up, 0)), (None, np.where(lg >= 0.1, np.maximum(up, 0), 0))):
        pl.check(L.pi_k_ffn_h_q8_f16(du.ptr, g_ptr, dl.ptr, 0.1, T, ff, dh.ptr, None), "ffn_h_q8")
        pl.sync()
        want = q8_values(h.astype(np.float32)).astype(np.float16)
        assert np.array_equal(dh.download(np.float16).reshape(T, ff), want)


@pytest.mark.parametrize("hot_frac", [1.0, 0.6, 0.0])
def test_chunk_weights_as_fp16(hot_frac):
    """A Q4_0 matrix expanded for a chunk's mat-mul ((q - 8) * d, dequantize_row_q4_0, rounded to fp16) and an fp16 matrix of a hybrid
    layer, both assembled from the compact matrix of the resident neurons and the rows of the others; the Q4_0 embedding rows of a chunk."""
    from powerinfer_amd import lib as pl
    L = pl.init()
    rng = np.random.default_rng(6)
    rows, cols = 1024, 640
    w = (rng.standard_normal((rows, cols)) * 0.02).astype(np.float32)
    wq = synth.quantize_q4_0(w)
    O = ol.oracle()
    deq = np.zeros((rows, cols), np.float32)
    O.pio_dequantize_row_q4_0(P(wq), P(deq), rows * cols)
    out = pl.DevBuf(rows * cols * 2)
    if hot_frac == 1.0:
        dw = pl.DevBuf(host=wq)
        pl.check(L.pi_k_dequant_q4_f16(dw.ptr, None, None, None, rows, cols, out.ptr, None), "dequant")
        pl.sync()
        assert np.array_equal(out.download(np.float16).reshape(rows, cols), deq.astype(np.float16))
        toks = rng.integers(0, rows, 33).astype(np.int32)
        dt, dx = pl.DevBuf(host=toks), pl.DevBuf(33 * cols * 4)
        pl.check(L.pi_k_embed_batch_q4(dw.ptr, cols, dt.ptr, 33, dx.ptr, None), "embed_batch_q4")
        pl.sync()
        assert np.array_equal(dx.download(np.float32).reshape(33, cols), deq[toks])
        return
    p = rng.random(rows)
    gid, bucket = synth.gpu_split(p, hot_frac)
    rest = np.flatnonzero(gid != 1)
    words = np.zeros(rows // 32, np.uint32)
    for j in bucket:
        words[j >> 5] |= np.uint32(1) << np.uint32(j & 31)
    prefix = np.concatenate([[0], np.cumsum([bin(int(v)).count("1") for v in words])[:-1]]).astype(np.int32)
    dwords, dprefix = pl.DevBuf(host=words), pl.DevBuf(host=prefix)
    pad = lambda a: a if a.size else np.zeros((1,) + a.shape[1:], a.dtype)  # noqa: E731
    hot_q, rest_q = pl.DevBuf(host=pad(wq[bucket])), pl.DevBuf(host=pad(wq[rest]))
    pl.check(L.pi_k_dequant_q4_f16(hot_q.ptr, rest_q.ptr, dwords.ptr, dprefix.ptr, rows, cols, out.ptr, None), "dequant split")
    pl.sync()
    assert np.array_equal(out.download(np.float16).reshape(rows, cols), deq.astype(np.float16))
    w16 = w.astype(np.float16)
    hot_h, rest_h = pl.DevBuf(host=pad(w16[bucket])), pl.DevBuf(host=pad(w16[rest]))
    pl.check(L.pi_k_assemble_rows_f16(hot_h.ptr, rest_h.ptr, dwords.ptr, dprefix.ptr, rows, cols, out.ptr, None), "assemble")
    pl.sync()
    assert np.array_equal(out.download(np.float16).reshape(rows, cols), w16)


@pytest.mark.parametrize("shape,has_gate,T", [((5120, 13824, 1280), True, 16), ((4096, 11008, 1024), False, 5)])
def test_batch_sparse_ffn_matches_oracle(shape, has_gate, T):
    """Config 3's FFN block (13B shape, 16 tokens): each weight row of the union of active sets is read once."""
    from powerinfer_amd import lib as pl
    L = pl.init()
    d, ff, r = shape
    Lr = synth.make_ffn_layer(seed=31 + T, d=d, ff=ff, r=r, wtype=ol.F16, has_gate=has_gate, mean_rate=0.11, T=T)
    x = Lr["x"]
    O = ol.oracle()
    o = ol.ffn_sparse(O, d, ff, r, T, ol.F16, has_gate, Lr["up"], Lr["gate"], Lr["down_t"], Lr["fc1"], Lr["fc2"], x, x,
                      np.zeros(ff, np.int32), 0.0, nth=8)
    ws = L.pi_workspace_create(ff, d)
    assert ws
    up, down, fc1, fc2 = (pl.DevBuf(host=Lr[k]) for k in ("up", "down_t", "fc1", "fc2"))
    gate = pl.DevBuf(host=Lr["gate"]) if has_gate else None
    xn = gpu_norm_round(pl, L, x)
    hidden, hid16 = pl.DevBuf(T * r * 4), pl.DevBuf(T * r * 2)
    logits, out = pl.DevBuf(T * ff * 4), pl.DevBuf(T * d * 4)
    union, n_union = pl.DevBuf(ff * 4), pl.DevBuf.zeros(4)
    resid = np.random.default_rng(3).standard_normal((T, d)).astype(np.float32)
    dres = pl.DevBuf(host=resid)
    pl.check(L.pi_k_gemm_f16(fc1.ptr, r, d, xn.ptr, T, pl.EPI_RELU, None, None, hidden.ptr, hid16.ptr, None), "fc1")
    pl.check(L.pi_k_batch_predictor_fc2(fc2.ptr, ff, r, hid16.ptr, T, 0.0, logits.ptr, ws, None), "fc2")
    pl.check(L.pi_k_batch_sparse_ffn(logits.ptr, T, ff, 0.0, up.ptr, gate.ptr if gate else None, down.ptr, d, xn.ptr,
                                     pl.EPI_ADD, dres.ptr, None, out.ptr, union.ptr, n_union.ptr, ws, None), "batch ffn")
    pl.sync()
    lg = logits.download(np.float32).reshape(T, ff)
    assert rel_err(lg, o["logits"]) < 1e-4
    mask_g, mask_o = ~(lg < 0.0), ~(o["logits"] < 0.0)
    assert (mask_g == mask_o).mean() >= 0.999
    n = int(n_union.download(np.int32)[0])
    assert np.array_equal(union.download(np.int32, n), np.nonzero(mask_g.any(0))[0])      # ascending union list, bit-exact for this mask
    got = out.download(np.float32).reshape(T, d) - resid
    for t in range(T):                                         # the oracle under the GPU's own logits: compared for every token
        ou = ol.ffn_under_logits(O, d, ff, ol.F16, has_gate, Lr["up"], Lr["gate"], Lr["down_t"], x[t], lg[t], 0.0)
        assert rel_err(got[t], ou["out"]) < 2e-3
        assert rel_err(got[t], ou["out"]) < 1e-4
    L.pi_workspace_destroy(ws)


def from_operand_layout(buf, T, cols):
    """[cols / 8][16 token slots][8] fp16 -> [T][cols] (the layout pi_k_norm_round_f16_ol and pi_k_gemm_f16_ol write)."""
    return buf.download(np.float16, 16 * cols).reshape(cols // 8, 16, 8)[:, :T, :].transpose(1, 0, 2).reshape(T, cols)


@pytest.mark.parametrize("rows,cols,T", [(72, 128, 1), (520, 640, 7), (1032, 384, 16), (4096, 4096, 16), (3000, 5120, 9)])
def test_gemm_in_the_operand_layout_matches_the_token_major_one_bit_for_bit(rows, cols, T):
    """pi_k_gemm_f16_ol against pi_k_gemm_f16 on shapes of both kernels behind them (column counts that are and are not multiples of
    256), one token, a ragged last row tile, every epilogue, and the fp16 copy in either layout."""
    from powerinfer_amd import lib as pl
    L = pl.init()
    rng = np.random.default_rng(rows + T)
    w = (0.05 * rng.standard_normal((rows, cols))).astype(np.float16)
    x = rng.standard_normal((T, cols)).astype(np.float32)
    a1, a2 = rng.standard_normal((T, rows)).astype(np.float32), rng.standard_normal((T, rows)).astype(np.float32)
    dw, dx, d1, d2 = pl.DevBuf(host=w), pl.DevBuf(host=x), pl.DevBuf(host=a1), pl.DevBuf(host=a2)
    na = pl.norm_arg(0, 0.0, None, None)
    xn, xo = pl.DevBuf.zeros(T * cols * 2), pl.DevBuf.zeros(16 * cols * 2)
    pl.check(L.pi_k_norm_round_f16(dx.ptr, T, cols, na, xn.ptr, None, None), "norm")
    pl.check(L.pi_k_norm_round_f16_ol(dx.ptr, T, cols, na, xo.ptr, None, None), "norm ol")
    for epi, p1, p2 in ((pl.EPI_NONE, None, None), (pl.EPI_RELU, None, None), (pl.EPI_ADD, d1.ptr, None), (pl.EPI_ADD2, d1.ptr, d2.ptr)):
        y, y16 = pl.DevBuf(T * rows * 4), pl.DevBuf.zeros(T * rows * 2)
        yo, yo16 = pl.DevBuf(T * rows * 4), pl.DevBuf.zeros(16 * rows * 2)
        pl.check(L.pi_k_gemm_f16(dw.ptr, rows, cols, xn.ptr, T, epi, p1, p2, y.ptr, y16.ptr, None), "gemm")
        pl.check(L.pi_k_gemm_f16_ol(dw.ptr, rows, cols, xo.ptr, T, epi, p1, p2, yo.ptr, yo16.ptr, None), "gemm ol")
        pl.sync()
        assert np.array_equal(y.download(np.float32).view(np.uint32), yo.download(np.float32).view(np.uint32)), epi
        assert np.array_equal(y16.download(np.float16, T * rows).reshape(T, rows).view(np.uint16), from_operand_layout(yo16, T, rows).view(np.uint16)), epi
    assert np.abs(y.download(np.float32)).max() > 0
    assert L.pi_k_gemm_f16_ol(dw.ptr, rows - 4, cols, xo.ptr, T, pl.EPI_NONE, None, None, yo.ptr, yo16.ptr, None) != 0          # fp16 copy: rows % 8
    assert L.pi_k_norm_round_f16_ol(dx.ptr, 17, cols, na, xo.ptr, None, None) != 0                                               # 16 token slots


@pytest.mark.parametrize("shape,has_gate,T", [((5120, 13824, 1280), True, 16), ((4096, 11008, 1024), False, 5), ((1024, 1024, 128), True, 3)])
def test_operand_layout_entry_points_match_the_token_major_ones_bit_for_bit(shape, has_gate, T):
    """The *_ol entry points keep a step's fp16 activations in the operand layout of the matrix cores ([cols / 8][16][8]); only the
    addresses of the activation loads and stores differ, so the FFN block of a step - norm + rounding, predictor fc1 (with its fp16
    copy for fc2), fc2 and its flags, union list, gate / up, down projection - must give the same bits either way."""
    from powerinfer_amd import lib as pl
    L = pl.init()
    d, ff, r = shape
    Lr = synth.make_ffn_layer(seed=17 + T, d=d, ff=ff, r=r, wtype=ol.F16, has_gate=has_gate, mean_rate=0.11, T=T)
    x = Lr["x"]
    nw = (1.0 + 0.1 * np.random.default_rng(5).standard_normal(d)).astype(np.float32)
    dx, dw = pl.DevBuf(host=np.ascontiguousarray(x, np.float32)), pl.DevBuf(host=nw)
    na = pl.norm_arg(1, 1e-5, dw, None)
    up, down, fc1, fc2 = (pl.DevBuf(host=Lr[k]) for k in ("up", "down_t", "fc1", "fc2"))
    gate = pl.DevBuf(host=Lr["gate"]) if has_gate else None
    resid = np.random.default_rng(3).standard_normal((T, d)).astype(np.float32)
    dres = pl.DevBuf(host=resid)
    ws = L.pi_workspace_create(ff, d)
    assert ws
    got = {}
    for tag, sfx in (("plain", ""), ("ol", "_ol")):
        fn = lambda name: getattr(L, name + sfx)
        slots = 16 if sfx else T
        xn, xp = pl.DevBuf.zeros(slots * d * 2), pl.DevBuf.zeros(slots * d * 2)
        hidden, hid16 = pl.DevBuf(T * r * 4), pl.DevBuf.zeros(slots * r * 2)
        logits, out = pl.DevBuf(T * ff * 4), pl.DevBuf(T * d * 4)
        union, n_union = pl.DevBuf(ff * 4), pl.DevBuf.zeros(4)
        pl.check(fn("pi_k_norm_round_f16")(dx.ptr, T, d, na, xn.ptr, xp.ptr, None), "norm")
        pl.check(fn("pi_k_gemm_f16")(fc1.ptr, r, d, xp.ptr, T, pl.EPI_RELU, None, None, hidden.ptr, hid16.ptr, None), "fc1")
        pl.check(fn("pi_k_batch_predictor_fc2")(fc2.ptr, ff, r, hid16.ptr, T, 0.0, logits.ptr, ws, None), "fc2")
        pl.check(fn("pi_k_batch_sparse_ffn")(logits.ptr, T, ff, 0.0, up.ptr, gate.ptr if gate else None, down.ptr, d, xn.ptr,
                                             pl.EPI_ADD, dres.ptr, None, out.ptr, union.ptr, n_union.ptr, ws, None), "ffn")
        pl.sync()
        n = int(n_union.download(np.int32)[0])
        unpack = (lambda b, c: from_operand_layout(b, T, c)) if sfx else (lambda b, c: b.download(np.float16, T * c).reshape(T, c))
        got[tag] = dict(xn=unpack(xn, d), xp=unpack(xp, d), hid16=unpack(hid16, r), hidden=hidden.download(np.float32), logits=logits.download(np.float32),
                        out=out.download(np.float32), union=union.download(np.int32, n))
    assert len(got["plain"]["union"]) > 0 and np.abs(got["plain"]["out"] - resid.ravel()).max() > 0
    for k in got["plain"]:
        assert np.array_equal(got["plain"][k].view(np.uint8), got["ol"][k].view(np.uint8)), k
    L.pi_workspace_destroy(ws)


@pytest.mark.parametrize("nh,nkv,hd,n_seq", [(8, 8, 128, 5), (16, 2, 64, 16)])
def test_lockstep_attention_writes_the_same_fp16_copy_in_either_layout(nh, nkv, hd, n_seq):
    """pi_k_attn_fused_batch_ol differs from pi_k_attn_fused_batch only in where the fp16 copy of the output lands (the operand layout
    of the output projection's mat-mul): same fp32 output, same fp16 values, same cache rows, over three steps of n_seq sequences."""
    from powerinfer_amd import lib as pl
    L = pl.init()
    rng = np.random.default_rng(nh + n_seq)
    n_ctx, gqa, d = 32, nkv * hd, nh * hd
    stride = nkv * n_ctx * hd
    tab = pl.DevBuf(n_ctx * hd * 4)
    pl.check(L.pi_k_rope_table(tab.ptr, n_ctx, hd, 0, float(np.float32(10000.0) ** np.float32(-2.0 / hd)), 1.0, None), "rope_table")
    caches = {k: (pl.DevBuf.zeros(n_seq * stride * 2), pl.DevBuf.zeros(n_seq * stride * 2)) for k in ("plain", "ol")}
    dq, dpos = pl.DevBuf(n_seq * (d + 2 * gqa) * 4), pl.DevBuf(n_seq * 4)
    for step in range(3):
        dq.upload(rng.standard_normal(n_seq * (d + 2 * gqa)).astype(np.float32))
        dpos.upload(np.full(n_seq, step, np.int32))
        res = {}
        for tag, fn in (("plain", L.pi_k_attn_fused_batch), ("ol", L.pi_k_attn_fused_batch_ol)):
            out, out16 = pl.DevBuf(n_seq * d * 4), pl.DevBuf.zeros(16 * d * 2)
            kc, vc = caches[tag]
            pl.check(fn(dq.ptr, d + 2 * gqa, tab.ptr, kc.ptr, vc.ptr, stride, n_seq, nh, nkv, hd, 0, n_ctx, dpos.ptr, out.ptr, d, out16.ptr, None), tag)
            pl.sync()
            h = from_operand_layout(out16, n_seq, d) if tag == "ol" else out16.download(np.float16, n_seq * d).reshape(n_seq, d)
            res[tag] = (out.download(np.float32), h, kc.download(np.uint16), vc.download(np.uint16))
        for a, b in zip(res["plain"], res["ol"]):
            assert np.array_equal(a.view(np.uint8), b.view(np.uint8))
        assert np.abs(res["plain"][0]).max() > 0


@pytest.mark.parametrize("nh,nkv,hd,n_seq", [(8, 8, 128, 5), (16, 2, 64, 16)])
def test_lockstep_attention_writes_the_q8_blocks_of_its_output(nh, nkv, hd, n_seq):
    """pi_k_attn_fused_batch_q8 leaves the Q8_0 blocks of the attention output (operand layout of the integer mat-mul, scales,
    -8 * sums) that pi_k_norm_q8_blocks without a norm makes of the fp32 output of pi_k_attn_fused_batch: the same bytes, so the
    Q4_0 steps need no launch between the attention and the output projection."""
    import ctypes as C
    from powerinfer_amd import lib as pl
    L = pl.init()
    rng = np.random.default_rng(nh + n_seq + 1)
    n_ctx, gqa, d = 32, nkv * hd, nh * hd
    stride = nkv * n_ctx * hd
    tab = pl.DevBuf(n_ctx * hd * 4)
    pl.check(L.pi_k_rope_table(tab.ptr, n_ctx, hd, 0, float(np.float32(10000.0) ** np.float32(-2.0 / hd)), 1.0, None), "rope_table")
    caches = {k: (pl.DevBuf.zeros(n_seq * stride * 2), pl.DevBuf.zeros(n_seq * stride * 2)) for k in ("two", "one")}
    dq, dpos = pl.DevBuf(n_seq * (d + 2 * gqa) * 4), pl.DevBuf(n_seq * 4)
    na = pl.Norm(0, 0.0, None, None)
    for step in range(3):
        dq.upload(rng.standard_normal(n_seq * (d + 2 * gqa)).astype(np.float32))
        dpos.upload(np.full(n_seq, step, np.int32))
        res = {}
        for tag in ("two", "one"):
            out = pl.DevBuf(n_seq * d * 4)
            q, dd, ss = pl.DevBuf.zeros(16 * d), pl.DevBuf.zeros(d // 32 * 16 * 4), pl.DevBuf.zeros(d // 32 * 16 * 4)
            kc, vc = caches[tag]
            if tag == "two":
                pl.check(L.pi_k_attn_fused_batch(dq.ptr, d + 2 * gqa, tab.ptr, kc.ptr, vc.ptr, stride, n_seq, nh, nkv, hd, 0, n_ctx, dpos.ptr, out.ptr, d, None, None), tag)
                pl.check(L.pi_k_norm_q8_blocks(out.ptr, n_seq, d, C.byref(na), q.ptr, dd.ptr, ss.ptr, None, None), "q8 blocks")
            else:
                pl.check(L.pi_k_attn_fused_batch_q8(dq.ptr, d + 2 * gqa, tab.ptr, kc.ptr, vc.ptr, stride, n_seq, nh, nkv, hd, 0, n_ctx, dpos.ptr, out.ptr, d,
                                                    q.ptr, dd.ptr, ss.ptr, None), tag)
            pl.sync()
            # token slots behind n_seq are never written by either
            qv = q.download(np.uint8).reshape(d // 32, 4, 16, 8)[:, :, :n_seq]
            res[tag] = (out.download(np.float32).view(np.uint32), qv, dd.download(np.uint32).reshape(-1, 16)[:, :n_seq], ss.download(np.int32).reshape(-1, 16)[:, :n_seq])
        for a, b in zip(res["two"], res["one"]):
            assert np.array_equal(a, b)
        assert res["one"][1].any()


def q4_split_on_device(pl, L, wq4, rows, cols):
    dw = pl.DevBuf(host=wq4)
    qs, ds = pl.DevBuf(rows * cols // 2), pl.DevBuf(rows * cols // 32 * 2)
    pl.check(L.pi_k_q4_split(dw.ptr, rows, cols, qs.ptr, ds.ptr, None), "q4 split")
    return qs, ds


def q8_blocks_on_device(pl, L, x, norm=None):
    import ctypes as C
    T, cols = x.shape
    dx = pl.DevBuf(host=np.ascontiguousarray(x, np.float32))
    q, d, s = pl.DevBuf(16 * cols), pl.DevBuf(cols // 32 * 16 * 4), pl.DevBuf(cols // 32 * 16 * 4)
    keep, na = [], pl.Norm(0, 0.0, None, None)
    if norm is not None:
        kind, eps, nw, nb = norm
        bw = pl.DevBuf(host=nw) if nw is not None else None
        bb = pl.DevBuf(host=nb) if nb is not None else None
        keep += [bw, bb]
        na = pl.Norm(kind, eps, bw.ptr if bw else None, bb.ptr if bb else None)
    pl.check(L.pi_k_norm_q8_blocks(dx.ptr, T, cols, C.byref(na), q.ptr, d.ptr, s.ptr, None, None), "q8 blocks")
    pl.sync()
    return q, d, s


@pytest.mark.parametrize("rows,cols,T", [(64, 256, 1), (520, 512, 5), (4096, 4096, 16), (12288, 4096, 16), (32000, 4096, 7), (1030, 1024, 16), (5120, 5120, 16)])
def test_gemm_q4_t16_matches_oracle(rows, cols, T):
    """The Q4_0 mat-mul of a step of up to 16 tokens on integer matrix cores against the reference's CPU mat-mul (Q4_0 rows times
    the Q8_0 blocks of the activations): the block sums are exact integers on both sides, what differs is the order in which the
    128 scaled block sums of a row are added in fp32, hence 1e-5.  One and two row tiles per workgroup, a row count off the tile,
    a single token, the residual epilogue."""
    from powerinfer_amd import lib as pl
    L = pl.init()
    rng = np.random.default_rng(rows + cols + T)
    wq = synth.encode((rng.standard_normal((rows, cols)) * 0.02).astype(np.float32), ol.Q4_0)
    x = rng.standard_normal((T, cols)).astype(np.float32)
    a1 = rng.standard_normal((T, rows)).astype(np.float32)
    want = np.zeros((T, rows), np.float32)
    assert ol.oracle().pio_mul_mat(ol.Q4_0, P(wq), rows, cols, P(x), T, P(want), 8) == 0
    qs, ds = q4_split_on_device(pl, L, wq, rows, cols)
    q, d, s = q8_blocks_on_device(pl, L, x)
    y, d1 = pl.DevBuf(T * rows * 4), pl.DevBuf(host=a1)
    pl.check(L.pi_memset(y.ptr, 0xFF, y.nbytes), "memset")
    pl.check(L.pi_k_gemm_q4_t16(qs.ptr, ds.ptr, rows, cols, q.ptr, d.ptr, s.ptr, T, pl.EPI_NONE, None, None, y.ptr, None), "gemm q4")
    pl.sync()
    assert rel_err(y.download(np.float32).reshape(T, rows), want) < 1e-5
    pl.check(L.pi_k_gemm_q4_t16(qs.ptr, ds.ptr, rows, cols, q.ptr, d.ptr, s.ptr, T, pl.EPI_ADD, d1.ptr, None, y.ptr, None), "gemm q4")
    pl.sync()
    assert rel_err(y.download(np.float32).reshape(T, rows), want + a1) < 1e-5
    assert L.pi_k_gemm_q4_t16(qs.ptr, ds.ptr, rows, cols, q.ptr, d.ptr, s.ptr, 17, pl.EPI_NONE, None, None, y.ptr, None) != 0       # T > 16
    assert L.pi_k_gemm_q4_t16(qs.ptr, ds.ptr, rows, cols, q.ptr, d.ptr, s.ptr, T, pl.EPI_ADD, None, None, y.ptr, None) != 0         # residual missing


@pytest.mark.parametrize("kind", [1, 2])
def test_norm_q8_blocks_match_the_reference_quantiser(kind):
    """Norm + Q8_0 blocks of a step's rows against the oracle's norm followed by quantize_row_q8_0: quants and scales bit for bit,
    and the block sums the mat-mul subtracts."""
    from powerinfer_amd import lib as pl
    L = pl.init()
    O = ol.oracle()
    T, cols = 5, 4096
    rng = np.random.default_rng(kind)
    x = rng.standard_normal((T, cols)).astype(np.float32) * 3
    nw = (1 + 0.1 * rng.standard_normal(cols)).astype(np.float32)
    nb = (0.1 * rng.standard_normal(cols)).astype(np.float32) if kind == 2 else None
    q, d, s = q8_blocks_on_device(pl, L, x, (kind, 1e-5, nw, nb))
    normed = np.zeros_like(x)
    (O.pio_rms_norm if kind == 1 else O.pio_norm)(P(x), cols, T, 1e-5, P(normed))
    normed = normed * nw
    if nb is not None:
        normed = normed + nb
    normed = np.ascontiguousarray(normed, np.float32)
    blocks = np.zeros((T, cols // 32, 34), np.uint8)
    for t in range(T):
        O.pio_quantize_row_q8_0(P(normed[t]), P(blocks[t]), cols)
    want_d = blocks[:, :, :2].copy().view(np.float16).reshape(T, cols // 32).astype(np.float32)
    want_q = blocks[:, :, 2:].copy().view(np.int8).reshape(T, cols)
    # the quants sit in the integer MFMA's operand layout: [block][group g][token][8 bytes], the group's bytes being elements 4g .. 4g + 3
    # and 16 + 4g .. 16 + 4g + 3 of the block
    raw = q.download(np.int8).reshape(cols // 32, 4, 16, 2, 4)                # [blk][g][t][half][byte]
    got_q = raw.transpose(2, 0, 3, 1, 4).reshape(16, cols)[:T]               # [t][blk][half][g][byte] = element 16 * half + 4 * g + byte
    got_d = d.download(np.float32).reshape(cols // 32, 16).T[:T]
    got_s = s.download(np.int32).reshape(cols // 32, 16).T[:T]
    assert np.array_equal(got_d, want_d)
    assert (got_q != want_q).mean() < 1e-3           # a value on a rounding boundary after the norm's last bit
    assert np.array_equal(got_s, -8 * got_q.reshape(T, cols // 32, 32).astype(np.int32).sum(-1))


@pytest.mark.parametrize("shape,has_gate,T", [((4096, 11008, 1024), True, 16), ((4096, 11008, 1024), False, 5), ((1024, 1024, 128), True, 3)])
def test_batch_sparse_ffn_q4_matches_oracle(shape, has_gate, T):
    """The sparse FFN of a step on Q4_0 weights (7B shape, 16 tokens; a gate-less layer; a small one): union list, up/gate dots of the
    union rows on integer matrix cores, h under the predictor's mask, its Q8_0 values, and the down projection over the union rows
    on fp32 matrix cores, against the CPU kernels under the same logits (GGML_OP_MUL_MAT_SPARSE, GGML_OP_AXPY with Q4_0 rows)."""
    from powerinfer_amd import lib as pl
    L = pl.init()
    O = ol.oracle()
    d, ff, r = shape
    Lr = synth.make_ffn_layer(seed=31 + T, d=d, ff=ff, r=r, wtype=ol.Q4_0, has_gate=has_gate, mean_rate=0.11, T=T)
    x = Lr["x"]
    ws = L.pi_workspace_create(ff, d)
    assert ws
    fc1, fc2 = pl.DevBuf(host=Lr["fc1"]), pl.DevBuf(host=Lr["fc2"])
    upq, ups = q4_split_on_device(pl, L, Lr["up"], ff, d)
    dnq, dns = q4_split_on_device(pl, L, Lr["down_t"], ff, d)
    gq, gs = q4_split_on_device(pl, L, Lr["gate"], ff, d) if has_gate else (None, None)
    xn = gpu_norm_round(pl, L, x)
    q, dd, s = q8_blocks_on_device(pl, L, x)
    hidden, hid16 = pl.DevBuf(T * r * 4), pl.DevBuf(T * r * 2)
    logits, out = pl.DevBuf(T * ff * 4), pl.DevBuf(T * d * 4)
    union, n_union = pl.DevBuf(ff * 4), pl.DevBuf.zeros(4)
    h, hq = pl.DevBuf.zeros(16 * ff * 4), pl.DevBuf.zeros(16 * ff * 4)
    resid = np.random.default_rng(3).standard_normal((T, d)).astype(np.float32)
    dres = pl.DevBuf(host=resid)
    pl.check(L.pi_k_gemm_f16(fc1.ptr, r, d, xn.ptr, T, pl.EPI_RELU, None, None, hidden.ptr, hid16.ptr, None), "fc1")
    for rep in range(2):                                       # the second pass finds the first one's h in the scratch buffers
        pl.check(L.pi_k_batch_predictor_fc2(fc2.ptr, ff, r, hid16.ptr, T, 0.0, logits.ptr, ws, None), "fc2")
        pl.check(L.pi_k_batch_sparse_ffn_q4(logits.ptr, T, ff, 0.0, upq.ptr, ups.ptr, gq.ptr if gq else None, gs.ptr if gs else None, dnq.ptr, dns.ptr, d,
                                            q.ptr, dd.ptr, s.ptr, pl.EPI_ADD, dres.ptr, None, out.ptr, h.ptr, hq.ptr, union.ptr, n_union.ptr, ws, None), "ffn q4")
    pl.sync()
    lg = logits.download(np.float32).reshape(T, ff)
    n = int(n_union.download(np.int32)[0])
    assert np.array_equal(union.download(np.int32, n), np.nonzero((~(lg < 0.0)).any(0))[0])
    got = out.download(np.float32).reshape(T, d) - resid
    hh = h.download(np.float32).reshape(16, ff)
    for t in range(T):
        ou = ol.ffn_under_logits(O, d, ff, ol.Q4_0, has_gate, Lr["up"], Lr["gate"], Lr["down_t"], x[t], lg[t], 0.0)
        assert rel_err(np.where(~(lg[t] < 0.0), hh[t], 0), ou["h"]) < 1e-5
        assert rel_err(got[t], ou["out"]) < 1e-4
    L.pi_workspace_destroy(ws)


@pytest.mark.parametrize("thr,ff", [(1e9, 1024), (-1e9, 1024), (-1e9, 12288), (-1e9, 8200)])
def test_batch_sparse_ffn_none_and_all_active(thr, ff):
    """Empty union (zero output, residual only) and the full union (every row of every matrix read once: the dense FFN).  With
    12288 and 8200 union rows the gate / up kernel, one workgroup per compute unit with at most 32 rows at a time, walks more than
    one chunk per workgroup (the second shape: a last chunk of 8 rows, on some of the units only)."""
    from powerinfer_amd import lib as pl
    L = pl.init()
    d, r, T = 1024, 128, 3
    Lr = synth.make_ffn_layer(seed=5, d=d, ff=ff, r=r, wtype=ol.F16, has_gate=True, T=T)
    x = Lr["x"]
    o = ol.ffn_sparse(ol.oracle(), d, ff, r, T, ol.F16, True, Lr["up"], Lr["gate"], Lr["down_t"], Lr["fc1"], Lr["fc2"], x, x,
                      np.zeros(ff, np.int32), thr, nth=8)
    ws = L.pi_workspace_create(ff, d)
    up, gate, down, fc1, fc2 = (pl.DevBuf(host=Lr[k]) for k in ("up", "gate", "down_t", "fc1", "fc2"))
    xn = gpu_norm_round(pl, L, x)
    hidden, hid16 = pl.DevBuf(T * r * 4), pl.DevBuf(T * r * 2)
    logits, out = pl.DevBuf(T * ff * 4), pl.DevBuf(T * d * 4)
    union, n_union = pl.DevBuf(ff * 4), pl.DevBuf.zeros(4)
    pl.check(L.pi_k_gemm_f16(fc1.ptr, r, d, xn.ptr, T, pl.EPI_RELU, None, None, hidden.ptr, hid16.ptr, None), "fc1")
    pl.check(L.pi_k_batch_predictor_fc2(fc2.ptr, ff, r, hid16.ptr, T, thr, logits.ptr, ws, None), "fc2")
    pl.check(L.pi_k_batch_sparse_ffn(logits.ptr, T, ff, thr, up.ptr, gate.ptr, down.ptr, d, xn.ptr,
                                     pl.EPI_NONE, None, None, out.ptr, union.ptr, n_union.ptr, ws, None), "batch ffn")
    pl.sync()
    n = int(n_union.download(np.int32)[0])
    got = out.download(np.float32).reshape(T, d)
    if thr > 0:
        assert n == 0 and (got == 0).all()
    else:
        assert n == ff and np.array_equal(union.download(np.int32, n), np.arange(ff))
        assert rel_err(got, o["out"]) < 1e-4
    L.pi_workspace_destroy(ws)


@pytest.mark.parametrize("wtype", [synth.F16, synth.Q4_0], ids=["f16", "q4_0"])
@pytest.mark.parametrize("arch", ["llama-tiny", "falcon-tiny"])
def test_batched_decode_matches_per_sequence_oracle(arch, wtype):
    """Four sequences with different prompts advance in lockstep (examples/batched/batched.cpp).  Sequences do not interact,
    so sequence t of the batch must reproduce a single-sequence run on the same tokens: against the CPU oracle (teacher
    forced, the trajectory-level criteria of the single-sequence tests) and against this library's own batch-1 engine.
    A Q4_0 model steps on the integer matrix-core kernels (one MFMA per pair of a Q4_0 weight block and a Q8_0 activation block,
    the CPU path's arithmetic): same criteria on the median; single steps of a Q4_0 model may sit further out (the single-token
    path itself is up to 4e-2 from the oracle on these models: one int8 rounding step of an activation is a visible share of a dot
    product, tests/test_oracle_math.py::test_q4_reference_departs_from_itself_beyond_the_logit_tolerance), so they are held to 1e-1."""
    from powerinfer_amd.model import Model
    q4 = wtype != synth.F16
    hp = synth.hparams(arch, seed=5, n_ctx=64, wtype=wtype, **(dict(pred_margin=True, head_pair=2048) if q4 else {}))          # Q4_0: a margin model, so that no neuron flips on a rounding step
    model = synth.make_model(hp)
    n_seq, n_steps = 4, 10
    rng = np.random.default_rng(11)
    toks = rng.integers(0, hp.n_vocab, (n_steps, n_seq)).astype(np.int32)
    gm = Model(hp).load(model)
    gm.batch_init(n_seq)
    batch_logits = np.zeros((n_steps, n_seq, hp.n_vocab), np.float32)
    batch_next = np.zeros((n_steps, n_seq), np.int32)
    for s in range(n_steps):
        nxt, lg = gm.batch_decode(toks[s], np.full(n_seq, s, np.int32))
        batch_logits[s], batch_next[s] = lg, nxt
        assert np.array_equal(nxt, lg.argmax(1))
    assert np.all(gm.batch_union() > 0)
    errs_o, errs_g, same = [], [], 0
    for t in range(n_seq):
        om = ol.OracleModel(model)
        gm.kv_clear()
        for s in range(n_steps):
            tok_o, lg_o = om.eval([int(toks[s, t])], s)
            tok_g, lg_g = gm.decode([int(toks[s, t])], s)
            errs_o.append(rel_err(batch_logits[s, t], lg_o))
            errs_g.append(rel_err(batch_logits[s, t], lg_g))
            same += int(batch_next[s, t] == tok_o)
        om.close()
    errs_o, errs_g = np.array(errs_o), np.array(errs_g)
    assert np.median(errs_o) < 1e-2, errs_o
    assert np.median(errs_g) < 1e-2, errs_g
    assert not q4 or max(errs_o.max(), errs_g.max()) < 1e-1, (errs_o, errs_g)
    assert same >= 0.9 * n_seq * n_steps, same
    # greedy continuation on the device equals stepping the same state by hand
    gm2 = Model(hp).load(model)
    gm2.batch_init(n_seq)
    nxt, _ = gm2.batch_decode(toks[0], np.zeros(n_seq, np.int32))
    gen, _ = gm2.batch_generate(6)
    gm3 = Model(hp).load(model)
    gm3.batch_init(n_seq)
    cur, _ = gm3.batch_decode(toks[0], np.zeros(n_seq, np.int32))
    assert np.array_equal(cur, nxt)
    for s in range(6):
        cur, _ = gm3.batch_decode(cur, np.full(n_seq, s + 1, np.int32))
        assert np.array_equal(gen[s], cur), s
    for m in (gm, gm2, gm3):
        m.close()


@pytest.mark.parametrize("arch", ["llama-tiny", "falcon-tiny"])
def test_lockstep_decoding_crosses_over_to_dense_ffn(arch):
    """The dense cross-over of batched decoding: with an active set that covers 95 % of every layer the union of the sequences' rows
    is above a switch set to 90 % of n_ff, so from the second step on every layer computes its FFN as dense gate / up mat-muls, h under
    the predictor's mask, and a dense down mat-mul.  The first step has no statistic yet and runs the union kernels.  Both forms
    against the CPU oracle per sequence (margin-protected model: logits within 1e-2 at every step, identical greedy tokens), against
    each other (an engine that never switches), and through the captured graph, which is re-captured when the choice changes."""
    from powerinfer_amd.model import Model
    hp = synth.hparams(arch, seed=6, n_ctx=48, mean_rate=0.95, pred_margin=True, head_pair=2048)
    model = synth.make_model(hp)
    n_seq, n_steps = 4, 6
    toks = np.random.default_rng(3).integers(0, hp.n_vocab, (n_steps, n_seq)).astype(np.int32)
    auto, never, always = Model(hp).load(model), Model(hp).load(model), Model(hp).load(model)
    for g in (auto, never, always):
        g.batch_init(n_seq)
    auto.batch_set_dense_above(0.9)                                # (the library's default is never)
    never.batch_set_dense_above(1.0)
    always.batch_set_dense_above(0.0)
    assert auto.batch_dense_layers() == 0 and never.batch_dense_layers() == 0 and always.batch_dense_layers() == hp.n_layer
    oms = [ol.OracleModel(model) for _ in range(n_seq)]
    nxt = None
    for s in range(n_steps):
        pos = np.full(n_seq, s, np.int32)
        nxt, lg_a = auto.batch_decode(toks[s], pos)
        nxt_n, lg_n = never.batch_decode(toks[s], pos)
        nxt_d, lg_d = always.batch_decode(toks[s], pos)
        assert auto.batch_dense_layers() == hp.n_layer and never.batch_dense_layers() == 0          # the statistic of this step decides the next
        assert np.all(auto.batch_union() > 0.9 * hp.n_ff) and np.array_equal(auto.batch_union(), never.batch_union())
        for t in range(n_seq):
            tok_o, lg_o = oms[t].eval([int(toks[s, t])], s)
            for lg in (lg_a, lg_n, lg_d):
                assert rel_err(lg[t], lg_o) < 1e-2, (s, t, rel_err(lg[t], lg_o))
            assert int(nxt[t]) == tok_o and int(nxt_n[t]) == tok_o and int(nxt_d[t]) == tok_o, (s, t)
            assert rel_err(lg_d[t], lg_n[t]) < 2e-3
        if s >= 1:                                                  # `auto` runs what `always` runs now, on a cache whose first cell came from the union kernels
            assert rel_err(lg_a, lg_d) < 2e-3
    # free-running on the device: `auto` captures its graph with the dense layers, `never` with the union kernels; same tokens
    gen_a, _ = auto.batch_generate(5)
    gen_n, _ = never.batch_generate(5)
    assert np.array_equal(gen_a, gen_n)
    for t in range(n_seq):
        cur = int(nxt[t])
        for s in range(5):
            cur, _ = oms[t].eval([cur], n_steps + s)
            assert int(gen_a[s, t]) == cur, (t, s)
        oms[t].close()
    # the choice changes under a captured graph: the next call captures again and continues from the same state
    auto.batch_set_dense_above(1.0)
    assert auto.batch_dense_layers() == 0
    more_a, _ = auto.batch_generate(3)
    more_n, _ = never.batch_generate(3)
    assert np.array_equal(more_a, more_n)
    for g in (auto, never, always):
        g.close()


SEED_13B_MOVING = 53       # a seed whose sixteen greedy paths spread over all four marker tokens, keep their top-2 gaps, and never pass a step where both head pairs project near zero (the logit tolerance is relative to the largest logit)
SEED_7B_Q4_BATCH = 44       # the 7B-width Q4_0 lockstep test's model


@pytest.mark.timeout(600)
@pytest.mark.parametrize("moving", [False, True], ids=["static", "moving"])
def test_batched_decode_13b_width_16_sequences(moving):
    """configs[3]'s own shape through the batch engine: d 5120, 40 heads, ff 13824, predictor rank 1280, vocab 32000, two layers,
    SIXTEEN sequences advancing in lockstep (the 5120-column MFMA mat-muls, the union-of-active-rows FFN and the 16-wide
    attention).  The predictors keep a margin from the threshold and the greedy choice a margin from the runner-up
    (synth.predictor_fc2_margin, hparams head_pair), so the stated tolerances are asserted verbatim per sequence: logits within
    1e-2 for every step of every sequence, and the greedy continuation of every sequence, running free on the device, equal
    to the CPU oracle's own.
    moving: the predictor's active set depends on the token each sequence is decoding (synth.predictor_fc2_moving), so the sixteen
    sequences disagree about which neurons fire and the union over the batch, which is what the batch kernels read, is larger than any
    single sequence's set - configs[3]'s point."""
    from powerinfer_amd.model import Model
    hp = synth.hparams("llama-13b", n_layer=2, n_ctx=32, seed=SEED_13B_MOVING if moving else 41, pred_margin=True, head_pair=2048, pred_moving=moving)
    model = synth.make_model(hp)
    n_seq, n_prompt, n_gen = 16, 4, 12
    rng = np.random.default_rng(17)
    toks = rng.integers(0, hp.n_vocab, (n_prompt, n_seq)).astype(np.int32)
    gm = Model(hp).load(model)
    gm.batch_init(n_seq)
    oms = [ol.OracleModel(model) for _ in range(n_seq)]
    nxt = None
    for s in range(n_prompt):
        nxt, lg = gm.batch_decode(toks[s], np.full(n_seq, s, np.int32))
        for t in range(n_seq):
            tok_o, lg_o = oms[t].eval([int(toks[s, t])], s)
            assert rel_err(lg[t], lg_o) < 1e-2, (s, t, rel_err(lg[t], lg_o))
            assert int(nxt[t]) == tok_o, (s, t)
            top = np.partition(lg_o, -2)[-2:]
            assert top[1] - top[0] > 2.5 * np.abs(lg[t] - lg_o).max(), (s, t)    # the winner's lead covers the difference seen
    union = gm.batch_union()
    n_on = int(round(hp.mean_rate * hp.n_ff))
    if not moving:
        assert np.all(union == n_on), union                    # the margin predictor's active set is the same for every token
    gen, _ = gm.batch_generate(n_gen)                          # [n_gen][n_seq], free-running on the device
    last_masks = []
    for t in range(n_seq):
        cur = int(nxt[t])
        oms[t].capture(1)
        for s in range(n_gen):
            cur, _ = oms[t].eval([cur], n_prompt + s)
            assert int(gen[s, t]) == cur, (t, s)
        last_masks.append(~(oms[t].cap_lg[:, 0] < hp.sparse_threshold))        # [n_layer][ff] of the last step
        oms[t].close()
    assert len(np.unique(gen)) >= 2                            # the sequences do not all repeat one token
    if moving:
        # the last lockstep step: the union the device reports is the union of the sixteen reference masks, layer by layer, and it
        # is larger than what any one sequence fires
        m = np.array(last_masks)                                # [n_seq][n_layer][ff]
        union = gm.batch_union()
        assert np.array_equal(union, m.any(0).sum(-1)), (union, m.any(0).sum(-1))
        assert np.all(union > m.sum(-1).max(0)), (union, m.sum(-1).max(0))
    gm.close()


@pytest.mark.timeout(600)
def test_batched_decode_7b_q4_width_16_sequences():
    """A Q4_0 model at the 7B width (d 4096, ff 11008, predictor rank 1024, vocab 32000, two layers), sixteen sequences in lockstep
    on the integer matrix-core kernels: per sequence against the CPU oracle, teacher forced (median of the logit distances 1e-2,
    single steps 1e-1, nine greedy tokens in ten equal), then the free-running continuation on the device against stepping the
    same state by hand."""
    from powerinfer_amd.model import Model
    hp = synth.hparams("llama-7b", n_layer=2, n_ctx=32, seed=SEED_7B_Q4_BATCH, wtype=synth.Q4_0, pred_margin=True, head_pair=2048)
    model = synth.make_model(hp)
    n_seq, n_steps = 16, 6
    rng = np.random.default_rng(23)
    toks = rng.integers(0, hp.n_vocab, (n_steps, n_seq)).astype(np.int32)
    gm = Model(hp).load(model)
    gm.batch_init(n_seq)
    oms = [ol.OracleModel(model) for _ in range(n_seq)]
    errs, same = [], 0
    for s in range(n_steps):
        nxt, lg = gm.batch_decode(toks[s], np.full(n_seq, s, np.int32))
        for t in range(n_seq):
            tok_o, lg_o = oms[t].eval([int(toks[s, t])], s)
            errs.append(rel_err(lg[t], lg_o))
            same += int(nxt[t] == tok_o)
    for om in oms:
        om.close()
    errs = np.array(errs)
    assert np.median(errs) < 1e-2 and errs.max() < 1e-1, errs
    assert same >= 0.9 * n_seq * n_steps, same
    assert np.all(gm.batch_union() > 0)
    gen, _ = gm.batch_generate(4)
    gm2 = Model(hp).load(model)
    gm2.batch_init(n_seq)
    cur = None
    for s in range(n_steps):
        cur, _ = gm2.batch_decode(toks[s], np.full(n_seq, s, np.int32))
    for s in range(4):
        cur, _ = gm2.batch_decode(cur, np.full(n_seq, n_steps + s, np.int32))
        assert np.array_equal(gen[s], cur), s
    gm.close(), gm2.close()


def test_batch_kv_sequence_edits():
    """llama_kv_cache_seq_rm / _seq_shift / _seq_cp on the sequences of a batch: one sequence takes a context shift, one is
    untouched, one is emptied and handed the first cells of its neighbour (a shared prefix).  The next lockstep token of every
    sequence must match a single-sequence engine that went through the same history."""
    from powerinfer_amd.model import Model
    hp = synth.hparams("llama-tiny", seed=9, n_ctx=48, sparse_threshold=-1e30)      # every neuron active: no predictor flips between the two paths
    model = synth.make_model(hp)
    n_seq, n0 = 3, 8
    rng = np.random.default_rng(21)
    toks = rng.integers(0, hp.n_vocab, (n0 + 1, n_seq)).astype(np.int32)
    gm = Model(hp).load(model)
    gm.batch_init(n_seq)
    for s in range(n0):
        gm.batch_decode(toks[s], np.full(n_seq, s, np.int32), want_logits=False)
    assert gm.batch_kv_seq_rm(0, 2, 5) == 5
    with pytest.raises(Exception):                               # sequence 0 has a gap open
        gm.batch_decode(toks[n0], np.array([5, 8, 6], np.int32))
    assert gm.batch_kv_seq_shift(0, 5, 8, -3) == 5
    assert gm.batch_kv_seq_rm(2, 0, -1) == 0
    assert gm.batch_kv_seq_cp(1, 2, 0, 6) == 6
    _, lg = gm.batch_decode(toks[n0], np.array([5, 8, 6], np.int32))
    ref = Model(hp).load(model)
    # sequence 0: the same shift on the single-sequence engine
    for s in range(n0):
        ref.decode([int(toks[s, 0])], s)
    ref.kv_seq_rm(2, 5)
    ref.kv_seq_shift(5, 8, -3)
    _, want0 = ref.decode([int(toks[n0, 0])], 5)
    # sequence 1: plain history
    ref.kv_clear()
    for s in range(n0):
        ref.decode([int(toks[s, 1])], s)
    _, want1 = ref.decode([int(toks[n0, 1])], 8)
    # sequence 2: the first six tokens of sequence 1, then its own token
    ref.kv_clear()
    for s in range(6):
        ref.decode([int(toks[s, 1])], s)
    _, want2 = ref.decode([int(toks[n0, 2])], 6)
    for got, want in zip(lg, (want0, want1, want2)):
        assert rel_err(got, want) < 2e-3
    # and the reference itself: its llama.cpp went through the same history with three sequence ids in one KV cache
    # (tests/golden/ref_llama_seq_edits.npz, written by tests/golden/make_llama_fixture.py)
    import importlib.util
    import os
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    spec = importlib.util.spec_from_file_location("make_llama_fixture", os.path.join(root, "tests", "golden", "make_llama_fixture.py"))
    fx = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(fx)
    g = dict(np.load(os.path.join(root, "tests", "golden", "ref_llama_seq_edits.npz")))
    # the fixture belongs to exactly this synthetic model: a change of the generator that moves the weights must come with a new
    # fixture, not with a silently skipped comparison
    assert np.array_equal(fx.model_sha(model), g["model_sha"]), "tests/golden/ref_llama_seq_edits.npz was made from other weights: rerun tests/golden/make_llama_fixture.py"
    assert np.array_equal(toks, g["tokens"])
    for q in range(n_seq):
        assert rel_err(lg[q], g["logits_last"][q]) < 2e-3, q
        assert int(np.argmax(lg[q])) == int(np.argmax(g["logits_last"][q]))
    gm.close(); ref.close()


def test_batch_init_rejects_unsupported_models():
    from powerinfer_amd import lib as pl
    from powerinfer_amd.model import Model
    hp = synth.hparams("llama-tiny", seed=2, n_ctx=32, hot_frac=0.5)          # a VRAM split: the host computes part of every layer
    m = Model(hp).load(synth.make_model(hp))
    with pytest.raises(pl.PiError):
        m.batch_init(4)
    with pytest.raises(pl.PiError):
        m.batch_decode([1], [0])
    m.close()


@pytest.mark.parametrize("wtype", [synth.F16, synth.Q4_0], ids=["f16", "q4_0"])
@pytest.mark.parametrize("arch", ["llama-tiny", "falcon-tiny"])
def test_prompt_chunks_match_token_by_token(arch, wtype):
    """A prompt handed over in one call is evaluated in chunks of up to 16 tokens (weights read once per chunk, causal attention
    inside the chunk); the result must agree with the CPU oracle evaluating the whole prompt as one batch (llama_decode with
    n_tokens > 1) and with feeding the same tokens one at a time.  The models' predictors keep a margin (no logit on the
    threshold, so no neuron flips on the order of a sum): an F16 model then agrees to 5e-3 for every prompt and every later
    step.  A Q4_0 model's chunks run on the integer matrix-core kernels (pi_k_gemm_q4_t16, pi_k_batch_sparse_ffn_q4), where one
    int8 rounding step of a Q8_0 activation still moves a logit by up to a per cent in either path (the single-token path,
    whose dots are the CPU's bit for bit, is as far from the oracle's batch evaluation as the chunks are), so its criterion
    is the median over several prompts."""
    from powerinfer_amd.model import Model
    hp = synth.hparams(arch, seed=12, n_ctx=64, wtype=wtype, pred_margin=True, head_pair=2048)
    model = synth.make_model(hp)
    rng = np.random.default_rng(4)
    err_oracle, err_single, err_after = [], [], []
    for n in (4, 10, 17, 22, 35):
        prompt = rng.integers(0, hp.n_vocab, n).astype(np.int32)
        nxt = rng.integers(0, hp.n_vocab, 3).astype(np.int32)
        ga, gb = Model(hp).load(model), Model(hp).load(model)
        _, lg_a = ga.decode(prompt, 0)                       # chunks of up to 16 tokens, the last token alone
        for i, t in enumerate(prompt):
            _, lg_b = gb.decode([int(t)], i)
        om = ol.OracleModel(model)
        _, lg_o = om.eval([int(t) for t in prompt], 0)
        err_oracle.append(rel_err(lg_a, lg_o))
        err_single.append(rel_err(lg_a, lg_b))
        for i, t in enumerate(nxt):                          # the caches the chunks left behind serve later single-token steps
            _, la = ga.decode([int(t)], n + i)
            _, lo = om.eval([int(t)], n + i)
            err_after.append(rel_err(la, lo))
        om.close()
        ga.close()
        gb.close()
    if wtype == synth.F16:
        assert max(err_oracle) < 5e-3 and max(err_after) < 5e-3 and max(err_single) < 5e-3, (err_oracle, err_after, err_single)
    else:
        assert np.median(err_oracle) < 1e-2, err_oracle
        assert np.median(err_after) < 1e-2, err_after
        assert np.median(err_single) < 5e-2 and max(err_single) < 0.3, err_single


@pytest.mark.timeout(300)
@pytest.mark.parametrize("name,kw,n_prompt,gemm", [("llama-tiny", dict(n_rank=256, n_ctx=192), 150, "own"), ("falcon-tiny", dict(n_rank=256, n_ctx=192), 150, "own"),
                                                   ("llama-tiny", dict(n_rank=256, n_ctx=192), 40, "own"),
                                                   ("llama-7b", dict(n_layer=2, n_ctx=160), 140, "own"), ("llama-7b", dict(n_layer=2, n_ctx=640), 600, "own"),
                                                   ("falcon-tiny", dict(n_rank=256, n_ctx=640), 600, "own"),
                                                   ("llama-tiny", dict(n_rank=256, n_ctx=192), 150, "lib"), ("falcon-tiny", dict(n_rank=256, n_ctx=640), 600, "lib"),
                                                   ("llama-tiny", dict(n_rank=256, n_ctx=192), 40, "lib"),
                                                   ("llama-7b", dict(n_layer=2, n_ctx=640), 600, "lib")])
def test_wide_prompt_chunks_match_the_oracle(name, kw, n_prompt, gemm, monkeypatch):
    """Prompts longer than 16 tokens go through chunks of up to 512 (dense mat-muls through the library, or on this library's own
    LDS-tiled mat-mul kernel with PI_PREFILL_GEMM=own; every weight row read once per chunk, the predictor's mask applied as zeros
    of h), then chunks of 16, then the last token alone.  On a margin-protected model (no neuron can flip, greedy
    decisions keep their distance) the logits after the prompt and of the steps behind it agree with the CPU oracle within the
    stated tolerance, and with the same engine fed 16 tokens at a time."""
    import os
    from powerinfer_amd.model import Model
    if gemm == "own":
        monkeypatch.setenv("PI_PREFILL_GEMM", "own")
    else:
        monkeypatch.delenv("PI_PREFILL_GEMM", raising=False)
    hp = synth.hparams(name, seed=5, pred_margin=True, head_pair=2048, **kw)
    model = synth.make_model(hp)
    rng = np.random.default_rng(8)
    prompt = rng.integers(0, hp.n_vocab, n_prompt).astype(np.int32)
    ga = Model(hp).load(model)
    tok_a, lg_a = ga.decode(prompt, 0)
    om = ol.OracleModel(model)
    tok_o, lg_o = om.eval([int(t) for t in prompt], 0)
    assert rel_err(lg_a, lg_o) < 1e-2, rel_err(lg_a, lg_o)
    assert tok_a == tok_o
    cur = tok_o
    for i in range(4):                                        # the cache the chunks left behind serves the following steps
        ta, la = ga.decode([cur], n_prompt + i)
        cur, lo = om.eval([cur], n_prompt + i)
        assert rel_err(la, lo) < 1e-2, (i, rel_err(la, lo))
        assert ta == cur
    om.close()
    os.environ["PI_NO_PREFILL_WIDE"] = "1"                  # the same prompt through chunks of 16 only
    try:
        gb = Model(hp).load(model)
        _, lg_b = gb.decode(prompt, 0)
    finally:
        del os.environ["PI_NO_PREFILL_WIDE"]
    assert rel_err(lg_a, lg_b) < 1e-2
    assert not np.array_equal(lg_a, lg_b) or n_prompt <= 17   # the two routes sum in different orders: identical bits would mean the wide route did not run
    ga.close(), gb.close()


@pytest.mark.timeout(600)
@pytest.mark.parametrize("name,wtype,hot_frac,kw,n_prompt", [("falcon-tiny", synth.Q4_0, 1.0, dict(n_rank=256, n_ctx=192), 150),
                                                             ("llama-7b", synth.Q4_0, 1.0, dict(n_layer=2, n_ctx=192), 140),
                                                             ("falcon-tiny", synth.Q4_0, 0.6, dict(n_rank=256, n_ctx=640), 600),
                                                             ("llama-tiny", synth.F16, 0.6, dict(n_rank=256, n_ctx=192), 150),
                                                             ("falcon-tiny", synth.F16, 0.5, dict(n_rank=256, n_ctx=192), 60),
                                                             ("llama-7b", synth.Q4_0, 0.6, dict(n_layer=2, n_ctx=640), 600)])
def test_wide_prompt_chunks_of_q4_and_hybrid_models(name, wtype, hot_frac, kw, n_prompt):
    """Prompts of Q4_0 models and of models with a VRAM split also go through chunks of up to 512 tokens: a Q4_0 matrix is expanded
    to fp16 for the chunk ((q - 8) * d) and multiplied with the values the CPU path's Q8_0 blocks keep of the activations, a
    hybrid layer's FFN matrices are assembled from the resident rows and the others' rows in pinned host memory.  On a
    margin-protected model the logits after the prompt and of the steps behind it agree with the CPU oracle within the stated
    tolerance, and with the same engine taking the prompt token by token.  With Q4_0 weights the tolerance is held on the median
    and every greedy token is identical: the reference, run against itself with norm weights moved by one unit in the last place,
    departs by more than 1e-2 on single tokens, because one int8 rounding step of an activation is a visible share of a dot product
    (tests/test_oracle_math.py::test_q4_reference_departs_from_itself_beyond_the_logit_tolerance)."""
    import os
    from powerinfer_amd.model import Model
    hp = synth.hparams(name, seed=5, pred_margin=True, head_pair=2048, wtype=wtype, hot_frac=hot_frac, **kw)
    model = synth.make_model(hp)
    rng = np.random.default_rng(8)
    prompt = rng.integers(0, hp.n_vocab, n_prompt).astype(np.int32)
    ga = Model(hp).load(model)
    tok_a, lg_a = ga.decode(prompt, 0)
    om = ol.OracleModel(model)
    tok_o, lg_o = om.eval([int(t) for t in prompt], 0)
    q4 = wtype != synth.F16
    errs = [rel_err(lg_a, lg_o)]
    assert errs[0] < 1e-2, errs
    assert tok_a == tok_o
    cur = tok_o
    for i in range(8):                                        # the cache the chunks left behind serves the following steps
        ta, la = ga.decode([cur], n_prompt + i)
        cur, lo = om.eval([cur], n_prompt + i)
        errs.append(rel_err(la, lo))
        assert ta == cur
    assert np.median(errs) < 1e-2 and max(errs) < (1e-1 if q4 else 1e-2), errs
    om.close()
    os.environ["PI_NO_PREFILL_WIDE"] = "1"                  # the same prompt token by token
    try:
        gb = Model(hp).load(model)
        _, lg_b = gb.decode(prompt, 0)
    finally:
        del os.environ["PI_NO_PREFILL_WIDE"]
    assert rel_err(lg_a, lg_b) < (5e-2 if q4 else 1e-2), rel_err(lg_a, lg_b)
    assert not np.array_equal(lg_a, lg_b)                     # identical bits would mean the chunk route did not run
    ga.close(), gb.close()


@pytest.mark.parametrize("n", [32000, 32001, 1000, 7])
def test_argmax_batch_takes_the_first_maximum(n):
    """pi_k_argmax_batch against numpy's argmax (the first maximum wins, as the greedy sampler's loop does, llama.cpp:8617-8631): ties
    inside one thread's 16-byte load, across threads and across waves, a row of -inf (token 0), a row with NaNs (never greater),
    row widths that take the 16-byte path (n % 4 == 0) and the element-wise one; positions advance, the step's tokens are recorded."""
    from powerinfer_amd import lib as pl
    L = pl.init()
    T = 16
    rng = np.random.default_rng(n)
    lg = rng.standard_normal((T, n)).astype(np.float32)
    lg[1, :] = 0.25                                                  # every element ties: token 0
    lg[2, [n - 1, n // 2, 3 % n]] = 9.0                                # ties far apart: the lowest index
    lg[3, min(5, n - 1)] = 9.0; lg[3, min(6, n - 1)] = 9.0           # ties within one 16-byte load
    lg[4, :] = -np.inf                                                # nothing compares greater: token 0
    lg[5, ::3] = np.nan                                               # NaNs never win
    lg[6, n - 1] = 50.0                                               # the last element
    want = np.array([int(np.nanargmax(np.where(np.isnan(r), -np.inf, r))) if np.isfinite(r[~np.isnan(r)]).any() else 0 for r in lg], np.int32)
    dl, dt = pl.DevBuf(host=lg), pl.DevBuf(T * 4)
    dp, ds, do = pl.DevBuf(host=np.arange(T, dtype=np.int32)), pl.DevBuf(host=np.array([1], np.int32)), pl.DevBuf(host=np.full(3 * T, -1, np.int32))
    pl.check(L.pi_k_argmax_batch(dl.ptr, n, T, dt.ptr, dp.ptr, ds.ptr, do.ptr, 3, None), "argmax")
    pl.sync()
    got = dt.download(np.int32)
    assert np.array_equal(got, want), (got, want)
    assert np.array_equal(dp.download(np.int32), np.arange(T) + 1)
    rec = do.download(np.int32).reshape(3, T)
    assert np.array_equal(rec[1], want) and np.all(rec[0] == -1) and np.all(rec[2] == -1)
