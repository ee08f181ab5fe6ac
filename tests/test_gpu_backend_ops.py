"""Every operator the decode graph offloads besides the sparse FFN (llm_build_norm, llm_build_kv_store, llm_build_kqv, RoPE,
embedding lookup; ggml-cuda.cu:9241-9333), each driven through ggml_cuda_compute_forward the way the reference's executor
drives a GPU node, against the golden vectors the compiled reference wrote (tests/golden/ops.npz) or the closed form."""
import ctypes as C

import numpy as np
import pytest

import oracle_lib as ol
from oracle_lib import _ptr as P

pytestmark = pytest.mark.gpu

F32, F16, Q4_0, I32 = 0, 1, 2, 18


def rel_err(a, b):
    return float(np.abs(a - b).max() / max(np.abs(b).max(), 1e-30))


def graph():
    from powerinfer_amd import lib as pl
    from ggml_graph import Graph
    return Graph(pl.load())


def test_norms_softmax_scale(golden):
    g = golden("ops")
    G = graph()
    x = G.new(F32, [320, 3], g["norm_x"], "x")
    rms = G.on_gpu(G.rms_norm(x, 1e-5))
    ln = G.on_gpu(G.norm(x, 1e-5))
    sx = G.new(F32, [77, 5], g["sm_x"], "sm_x")
    sm = G.on_gpu(G.soft_max(sx))
    fac = G.new(F32, [1], np.array([0.17677669], np.float32), "kq_scale")
    sc = G.on_gpu(G.scale(x, fac))
    G.compute()
    assert not G.cpu_run
    assert rel_err(G.host(rms), g["rms_y"]) < 2e-6
    assert rel_err(G.host(ln), g["ln_y"]) < 2e-6
    assert np.abs(G.host(sm) - g["sm_y"]).max() < 2e-6 and (G.host(sm)[:, 60:] == 0).all()       # masked tail stays exactly zero
    assert np.array_equal(G.host(sc), g["norm_x"] * np.float32(0.17677669))


@pytest.mark.parametrize("mode", [0, 2])
def test_rope_modes(golden, mode):
    g = golden("ops")
    G = graph()
    x = G.new(F32, [64, 3, 4], g["rope_x"], "x")                 # [hd, n_head, T]
    pos = G.new(I32, [4], g["rope_pos"], "pos")
    y = G.on_gpu(G.rope(x, pos, 64, mode))
    G.compute()
    assert not G.cpu_run
    assert np.abs(G.host(y) - g[f"rope{mode}_y"]).max() < 2e-5   # position 300: cosf/sinf of the device vs the host's, angles identical


@pytest.mark.parametrize("tag,mode,n_orig,fs,ext,attn,bf,bs", [("lin0", 0, 0, 0.25, 0.0, 1.0, 32.0, 1.0), ("lin2", 2, 0, 0.5, 0.0, 1.0, 32.0, 1.0),
                                                               ("yarn0", 0, 256, 0.25, 1.0, 1.0, 32.0, 1.0), ("yarn0b", 0, 128, 0.125, 0.7, 1.3, 16.0, 2.0),
                                                               ("yarn2", 2, 256, 0.25, 1.0, 1.0, 32.0, 1.0)])
def test_rope_with_linear_and_yarn_scaling(golden, tag, mode, n_orig, fs, ext, attn, bf, bs):
    """ROPE nodes as a model with a scaled context builds them (ggml_rope_custom, llama.cpp:4900-4960): linear scaling and YaRN
    (rope_yarn, ggml.c:11124-11161), against what the compiled reference wrote (tests/golden/rope_scaled.npz)."""
    g = golden("rope_scaled")
    G = graph()
    x = G.new(F32, [64, 3, 5], g["x"], "x")                      # [hd, n_head, T]
    pos = G.new(I32, [5], g["pos"], "pos")
    y = G.on_gpu(G.rope(x, pos, 64, mode, freq_scale=fs, n_orig_ctx=n_orig, ext_factor=ext, attn_factor=attn, beta_fast=bf, beta_slow=bs))
    G.compute()
    assert not G.cpu_run
    assert np.abs(G.host(y) - g[tag]).max() < 3e-5               # positions up to 2047: cosf / sinf of the device against the host's


@pytest.mark.parametrize("mode", [0, 2])
def test_k_shift_rope_in_place_over_a_cache_view(mode):
    """The K-shift graph (llama.cpp:4332-4381): ggml_rope_custom_inplace over a 3-D view [hd, n_head_kv, n_ctx] of one layer's fp16 K
    cache, the position operand holding each cell's delta.  Against the oracle's RoPE on the fp32 values of the same cells, rounded
    to fp16 as ggml_compute_forward_rope_f16 stores them (ggml.c:11327-11460); the other layer's cells must stay untouched."""
    hd, nkv, nctx, n_layer, il = 64, 2, 24, 2, 1
    gqa = hd * nkv
    rng = np.random.default_rng(40 + mode)
    cache = rng.standard_normal(n_layer * nctx * gqa).astype(np.float16)
    delta = rng.integers(-9, 1, nctx).astype(np.int32)
    G = graph()
    kc = G.on_gpu(G.new(F16, [n_layer * nctx * gqa], cache.copy().view(np.uint16), "cache_k"))     # the tensor's host buffer is overwritten on read-back
    G.L.ggml_cuda_copy_to_device(C.byref(kc))
    kv = G.on_gpu(G.view(kc, [hd, nkv, nctx], [hd * 2, gqa * 2], il * nctx * gqa * 2, "k_view"))
    pos = G.new(I32, [nctx], delta, "K_shift")
    G.on_gpu(G.rope_inplace(kv, pos, hd, mode, name="K_shifted"))
    G.compute()
    assert not G.cpu_run, G.cpu_run
    got = G.host(kc, np.uint16).view(np.float16).reshape(n_layer, nctx, nkv, hd)
    O = ol.oracle()
    x = np.ascontiguousarray(cache.reshape(n_layer, nctx, nkv, hd)[il].astype(np.float32))
    want = np.zeros_like(x)
    O.pio_rope(P(x), hd, nkv, nctx, P(delta), hd, mode, 10000.0, 1.0, P(want))
    assert np.array_equal(got[0], cache.reshape(n_layer, nctx, nkv, hd)[0])
    diff = np.abs(got[il].astype(np.float32) - want.astype(np.float16).astype(np.float32))
    assert (diff > 0).mean() < 5e-3 and diff.max() <= 2e-3 * np.abs(want).max()      # a handful of fp16 rounding ties from the device's cosf / sinf
    assert not np.array_equal(got[il], cache.reshape(n_layer, nctx, nkv, hd)[il])


@pytest.mark.parametrize("wtype", [F16, Q4_0])
def test_dense_mul_mat_two_tokens_and_get_rows(golden, wtype):
    g = golden("ops")
    tag = "mm_f16" if wtype == F16 else "mm_q4"
    w, x, want = g[tag + "_w"], g[tag + "_x"], g[tag + "_y"]
    rows, cols = want.shape[1], x.shape[1]
    G = graph()
    tw = G.weight_to_gpu(G.new(wtype, [cols, rows], w, "w"))
    y = G.on_gpu(G.mul_mat(tw, G.new(F32, [cols, 2], x, "x")))
    ids = np.array([3, 0, rows - 1], np.int32)
    emb = G.on_gpu(G.get_rows(tw, G.new(I32, [3], ids, "ids")))
    G.compute()
    assert not G.cpu_run
    assert rel_err(G.host(y), want) < 5e-6
    if wtype == F16:
        table = w.astype(np.float32)
    else:
        table = np.zeros((rows, cols), np.float32)
        for r in range(rows):
            ol.oracle().pio_dequantize_row_q4_0(P(np.ascontiguousarray(w[r])), P(table[r]), cols)
    assert np.array_equal(G.host(emb), table[ids])


@pytest.mark.parametrize("T", [20, 70])
def test_dense_mul_mat_of_a_prompt_batch(T):
    """MUL_MAT with a batch of prompt tokens at the boundary (the reference's cuBLAS leg, ggml-cuda.cu:7662-7756): 20 tokens go
    through this library's 16-token mat-mul kernel, 70 through one library mat-mul over all of them; both against the
    reference's CPU mat-mul (activations rounded to fp16, ggml.c:9598-9807) as the oracle restates it."""
    rng = np.random.default_rng(T)
    rows, cols = 1000, 1024
    w = (rng.standard_normal((rows, cols)) * 0.02).astype(np.float16)
    x = rng.standard_normal((T, cols)).astype(np.float32)
    want = np.zeros((T, rows), np.float32)
    assert ol.oracle().pio_mul_mat(ol.F16, P(w), rows, cols, P(x), T, P(want), 4) == 0
    G = graph()
    tw = G.weight_to_gpu(G.new(F16, [cols, rows], w, "w"))
    y = G.on_gpu(G.mul_mat(tw, G.new(F32, [cols, T], x, "x")))
    G.compute()
    assert not G.cpu_run
    assert rel_err(G.host(y), want) < 1e-5


def test_kv_store_and_attention_core_as_the_graph_builds_them(golden):
    """llm_build_kv_store (llama.cpp:4383-4418): K rows copied F32 -> F16 into a 1-D cache view, V transposed into a strided view;
    llm_build_kqv (:4764-4850): K . q over a strided 3-D view of the cache against the permuted q, scale, mask add, softmax,
    V . p over the transposed cache, permute + cont.  Five prompt tokens at once (the golden case att0), GQA 4 heads over 2."""
    g = golden("ops")
    hd, nh, nkv, nctx, T = 32, 4, 2, 48, 5
    gqa = nkv * hd
    q, k, v, want = g["att0_q"], g["att0_k"], g["att0_v"], g["att0_o"]
    G = graph()
    kc = G.on_gpu(G.new(F16, [nctx * gqa], np.zeros(nctx * gqa, np.uint16), "cache_k"))
    vc = G.on_gpu(G.new(F16, [nctx * gqa], np.zeros(nctx * gqa, np.uint16), "cache_v"))
    G.L.ggml_cuda_copy_to_device(C.byref(kc)); G.L.ggml_cuda_copy_to_device(C.byref(vc))
    # Kcur / Vcur / Qcur are results of device nodes in the real graph: resident, so that views of them share their device memory
    k_cur = G.weight_to_gpu(G.new(F32, [gqa, T], k.reshape(T, gqa), "Kcur"))
    v_cur = G.weight_to_gpu(G.new(F32, [gqa, T], v.reshape(T, gqa), "Vcur"))
    # store: k_cache_view = view_1d(T * gqa at cell 0), v_cache_view = view_2d(T, gqa, nb1 = nctx * 2) of the transposed V
    k_view = G.on_gpu(G.view(kc, [T * gqa], [], 0, "k_cache_view"))
    v_t = G.on_gpu(G.permute(v_cur, (1, 0, 2, 3), "v_cur_t"))     # ggml_transpose: [T, gqa] with swapped strides
    v_view = G.on_gpu(G.view(vc, [T, gqa], [nctx * 2], 0, "v_cache_view"))
    G.on_gpu(G.cpy(k_cur, k_view, "k_store"))
    G.on_gpu(G.cpy(v_t, v_view, "v_store"))
    # attention
    tq = G.weight_to_gpu(G.new(F32, [hd, nh, T], q, "Qcur"))
    qp = G.on_gpu(G.permute(tq, (0, 2, 1, 3), "q"))               # [hd, T, nh]
    kk = G.on_gpu(G.view(kc, [hd, T, nkv], [gqa * 2, hd * 2], 0, "k"))          # n_kv = T cells
    kq = G.on_gpu(G.mul_mat(kk, qp, "kq"))                        # [n_kv, T, nh]
    fac = G.new(F32, [1], np.array([1.0 / np.sqrt(hd)], np.float32), "kq_scale")
    kqs = G.on_gpu(G.scale(kq, fac, "kq_scaled"))
    mask = np.where(np.arange(T)[None, :] > np.arange(T)[:, None], -np.inf, 0).astype(np.float32)       # [T][n_kv] causal
    kqm = G.on_gpu(G.add(kqs, G.new(F32, [T, T], mask, "KQ_mask"), "kq_masked"))
    kqsm = G.on_gpu(G.soft_max(kqm, "kq_soft_max"))
    vv = G.on_gpu(G.view(vc, [T, hd, nkv], [nctx * 2, nctx * 2 * hd], 0, "v"))  # [n_kv, hd, nkv] of the transposed cache
    kqv = G.on_gpu(G.mul_mat(vv, kqsm, "kqv"))                    # [hd, T, nh]
    merged = G.on_gpu(G.permute(kqv, (0, 2, 1, 3), "kqv_merged"))   # [hd, nh, T], a view of kqv on the device
    out = G.on_gpu(G.cont(merged, "kqv_merged_cont"))
    G.compute()
    assert not G.cpu_run, G.cpu_run                             # every node ran on the backend
    got_k = G.host(kc, np.uint16).reshape(nctx, gqa)
    got_v = G.host(vc, np.uint16).reshape(gqa, nctx)
    assert np.array_equal(got_k[:T], k.reshape(T, gqa).astype(np.float16).view(np.uint16)) and not got_k[T:].any()
    assert np.array_equal(got_v[:, :T], v.astype(np.float16).view(np.uint16).T) and not got_v[:, T:].any()
    assert rel_err(G.host(out).reshape(T, nh * hd), want) < 1e-5
