"""The reference's backend entry points (ggml_cuda_* in include/ggml_backend_abi.h) driven the way ggml's executor
drives them, on the op sequence llm_build_ffn_sparse emits (llama.cpp:4652-4757): full-GPU fast path and the
hybrid CPU part + GPU part + ggml_add variant."""
import ctypes as C

import numpy as np
import pytest

import oracle_lib as ol
from powerinfer_amd import synth

pytestmark = pytest.mark.gpu


def rel_err(a, b):
    return float(np.abs(a - b).max() / max(np.abs(b).max(), 1e-30))


def out_under(L, wtype, has_gate, x, lg, thr=0.0):
    """[T][d] output of the CPU oracle for the masks the given predictor logits [T][ff] imply."""
    return np.stack([ol.ffn_under_logits(ol.oracle(), L["d"], L["ff"], wtype, has_gate, L["up"], L["gate"], L["down_t"], x[t], lg[t], thr)["out"]
                     for t in range(x.shape[0])])


def build_ffn(G, L, x, wtype, full_gpu, gid=None, bucket=None):
    """llm_build_ffn_sparse for T tokens; returns (idx, out)."""
    d, ff, r, T = L["d"], L["ff"], L["r"], x.shape[0]
    has_gate = L["gate"] is not None
    t_x = G.new(0, [d, T], x, "ffn_input")
    fc1 = G.weight_to_gpu(G.new(1, [d, r], L["fc1"], "fc1"))
    fc2 = G.weight_to_gpu(G.new(1, [r, ff], L["fc2"], "fc2"))
    names = ("up", "gate", "down_t") if has_gate else ("up", "down_t")
    if full_gpu:
        W = {n: G.weight_to_gpu(G.new(wtype, [d, ff], L[n], n + "_gpu")) for n in names}
    else:
        Wc = {n: G.new(wtype, [d, ff], L[n], n) for n in names}
        Wg = {n: G.weight_to_gpu(G.new(wtype, [d, bucket.size], np.ascontiguousarray(L[n][bucket]), n + "_gpu")) for n in names}
        t_gid = G.new(18, [ff], gid, "gpu_idx")
        t_bkt = G.new(18, [bucket.size], bucket, "gpu_bucket")
    idx = G.on_gpu(G.mul_mat(fc1, t_x, "mlp_pre_hidden"))
    idx = G.on_gpu(G.relu(idx, "mlp_pre_relu"))
    idx = G.mul_mat(fc2, idx, "mlp_pre_out")
    if full_gpu:
        G.on_gpu(idx)

    def sparse_mm(n):
        if full_gpu:
            return G.on_gpu(G.mul_mat_idx(W[n], t_x, idx, None, f"ffn_{n}_sparse"))
        cpu = G.mul_mat_idx(Wc[n], t_x, idx, t_gid, f"ffn_{n}_sparse")
        gpu = G.on_gpu(G.mul_mat_idx_upscale(Wg[n], t_x, idx, t_bkt, ff, f"ffn_{n}_sparse_gpu"))
        return G.add(cpu, gpu, f"ffn_{n}_sparse_merged")

    up = sparse_mm("up")
    if has_gate:
        gate = sparse_mm("gate")
        act = G.relu(gate, "ffn_gate_act")
        cur = G.mul(act, up, "ffn_gate_par")
        if full_gpu:
            G.on_gpu(act), G.on_gpu(cur)
    else:
        cur = G.relu(up, "ffn_up_act")
        if full_gpu:
            G.on_gpu(cur)
    if full_gpu:
        out = G.on_gpu(G.axpy(W["down_t"], cur, idx, None, "ffn_down_sparse"))
    else:
        cpu = G.axpy(Wc["down_t"], cur, idx, t_gid, "ffn_down_sparse")
        gpu = G.on_gpu(G.axpy(Wg["down_t"], cur, idx, t_bkt, "ffn_down_sparse_gpu"))
        out = G.on_gpu(G.add(cpu, gpu, "ffn_down_sparse_merged"))
    return idx, out


@pytest.mark.parametrize("wtype", [ol.F16, ol.Q4_0])
@pytest.mark.parametrize("has_gate", [True, False])
def test_full_gpu_graph(wtype, has_gate):
    from powerinfer_amd import lib as pl
    from ggml_graph import Graph
    d, ff, r, T = 1024, 4096, 128, 2
    L = synth.make_ffn_layer(seed=61 + wtype, d=d, ff=ff, r=r, wtype=wtype, has_gate=has_gate, mean_rate=0.15, T=T)
    G = Graph(pl.load())
    idx, out = build_ffn(G, L, L["x"], wtype, True)
    G.compute(0.0)
    assert not G.cpu_run, G.cpu_run                      # every node was taken by the backend
    o = ol.ffn_sparse(ol.oracle(), d, ff, r, T, wtype, has_gate, L["up"], L["gate"], L["down_t"], L["fc1"], L["fc2"], L["x"], L["x"],
                      np.zeros(ff, np.int32), 0.0, nth=4)
    lg = G.host(idx)
    assert rel_err(lg, o["logits"]) < 1e-5
    assert ((lg >= 0) == (o["logits"] >= 0)).mean() >= 0.999
    assert rel_err(G.host(out), out_under(L, wtype, has_gate, L["x"], lg)) < 1e-4


@pytest.mark.parametrize("wtype", [ol.F16, ol.Q4_0])
def test_hybrid_graph_cpu_part_plus_gpu_part(wtype):
    from powerinfer_amd import lib as pl
    from ggml_graph import Graph
    d, ff, r, T = 1024, 4096, 128, 2
    L = synth.make_ffn_layer(seed=71, d=d, ff=ff, r=r, wtype=wtype, mean_rate=0.15, T=T)
    gid, bucket = synth.gpu_split(L["p"], 0.6)
    G = Graph(pl.load())
    idx, out = build_ffn(G, L, L["x"], wtype, False, gid, bucket)
    G.compute(0.0)
    # weights on the CPU: the backend must hand those sparse nodes back (ggml-cuda.cu:9226-9230)
    assert {"ffn_up_sparse", "ffn_gate_sparse", "ffn_down_sparse"} <= set(G.cpu_run)
    assert {"ffn_up_sparse_gpu", "ffn_gate_sparse_gpu", "ffn_down_sparse_gpu", "mlp_pre_out"} <= set(G.gpu_run)
    o = ol.ffn_sparse(ol.oracle(), d, ff, r, T, wtype, 1, L["up"], L["gate"], L["down_t"], L["fc1"], L["fc2"], L["x"], L["x"],
                      np.zeros(ff, np.int32), 0.0, nth=4)
    lg = G.host(idx)
    assert rel_err(lg, o["logits"]) < 1e-5
    assert ((lg >= 0) == (o["logits"] >= 0)).mean() >= 0.999
    assert rel_err(G.host(out), out_under(L, wtype, True, L["x"], lg)) < 1e-4


@pytest.mark.timeout(300)
def test_full_gpu_graph_13b_step_of_16():
    """configs[3]'s step as the reference's graph hands it over: 16 tokens through the FFN block of a 13B layer (d 5120, ff 13824,
    predictor rank 1024), every node on the backend.  The sparse operators take the batch route (union of the active rows, each
    weight row read once for the 16 tokens, matrix cores) instead of 16 single-token passes (ggml-cuda.cu:6994-7034, 8787-8814)."""
    from powerinfer_amd import lib as pl
    from ggml_graph import Graph
    d, ff, r, T = 5120, 13824, 1024, 16
    L = synth.make_ffn_layer(seed=67, d=d, ff=ff, r=r, wtype=ol.F16, has_gate=True, T=T)
    G = Graph(pl.load())
    idx, out = build_ffn(G, L, L["x"], ol.F16, True)
    G.compute(0.0)
    assert not G.cpu_run, G.cpu_run
    o = ol.ffn_sparse(ol.oracle(), d, ff, r, T, ol.F16, True, L["up"], L["gate"], L["down_t"], L["fc1"], L["fc2"], L["x"], L["x"],
                      np.zeros(ff, np.int32), 0.0, nth=8)
    lg = G.host(idx)
    # fp32 sums of 5120 products in another order than the oracle's, then the fp16 rounding of the hidden vector: a hidden value that
    # falls on the other side of a rounding boundary moves a logit by 2^-11 of one term; the largest of the 221 184 logits' errors
    # comes out at 0.9e-5 to 1.1e-5 of the largest logit, whichever way the columns are split over the waves
    assert rel_err(lg, o["logits"]) < 2e-5
    assert ((lg >= 0) == (o["logits"] >= 0)).mean() >= 0.999
    assert rel_err(G.host(out), out_under(L, ol.F16, True, L["x"], lg)) < 1e-4
    per_token = ((lg >= 0).sum(1))
    assert per_token.min() > 0 and len(set(per_token.tolist())) > 1          # the tokens' active sets differ: the union is a real union


def test_backend_info_entry_points():
    from powerinfer_amd import lib as pl
    L = pl.load()
    L.ggml_init_cublas()
    L.ggml_cublas_loaded.restype = C.c_bool
    assert L.ggml_cublas_loaded()
    assert L.ggml_cuda_get_device_count() >= 1
    buf = C.create_string_buffer(128)
    L.ggml_cuda_get_device_description.argtypes = [C.c_int, C.c_char_p, C.c_size_t]
    L.ggml_cuda_get_device_description(0, buf, 128)
    assert buf.value.startswith(b"gfx950")
    L.ggml_cuda_get_free_memory.restype = C.c_size_t
    assert L.ggml_cuda_get_free_memory(0) > (100 << 30)
    L.ggml_cuda_host_malloc.restype = C.c_void_p
    L.ggml_cuda_host_malloc.argtypes = [C.c_size_t]
    L.ggml_cuda_host_free.argtypes = [C.c_void_p]
    p = L.ggml_cuda_host_malloc(1 << 20)
    assert p
    L.ggml_cuda_host_free(p)
    L.ggml_backend_cuda_init.restype = C.c_void_p
    assert L.ggml_backend_cuda_init() is None


@pytest.mark.parametrize("wtype", [ol.F16, ol.Q4_0])
@pytest.mark.parametrize("hot_frac", [1.0, 0.6])
def test_reference_executor_drives_this_backend(wtype, hot_frac):
    """Drop-in check of the boundary: oracle/_ref/libpi_ref_gpu.so is the REFERENCE's ggml.c compiled with
    -DGGML_USE_CUBLAS and linked against libpowerinfer_hip.so in place of ggml-cuda.cu.  Its own op constructors,
    graph and two-thread executor run llm_build_ffn_sparse's op sequence (full-GPU, and hybrid CPU part + GPU part
    + ggml_add), ONE evaluation each.

    Every node this backend computes is deterministic and is checked strictly: the predictor logits, the backend's share of
    the down projection and the final ggml_add of the two shares.  The hybrid graph's host share is computed by the reference's
    own CPU axpy on two threads (the executor asserts n_threads > 1 for hybrid graphs), and that kernel adds each thread's
    partial vector into the output without a lock, eight floats at a time (`res += tmp`, ggml.c:14433-14458): an 8-float
    group of the HOST node may therefore hold the sum of both threads' rows or of either thread's rows alone.  Only that node
    gets this three-way acceptance, per 8-float group, and the groups that lost a share are counted in the report."""
    import os
    so = os.path.join(ol.ODIR, "_ref", "libpi_ref_gpu.so")
    if not os.path.exists(so):
        pytest.skip("oracle/_ref/libpi_ref_gpu.so was not built (needs the reference tree at build time)")
    R = C.CDLL(so)
    vp, i, f = C.c_void_p, C.c_int, C.c_float
    R.ref_ffn_sparse_gpu_parts.argtypes = [i] * 6 + [vp] * 9 + [i, f] + [vp] * 5
    R.ref_init()
    d, ff, r, T = 1024, 4096, 128, 2
    L = synth.make_ffn_layer(seed=81 + wtype, d=d, ff=ff, r=r, wtype=wtype, mean_rate=0.15, T=T)
    gid, bucket = synth.gpu_split(L["p"], hot_frac)
    hybrid = hot_frac < 1.0
    n_bucket = bucket.size if hybrid else 0
    lg, out = np.zeros((T, ff), np.float32), np.zeros((T, d), np.float32)
    h, part_cpu, part_gpu = np.zeros((T, ff), np.float32), np.zeros((T, d), np.float32), np.zeros((T, d), np.float32)
    P = ol._ptr
    O = ol.oracle()
    o = ol.ffn_sparse(O, d, ff, r, T, wtype, 1, L["up"], L["gate"], L["down_t"], L["fc1"], L["fc2"], L["x"], L["x"], np.zeros(ff, np.int32), 0.0, nth=4)
    rc = R.ref_ffn_sparse_gpu_parts(d, ff, r, T, wtype, 1, P(L["up"]), P(L["gate"]), P(L["down_t"]), P(L["fc1"]), P(L["fc2"]), P(L["x"]), P(L["x"]),
                                    P(gid), P(bucket), n_bucket, 0.0, P(lg), P(out), P(h), P(part_cpu), P(part_gpu))
    assert rc == 0
    assert rel_err(lg, o["logits"]) < 1e-5                                   # mlp_pre_out: a backend node
    assert ((lg >= 0) == (o["logits"] >= 0)).mean() >= 0.999
    if not hybrid:
        assert rel_err(out, out_under(L, wtype, True, L["x"], lg)) < 1e-4    # every node ran on the backend
        return
    raced = 0
    for t in range(T):
        u = ol.ffn_under_logits(O, d, ff, wtype, True, L["up"], L["gate"], L["down_t"], L["x"][t], lg[t], 0.0)      # up/gate/h over all neurons
        scale = np.abs(u["out"]).max()
        assert rel_err(h[t], u["h"]) < 1e-4                                  # ffn_*_sparse (host) + ffn_*_sparse_gpu (backend) merged
        # the backend's share of the down projection: rows of the bucket, h as the graph merged it
        want_gpu = ol.axpy_under_logits(O, d, ff, wtype, L["down_t"], h[t], lg[t], 0.0, skip=1 - gid)
        assert np.abs(part_gpu[t] - want_gpu).max() < 1e-4 * scale, "ffn_down_sparse_gpu (backend node)"
        # the final ggml_add ran on the backend
        assert np.abs(out[t] - (part_cpu[t] + part_gpu[t])).max() <= 1e-6 * scale, "ffn_down_sparse_merged (backend node)"
        # the host node: both threads' rows, or (lost update) the rows of one thread only, per 8-float group
        dr = (ff + 1) // 2
        first = np.arange(ff) < dr
        cands = [ol.axpy_under_logits(O, d, ff, wtype, L["down_t"], h[t], lg[t], 0.0, skip=sk)
                 for sk in (gid, gid | (~first).astype(np.int32), gid | first.astype(np.int32))]
        err = np.stack([np.abs(part_cpu[t] - c).reshape(-1, 8).max(1) for c in cands])      # [3][d/8]
        assert (err.min(0) < 1e-4 * scale).all(), f"host node ffn_down_sparse: errors vs (both, thread 0, thread 1) {err.max(1) / scale}"
        raced += int((err[0] >= 1e-4 * scale).sum())
    print(f"host axpy groups of 8 floats that lost one thread's share: {raced} of {T * d // 8}")


def backend_stats(L):
    st = (C.c_int64 * 4)()
    L.pi_ggml_backend_get_stats(st)
    return dict(deferred=int(st[0]), flushed=int(st[1]), fused=int(st[2]), attn_fused=int(st[3]))


def build_decode_ffn(G, L, norm, has_gate, spoiler=None):
    """One token through llm_build_norm + llm_build_ffn_sparse (llama.cpp:4420-4450, 4652-4757) with every tensor on the device, in the
    node order the reference's graph has.  norm: 0 none (the FFN reads the vector as it is, Falcon's order of things), 1 RMSNorm * w,
    2 LayerNorm * w + b.  spoiler: name of a node after which an unrelated node (a SCALE) is slipped in, which must break the window."""
    d, ff, r = L["d"], L["ff"], L["r"]
    F = G.weight_to_gpu(G.new(0, [d, 1], L["x"][:1], "ffn_inp"))
    rng = np.random.default_rng(4)
    nw = (1 + 0.1 * rng.standard_normal(d)).astype(np.float32)
    nb = (0.1 * rng.standard_normal(d)).astype(np.float32)
    if norm:
        cur = G.on_gpu(G.rms_norm(F, 1e-5, "norm") if norm == 1 else G.norm(F, 1e-5, "norm"))
        cur = G.on_gpu(G.mul(cur, G.weight_to_gpu(G.new(0, [d], nw, "ffn_norm.weight")), "norm_w"))
        if norm == 2:
            cur = G.on_gpu(G.add(cur, G.weight_to_gpu(G.new(0, [d], nb, "ffn_norm.bias")), "ffn_norm"))
    else:
        cur = F
    one = G.weight_to_gpu(G.new(0, [1], np.ones(1, np.float32), "one"))
    extra = []

    def node(t):
        G.on_gpu(t)
        if spoiler and t.name.decode() == spoiler:
            extra.append(G.on_gpu(G.scale(F, one, "unrelated")))
        return t
    fc1 = G.weight_to_gpu(G.new(1, [d, r], L["fc1"], "fc1"))
    fc2 = G.weight_to_gpu(G.new(1, [r, ff], L["fc2"], "fc2"))
    W = {n: G.weight_to_gpu(G.new(1, [d, ff], L[n], n + "_gpu")) for n in (("up", "gate", "down_t") if has_gate else ("up", "down_t"))}
    idx = node(G.mul_mat(fc1, F, "mlp_pre_hidden"))
    idx = node(G.relu(idx, "mlp_pre_relu"))
    idx = node(G.mul_mat(fc2, idx, "mlp_pre_out"))
    up = node(G.mul_mat_idx(W["up"], cur, idx, None, "ffn_up_sparse"))
    if has_gate:
        gate = node(G.mul_mat_idx(W["gate"], cur, idx, None, "ffn_gate_sparse"))
        act = node(G.relu(gate, "ffn_gate_act"))
        h = node(G.mul(act, up, "ffn_gate_par"))
    else:
        h = node(G.relu(up, "ffn_up_act"))
    out = node(G.axpy(W["down_t"], h, idx, None, "ffn_down_sparse"))
    res = G.on_gpu(G.add(out, F, "l_out"))
    xn = ol.apply_norm(L["x"][0], norm, nw, nb if norm == 2 else None, 1e-5)
    return dict(idx=idx, h=h, out=out, res=res, xn=xn, extra=extra)


@pytest.mark.parametrize("d,ff,r,has_gate,norm", [(4096, 11008, 1024, True, 1), (4096, 2048, 512, False, 2), (8192, 4096, 512, False, 0),
                                                  (4096, 2048, 512, True, 0)])
def test_ffn_block_of_one_token_is_one_fused_launch(d, ff, r, has_gate, norm):
    """The node window of the boundary: the single-token sequence llm_build_ffn_sparse emits is held back node by node and computed as
    pi_k_gemv + pi_k_sparse_ffn (the residual add behind the AXPY node as its epilogue) when the window is flushed.  The output, the predictor logits and h are those of the node-by-node
    evaluation (and of the CPU oracle under the same logits); the counters show the block went through the fused path once."""
    from powerinfer_amd import lib as pl
    from ggml_graph import Graph
    Lc = pl.load()
    L = synth.make_ffn_layer(seed=17, d=d, ff=ff, r=r, wtype=ol.F16, has_gate=has_gate, T=1)
    got = {}
    for fuse in (1, 0):
        G = Graph(Lc)
        Lc.pi_ggml_backend_set_fusion(fuse)
        s0 = backend_stats(Lc)
        B = build_decode_ffn(G, L, norm, has_gate)
        G.compute(0.0)
        assert not G.cpu_run, G.cpu_run
        got[fuse] = {k: G.host(B[k]).copy() for k in ("idx", "h", "out", "res")}
        s1 = backend_stats(Lc)
        assert s1["fused"] - s0["fused"] == fuse
        if fuse:
            assert s1["deferred"] - s0["deferred"] >= (6 if has_gate else 5) + (0 if norm == 0 else norm + 1)
        else:
            assert s1["deferred"] == s0["deferred"]
        lg = got[fuse]["idx"]
        o = ol.ffn_under_logits(ol.oracle(), d, ff, ol.F16, has_gate, L["up"], L["gate"], L["down_t"], B["xn"], lg, 0.0)
        if not fuse:          # fused, the residual add is the block's epilogue: the AXPY node's own vector is not written (nothing but that add reads it)
            assert rel_err(got[fuse]["out"], o["out"]) < 1e-4
        assert rel_err(got[fuse]["h"], o["h"]) < 1e-4 if "h" in o else True
        assert rel_err(got[fuse]["res"], o["out"] + L["x"][0]) < 1e-4
    Lc.pi_ggml_backend_set_fusion(1)
    assert rel_err(got[1]["idx"], got[0]["idx"]) < 1e-5
    assert ((got[1]["idx"] >= 0) == (got[0]["idx"] >= 0)).mean() >= 0.999
    assert np.array_equal(got[1]["h"] != 0, (got[1]["idx"] >= 0) & (got[1]["h"] != 0))     # h is zero wherever the predictor says inactive


@pytest.mark.parametrize("spoiler", ["mlp_pre_out", "ffn_up_sparse", "ffn_gate_act"])
def test_an_unrelated_node_breaks_the_window(spoiler):
    """A node that is not part of the block arrives in the middle of it: everything pending runs, in order, before it, nothing is
    fused, and every intermediate vector exists as in a node-by-node evaluation."""
    from powerinfer_amd import lib as pl
    from ggml_graph import Graph
    Lc = pl.load()
    d, ff, r = 4096, 2048, 512
    L = synth.make_ffn_layer(seed=19, d=d, ff=ff, r=r, wtype=ol.F16, has_gate=True, T=1)
    Lc.pi_ggml_backend_set_fusion(1)
    G = Graph(Lc)
    s0 = backend_stats(Lc)
    B = build_decode_ffn(G, L, 1, True, spoiler=spoiler)
    G.compute(0.0)
    s1 = backend_stats(Lc)
    assert s1["fused"] == s0["fused"] and s1["flushed"] > s0["flushed"]
    lg = G.host(B["idx"])
    o = ol.ffn_under_logits(ol.oracle(), d, ff, ol.F16, True, L["up"], L["gate"], L["down_t"], B["xn"], lg, 0.0)
    assert rel_err(G.host(B["out"]), o["out"]) < 1e-4
    assert rel_err(G.host(B["extra"][0]), L["x"][0]) == 0.0
