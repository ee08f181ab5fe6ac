"""HIP sparse-FFN kernels (through the C ABI) against the CPU oracle and the reference's golden vectors.

Tolerances (north star): index lists bit-exact for an identical mask; masks agree on >= 99.9 % of neurons;
FFN output within 2e-3 relative error (measured here as max |diff| / max |ref|)."""
import numpy as np
import pytest

import oracle_lib as ol
from powerinfer_amd import synth

pytestmark = pytest.mark.gpu

FFN_REL_TOL = 2e-3
MASK_AGREE = 0.999


def rel_err(a, b):
    return float(np.abs(a - b).max() / max(np.abs(b).max(), 1e-30))


def under(L, d, ff, wtype, has_gate, xn, logits, thr=0.0, gpu_idx=None):
    """The CPU oracle's FFN for the mask the GPU's own predictor logits imply: the output comparison then never depends on a
    neuron whose logit sits on the threshold having fallen the same way on both sides."""
    return ol.ffn_under_logits(ol.oracle(), d, ff, wtype, has_gate, L["up"], L["gate"], L["down_t"], xn, logits, thr, gpu_idx)


def check_token(g, o, ff, thr=0.0, gid=None):
    """g: GPU result dict for one token, o: oracle dict rows for the same token."""
    mask_g = np.zeros(ff, bool)
    cand = np.arange(ff) if gid is None else gid
    mask_g[cand[g["active"]]] = True
    mask_o = ~(o["logits"] < thr)
    if gid is not None:
        keep = np.zeros(ff, bool)
        keep[gid] = True
        mask_o &= keep
    agree = (mask_g == mask_o).mean()
    assert agree >= MASK_AGREE, agree
    # identical mask => identical list: the list must be exactly the ascending indices of the GPU's own mask
    own = ~(g["logits"] < thr)
    want = np.nonzero(own)[0] if gid is None else np.nonzero(own[gid])[0]
    assert np.array_equal(g["active"], want)
    assert rel_err(g["logits"], o["logits"]) < 1e-4
    same = mask_g == mask_o
    return same


@pytest.mark.parametrize("name", ["ffn_f16_gate", "ffn_f16_nogate", "ffn_q4_gate", "ffn_q4_nogate"])
def test_ffn_vs_reference_golden(golden, name):
    from powerinfer_amd.ops import SparseFFN
    g = golden(name)
    d, ff, r, T, wt, hg = (int(g[k]) for k in ("d", "ff", "r", "T", "wtype", "has_gate"))
    ffn = SparseFFN(d, ff, r, wt, g["up"], g["gate"] if hg else None, g["down_t"], g["fc1"], g["fc2"])
    for t in range(T):
        res = ffn.forward(g["x_ffn"][t], g["x_pred"][t])
        assert np.array_equal(res["active"], np.nonzero(g["logits"][t] >= 0)[0])
        assert rel_err(res["logits"], g["logits"][t]) < 1e-5
        assert rel_err(res["up"], g["up_out"][t]) < 1e-5
        if hg:
            assert rel_err(res["gate"], g["gate_out"][t]) < 1e-5
        assert rel_err(res["h"], g["h"][t]) < 1e-5
        assert rel_err(res["out"], g["out"][t]) < 1e-4
    ffn.close()


@pytest.mark.parametrize("wtype", [ol.F16, ol.Q4_0])
@pytest.mark.parametrize("has_gate", [True, False])
def test_ffn_7b_shape_vs_oracle(wtype, has_gate):
    """Config 0: one 7B-shaped layer, Zipf predictor, all neurons on the GPU."""
    from powerinfer_amd.ops import SparseFFN
    d, ff, r, T = 4096, 11008, 1024, 3
    L = synth.make_ffn_layer(seed=21 + wtype, d=d, ff=ff, r=r, wtype=wtype, has_gate=has_gate, T=T)
    O = ol.oracle()
    o = ol.ffn_sparse(O, d, ff, r, T, wtype, has_gate, L["up"], L["gate"], L["down_t"], L["fc1"], L["fc2"], L["x"], L["x"],
                      np.zeros(ff, np.int32), 0.0, nth=8)
    ffn = SparseFFN(d, ff, r, wtype, L["up"], L["gate"], L["down_t"], L["fc1"], L["fc2"])
    for t in range(T):
        res = ffn.forward(L["x"][t], L["x"][t])
        ot = {k: v[t] for k, v in o.items()}
        check_token(res, ot, ff)
        assert 600 < res["active"].size < 1700
        ou = under(L, d, ff, wtype, has_gate, L["x"][t], res["logits"])
        assert rel_err(res["up"], ou["up"]) < 1e-5
        assert rel_err(res["h"], ou["h"]) < 1e-4
        assert rel_err(res["out"], ou["out"]) < (1e-4 if wtype == ol.F16 else FFN_REL_TOL)      # F16: fp32 summation order only
        # fused route (what the decode loop runs): the up/gate kernel builds the list from the mask words itself
        fus = ffn.forward(L["x"][t], L["x"][t], dense_outputs=False)
        assert np.array_equal(fus["active"], res["active"])
        assert np.array_equal(fus["h_compact"], res["h_compact"])
        assert rel_err(fus["out"], res["out"]) < 1e-5
    ffn.close()


@pytest.mark.parametrize("route", ["one", "two"])
@pytest.mark.parametrize("has_gate", [True, False])
@pytest.mark.parametrize("norm", [0, 1, 2])
def test_fused_routes_7b_shape(has_gate, norm, route):
    """pi_k_sparse_ffn (what the F16 decode loop runs at d = 4096) and pi_k_pred_upgate + pi_k_sparse_axpy_dense
    against the oracle, with the fused RMSNorm / LayerNorm prologue and the residual epilogue."""
    run_fused_route(has_gate, norm, route, 4096, 11008, 1024)


@pytest.mark.parametrize("has_gate,norm", [(False, 2), (True, 1)])
def test_one_launch_route_wide_rows(has_gate, norm):
    """The 8192-column instantiation (Falcon-40B width; each lane holds two 8-column chunks), rank-512 predictor."""
    run_fused_route(has_gate, norm, "one", 8192, 4096, 512)


@pytest.mark.parametrize("has_gate,norm", [(True, 1), (False, 2), (True, 0)])
def test_one_launch_route_13b_layer(has_gate, norm):
    """One FFN block at the 13B shape (13824 x 5120, predictor rank 1280 = two and a half chunks of 512): ten waves per workgroup, one
    workgroup per compute unit, the last half chunk of the predictor rows read by half the lanes."""
    from powerinfer_amd import lib as pl
    assert pl.load().pi_k_sparse_ffn_supported(13824, 1280, 5120) == 1
    assert pl.load().pi_k_sparse_ffn_hot_supported(13824, 1280, 5120) == 0          # hybrid layers of this width keep the list kernels
    assert pl.load().pi_k_sparse_ffn_workgroups(13824, 1280, 5120) == 256
    run_fused_route(has_gate, norm, "one", 5120, 13824, 1280, T=2)


def test_one_launch_route_falcon40b_layer():
    """One FFN block at the full Falcon-40B shape (32768 x 8192, no gate, LayerNorm, rank 1024): the instantiation in which a
    workgroup takes four groups of 32 neurons and stores one partial vector for all of them."""
    run_fused_route(False, 2, "one", 8192, 32768, 1024, T=1, mean_rate=0.08)


def run_fused_route(has_gate, norm, route, d, ff, r, T=3, mean_rate=0.10):
    from powerinfer_amd import lib as pl
    from powerinfer_amd.ops import SparseFFN
    L = synth.make_ffn_layer(seed=77 + norm, d=d, ff=ff, r=r, wtype=ol.F16, has_gate=has_gate, T=T, mean_rate=mean_rate)
    rng = np.random.default_rng(5)
    nw = (1 + 0.1 * rng.standard_normal(d)).astype(np.float32) if norm else None
    nb = (0.1 * rng.standard_normal(d)).astype(np.float32) if norm == 2 else None
    eps = 1e-5
    O = ol.oracle()
    P = ol._ptr
    ffn = SparseFFN(d, ff, r, ol.F16, L["up"], L["gate"], L["down_t"], L["fc1"], L["fc2"], norm_kind=norm, norm_w=nw, norm_b=nb, eps=eps)
    for t in range(T):
        x = np.ascontiguousarray(L["x"][t:t + 1], np.float32)
        xn = x.copy()
        if norm == 1:
            O.pio_rms_norm(P(x), d, 1, eps, P(xn)); xn = np.ascontiguousarray(xn * nw, np.float32)
        elif norm == 2:
            O.pio_norm(P(x), d, 1, eps, P(xn)); xn = np.ascontiguousarray(xn * nw + nb, np.float32)
        o = ol.ffn_sparse(O, d, ff, r, 1, ol.F16, has_gate, L["up"], L["gate"], L["down_t"], L["fc1"], L["fc2"], xn, x,
                          np.zeros(ff, np.int32), 0.0, nth=8)
        resid = rng.standard_normal(d).astype(np.float32)
        res = (ffn.forward_one_launch if route == "one" else ffn.forward_two_launch)(x[0], x[0], epilogue=pl.EPI_ADD, resid=resid)
        assert rel_err(res["logits"], o["logits"][0]) < 1e-4
        mask_g, mask_o = ~(res["logits"] < 0.0), ~(o["logits"][0] < 0.0)
        assert (mask_g == mask_o).mean() >= MASK_AGREE
        assert res["n_active"] == int(mask_g.sum())
        assert not np.isnan(res["h"]).any()
        assert np.all(res["h"][~mask_g] == 0.0)               # every inactive neuron written as 0
        ou = under(L, d, ff, ol.F16, has_gate, xn, res["logits"])
        assert rel_err(res["h"], ou["h"]) < 1e-4
        assert rel_err(res["out"] - resid, ou["out"]) < 1e-4
    ffn.close()


def q8_blocks_np(v):
    """Q8_0 over blocks of 32 as quantize_row_q8_0 does on x86 (ggml-quants.c:702-760): returns (q int32, d float32 per element)."""
    v = np.asarray(v, np.float32).reshape(-1, 32)
    amax = np.abs(v).max(1)
    d = (amax / np.float32(127.0)).astype(np.float32)
    idv = np.where(amax != 0, np.float32(127.0) / np.where(amax != 0, amax, 1), 0).astype(np.float32)
    q = np.rint(v * idv[:, None]).astype(np.int32)
    return q.reshape(-1), np.repeat(d.astype(np.float16).astype(np.float32), 32)


def q4_rows_np(raw, rows, d):
    """(nibble - 8) [len(rows), d] int32 and the fp32 block scales [len(rows), d/32] of Q4_0 rows."""
    b = raw[rows].reshape(len(rows), d // 32, 18)
    dw = b[:, :, :2].copy().view(np.float16).astype(np.float32)[:, :, 0]
    qs = b[:, :, 2:]
    v = np.concatenate([qs & 0x0F, qs >> 4], axis=2).astype(np.int32) - 8
    return v.reshape(len(rows), d), dw


@pytest.mark.parametrize("has_gate", [True, False])
@pytest.mark.parametrize("norm", [0, 1, 2])
def test_q4_fused_route_7b_shape(has_gate, norm):
    """pi_k_pred_upgate_q4 + pi_k_axpy_q4_partials/_reduce (what the Q4_0 decode loop runs at d = 4096), all neurons resident,
    against the oracle; the Q8_0 blocks the kernel hands to a host share are checked against the closed form."""
    from powerinfer_amd import lib as pl
    from powerinfer_amd.ops import SparseFFN
    d, ff, r, T = 4096, 11008, 1024, 3
    L = synth.make_ffn_layer(seed=90 + norm, d=d, ff=ff, r=r, wtype=ol.Q4_0, has_gate=has_gate, T=T)
    rng = np.random.default_rng(6)
    nw = (1 + 0.1 * rng.standard_normal(d)).astype(np.float32) if norm else None
    nb = (0.1 * rng.standard_normal(d)).astype(np.float32) if norm == 2 else None
    eps = 1e-5
    O, P = ol.oracle(), ol._ptr
    ffn = SparseFFN(d, ff, r, ol.Q4_0, L["up"], L["gate"], L["down_t"], L["fc1"], L["fc2"], norm_kind=norm, norm_w=nw, norm_b=nb, eps=eps)
    for t in range(T):
        x = np.ascontiguousarray(L["x"][t:t + 1], np.float32)
        xn = x.copy()
        if norm == 1:
            O.pio_rms_norm(P(x), d, 1, eps, P(xn)); xn = np.ascontiguousarray(xn * nw, np.float32)
        elif norm == 2:
            O.pio_norm(P(x), d, 1, eps, P(xn)); xn = np.ascontiguousarray(xn * nw + nb, np.float32)
        o = ol.ffn_sparse(O, d, ff, r, 1, ol.Q4_0, has_gate, L["up"], L["gate"], L["down_t"], L["fc1"], L["fc2"], xn, x,
                          np.zeros(ff, np.int32), 0.0, nth=8)
        resid = rng.standard_normal(d).astype(np.float32)
        res = ffn.forward_q4_fused(x[0], x[0], epilogue=pl.EPI_ADD, resid=resid)
        assert rel_err(res["logits"], o["logits"][0]) < 1e-4
        mask_g, mask_o = ~(res["logits"] < 0.0), ~(o["logits"][0] < 0.0)
        assert (mask_g == mask_o).mean() >= MASK_AGREE
        assert res["n_active"] == int(mask_g.sum())
        assert not np.isnan(res["h"]).any()
        assert np.all(res["h"][~mask_g] == 0.0)
        # Q8_0 blocks of the normalised input: int8 values may differ by one step where the norm differs in the last place
        blocks = res["xq8"].reshape(d // 32, 34)
        qg = blocks[:, 2:].copy().view(np.int8).astype(np.int32).reshape(-1)
        dg = np.repeat(blocks[:, :2].copy().view(np.float16).astype(np.float32)[:, 0], 32)
        qo, do = q8_blocks_np(xn[0])
        assert np.abs(qg - qo).max() <= 1 and (qg != qo).mean() < 1e-3
        assert np.allclose(dg, do, rtol=2e-3)
        ou = under(L, d, ff, ol.Q4_0, has_gate, xn, res["logits"])
        assert rel_err(res["h"], ou["h"]) < 1e-4
        assert rel_err(res["out"] - resid, ou["out"]) < FFN_REL_TOL     # an int8 step of h where h * 127/amax sits on a rounding boundary
    ffn.close()


@pytest.mark.parametrize("has_gate,norm,hot_frac", [(True, 1, 1.0), (False, 2, 1.0), (True, 1, 0.6), (False, 0, 0.5)])
def test_q4_one_launch_route_7b_shape(has_gate, norm, hot_frac):
    """pi_k_sparse_ffn_q4_partials + pi_k_sparse_ffn_q4_reduce: the Q4_0 layer in one launch plus the reduction, every neuron's rows
    in one set of matrices or split into a compact resident set and the others (ascending).  Against the CPU reference evaluated
    under the device's own logits, and against the two-launch route (same arithmetic per element, partial sums grouped by 32 neurons
    instead of 128)."""
    from powerinfer_amd import lib as pl
    from powerinfer_amd.ops import SparseFFN
    d, ff, r, T = 4096, 11008, 1024, 2
    L = synth.make_ffn_layer(seed=70 + norm, d=d, ff=ff, r=r, wtype=ol.Q4_0, has_gate=has_gate, T=T)
    rng = np.random.default_rng(7)
    nw = (1 + 0.1 * rng.standard_normal(d)).astype(np.float32) if norm else None
    nb = (0.1 * rng.standard_normal(d)).astype(np.float32) if norm == 2 else None
    eps = 1e-5
    O, P = ol.oracle(), ol._ptr
    bucket, rest = None, None
    if hot_frac < 1.0:
        gid, bucket = synth.gpu_split(L["p"], hot_frac)
        cold = np.flatnonzero(gid != 1)
        rest = (L["up"][cold], L["gate"][cold] if has_gate else None, L["down_t"][cold])
    ffn = SparseFFN(d, ff, r, ol.Q4_0, L["up"], L["gate"], L["down_t"], L["fc1"], L["fc2"], bucket=bucket, norm_kind=norm, norm_w=nw, norm_b=nb, eps=eps)
    ref2 = SparseFFN(d, ff, r, ol.Q4_0, L["up"], L["gate"], L["down_t"], L["fc1"], L["fc2"], norm_kind=norm, norm_w=nw, norm_b=nb, eps=eps)
    for t in range(T):
        x = np.ascontiguousarray(L["x"][t:t + 1], np.float32)
        xn = x.copy()
        if norm == 1:
            O.pio_rms_norm(P(x), d, 1, eps, P(xn)); xn = np.ascontiguousarray(xn * nw, np.float32)
        elif norm == 2:
            O.pio_norm(P(x), d, 1, eps, P(xn)); xn = np.ascontiguousarray(xn * nw + nb, np.float32)
        resid = rng.standard_normal(d).astype(np.float32)
        res = ffn.forward_q4_one_launch(x[0], x[0], epilogue=pl.EPI_ADD, resid=resid, rest=rest)
        two = ref2.forward_q4_fused(x[0], x[0], epilogue=pl.EPI_ADD, resid=resid)
        assert np.array_equal(res["logits"], two["logits"]) and np.array_equal(res["h"], two["h"])
        assert res["n_active"] == two["n_active"] == int((~(res["logits"] < 0.0)).sum())
        assert rel_err(res["out"], two["out"]) < 1e-5
        ou = under(L, d, ff, ol.Q4_0, has_gate, xn, res["logits"])
        assert rel_err(res["h"], ou["h"]) < 1e-4
        assert rel_err(res["out"] - resid, ou["out"]) < FFN_REL_TOL
    ffn.close(), ref2.close()


@pytest.mark.parametrize("has_gate,norm", [(True, 1), (False, 2)])
def test_f16_fused_route_hybrid_share(has_gate, norm):
    """The fused F16 kernels on a hot/cold split at the 7B width: the resident 60 % come from compact matrices through the hot
    words / prefix; their output must equal what the oracle computes for exactly those neurons (gpu_idx inverted), and the
    normalised fp16 input handed to the host share must be the oracle's."""
    from powerinfer_amd.ops import SparseFFN
    d, ff, r, T = 4096, 4096, 512, 2
    L = synth.make_ffn_layer(seed=35 + norm, d=d, ff=ff, r=r, wtype=ol.F16, has_gate=has_gate, mean_rate=0.15, T=T)
    gid, bucket = synth.gpu_split(L["p"], 0.6)
    rng = np.random.default_rng(8)
    nw = (1 + 0.1 * rng.standard_normal(d)).astype(np.float32)
    nb = (0.1 * rng.standard_normal(d)).astype(np.float32) if norm == 2 else None
    eps = 1e-5
    O, P = ol.oracle(), ol._ptr
    ffn = SparseFFN(d, ff, r, ol.F16, L["up"], L["gate"], L["down_t"], L["fc1"], L["fc2"], bucket=bucket, norm_kind=norm, norm_w=nw, norm_b=nb, eps=eps)
    for t in range(T):
        x = np.ascontiguousarray(L["x"][t:t + 1], np.float32)
        xn = x.copy()
        if norm == 1:
            O.pio_rms_norm(P(x), d, 1, eps, P(xn)); xn = np.ascontiguousarray(xn * nw, np.float32)
        else:
            O.pio_norm(P(x), d, 1, eps, P(xn)); xn = np.ascontiguousarray(xn * nw + nb, np.float32)
        share = ol.ffn_sparse(O, d, ff, r, 1, ol.F16, has_gate, L["up"], L["gate"], L["down_t"], L["fc1"], L["fc2"], xn, x, 1 - gid, 0.0)
        res = ffn.forward_one_launch_hot(x[0], x[0])
        mask_g, mask_o = ~(res["logits"] < 0.0), ~(share["logits"][0] < 0.0)
        assert rel_err(res["logits"], share["logits"][0]) < 1e-4
        assert res["n_active"] == int((mask_g & (gid == 1)).sum())
        assert np.all(res["h"][gid == 0] == 0.0) and np.all(res["h"][~mask_g] == 0.0)
        assert (res["xn16"] != xn[0].astype(np.float16)).mean() < 1e-3              # a last-place step of the norm at most
        assert (mask_g == mask_o).mean() >= MASK_AGREE
        su = under(L, d, ff, ol.F16, has_gate, xn, res["logits"], gpu_idx=1 - gid)      # the resident neurons only, under the GPU's mask
        assert rel_err(res["h"], su["h"]) < 1e-4
        assert rel_err(res["out"], su["out"]) < 1e-4
    ffn.close()


def test_q4_fused_route_hybrid_share():
    """Hot/cold split at the 7B width: the kernels see only the resident 60 % (compact matrices, hot words / prefix); with the
    cold neurons' h filled in before the down projection, GPU share + cold share (numpy, same Q8_0 blocks of h) must equal the
    oracle computing every neuron."""
    from powerinfer_amd.ops import SparseFFN
    d, ff, r, T = 4096, 4096, 512, 2
    L = synth.make_ffn_layer(seed=33, d=d, ff=ff, r=r, wtype=ol.Q4_0, mean_rate=0.15, T=T)
    gid, bucket = synth.gpu_split(L["p"], 0.6)
    O = ol.oracle()
    full = ol.ffn_sparse(O, d, ff, r, T, ol.Q4_0, 1, L["up"], L["gate"], L["down_t"], L["fc1"], L["fc2"], L["x"], L["x"], np.zeros(ff, np.int32), 0.0)
    ffn = SparseFFN(d, ff, r, ol.Q4_0, L["up"], L["gate"], L["down_t"], L["fc1"], L["fc2"], bucket=bucket)
    for t in range(T):
        cold = gid == 0
        got = {}

        def fill(h):
            assert np.all(h[cold] == 0.0)                       # the kernel writes zeros outside its share
            # every neuron on the CPU under the logits the GPU just produced: the cold neurons' h comes from there
            got["full"] = under(L, d, ff, ol.Q4_0, True, L["x"][t], ffn.logits.download(np.float32))
            h[cold] = got["full"]["h"][cold]
            return h

        res = ffn.forward_q4_fused(L["x"][t], L["x"][t], fill_h=fill)
        fu = got["full"]
        mask_g, mask_o = ~(res["logits"] < 0.0), ~(full["logits"][t] < 0.0)
        assert rel_err(res["logits"], full["logits"][t]) < 1e-4
        assert (mask_g == mask_o).mean() >= MASK_AGREE
        assert res["n_active"] == int((mask_g & ~cold).sum())
        assert rel_err(res["h"][~cold], fu["h"][~cold]) < 1e-4
        hm = res["h"].copy(); hm[cold] = fu["h"][cold]
        q, dh = q8_blocks_np(hm)
        rows = np.nonzero(cold & (q != 0))[0]
        v, dw = q4_rows_np(L["down_t"], rows, d)
        contrib = (v * q[rows, None]).astype(np.float32) * (np.repeat(dw, 32, axis=1) * dh[rows, None])
        cold_out = contrib.sum(0, dtype=np.float32)
        assert rel_err(res["out"] + cold_out, fu["out"]) < FFN_REL_TOL
    ffn.close()


def test_q4_hybrid_layer_with_stream_handovers():
    """The hybrid Q4_0 layer as the decode loop queues it: predictor, signal, resident up/gate rows, signal, wait, down projection,
    wait, reduction - all queued at once, the host share (here numpy, from the logits and the Q8_0 input the device wrote to pinned
    memory) computed while the stream waits for it.  The resident share is bit-identical to the route with a launch boundary per
    exchange (pi_k_pred_upgate_q4 -> fill h -> axpy -> reduce), and GPU share + host share equals every neuron on the CPU."""
    from powerinfer_amd.ops import SparseFFN
    d, ff, r = 4096, 4096, 512
    L = synth.make_ffn_layer(seed=34, d=d, ff=ff, r=r, wtype=ol.Q4_0, mean_rate=0.15, T=1)
    gid, bucket = synth.gpu_split(L["p"], 0.6)
    cold = gid == 0
    ffn = SparseFFN(d, ff, r, ol.Q4_0, L["up"], L["gate"], L["down_t"], L["fc1"], L["fc2"], bucket=bucket)
    x = L["x"][0]
    ref, got = {}, {}

    def fill(h):
        ref["full"] = under(L, d, ff, ol.Q4_0, True, x, ffn.logits.download(np.float32))
        h[cold] = ref["full"]["h"][cold]
        return h
    base = ffn.forward_q4_fused(x, x, fill_h=fill)

    def cold_share(hm):
        q, dh = q8_blocks_np(hm)
        rows = np.nonzero(cold & (q != 0))[0]
        v, dw = q4_rows_np(L["down_t"], rows, d)
        contrib = (v * q[rows, None]).astype(np.float32) * (np.repeat(dw, 32, axis=1) * dh[rows, None])
        return contrib.sum(0, dtype=np.float32)

    def host_h(logits, xq8):
        assert np.array_equal(xq8, base["xq8"])                # the Q8_0 blocks of the normalised input, as the one-launch route writes them
        got["full"] = under(L, d, ff, ol.Q4_0, True, x, logits)
        act = np.nonzero(cold & ~(logits < 0.0))[0]
        return {int(j): got["full"]["h"][j] for j in act}

    def host_out(h_full):
        got["h_full"] = h_full
        return cold_share(h_full)
    res = ffn.forward_q4_handover(x, x, host_h, host_out)
    assert res["status"] == 0
    assert np.array_equal(res["logits"], base["logits"])
    thr_bits = np.packbits(~(base["logits"] < ffn.thr), bitorder="little").view(np.uint32)
    assert np.array_equal(res["words"], thr_bits)               # the activity words the host lists its neurons from
    hm = base["h"].copy(); hm[cold] = ref["full"]["h"][cold]
    assert np.array_equal(got["h_full"], hm)                    # resident entries from the device, the others from the host, zeros elsewhere
    assert res["n_active"] == base["n_active"]
    assert np.array_equal(res["out"], base["out"] + cold_share(hm))      # same partial sums, host share added by the reduction
    assert rel_err(res["out"], got["full"]["out"]) < FFN_REL_TOL

    ffn.close()


@pytest.mark.parametrize("wtype", [ol.F16, ol.Q4_0])
def test_hybrid_split_gpu_share(wtype):
    """Config 2 split: the GPU holds the hottest 60 % of neurons (compact matrices + gpu_bucket) and
    produces exactly the share the CPU skips: CPU_part(gpu_idx) + GPU_part == all neurons."""
    from powerinfer_amd.ops import SparseFFN
    d, ff, r = 1024, 4096, 128
    L = synth.make_ffn_layer(seed=31, d=d, ff=ff, r=r, wtype=wtype, mean_rate=0.2, T=2)
    gid, bucket = synth.gpu_split(L["p"], 0.6)
    O = ol.oracle()
    args = (d, ff, r, 2, wtype, 1, L["up"], L["gate"], L["down_t"], L["fc1"], L["fc2"], L["x"], L["x"])
    full = ol.ffn_sparse(O, *args, np.zeros(ff, np.int32), 0.0)
    gpu_share = ol.ffn_sparse(O, *args, 1 - gid, 0.0)          # oracle computing only the GPU's neurons
    ffn = SparseFFN(d, ff, r, wtype, L["up"], L["gate"], L["down_t"], L["fc1"], L["fc2"], bucket=bucket)
    for t in range(2):
        res = ffn.forward(L["x"][t], L["x"][t])
        check_token(res, {k: v[t] for k, v in full.items()}, ff, gid=bucket)
        assert (res["up"][gid == 0] == 0).all()                # upscale writes bucket positions only
        su = under(L, d, ff, wtype, True, L["x"][t], res["logits"], gpu_idx=1 - gid)      # the GPU's neurons under the GPU's mask
        assert rel_err(res["up"], su["up"]) < 1e-5
        assert rel_err(res["logits"], gpu_share["logits"][t]) < 1e-4
        if wtype == ol.F16:                                    # Q8_0 scales of h need the merged h (tested at model level)
            assert rel_err(res["out"], su["out"]) < 1e-4
    ffn.close()


def test_threshold_and_empty_list():
    from powerinfer_amd.ops import SparseFFN
    d, ff, r = 256, 1024, 64
    L = synth.make_ffn_layer(seed=41, d=d, ff=ff, r=r)
    O = ol.oracle()
    for thr in (0.05, 1e9, -1e9):
        o = ol.ffn_sparse(O, d, ff, r, 1, ol.F16, 1, L["up"], L["gate"], L["down_t"], L["fc1"], L["fc2"], L["x"], L["x"],
                          np.zeros(ff, np.int32), thr)
        ffn = SparseFFN(d, ff, r, ol.F16, L["up"], L["gate"], L["down_t"], L["fc1"], L["fc2"], threshold=thr)
        res = ffn.forward(L["x"][0], L["x"][0])
        assert np.array_equal(res["active"], np.nonzero(~(o["logits"][0] < thr))[0])
        if thr == 1e9:
            assert res["active"].size == 0 and (res["out"] == 0).all()
        if thr == -1e9:
            assert res["active"].size == ff
        assert np.abs(res["out"] - o["out"][0]).max() <= 1e-4 * max(np.abs(o["out"][0]).max(), 1e-6)
        ffn.close()


@pytest.mark.parametrize("route", ["one", "two"])
def test_fused_routes_thresholds_none_some_all(route):
    """The fused kernels at the extremes of the activity test: nothing active (zero output), a raised threshold, and every
    neuron active (32 per workgroup: the chunk loop of the one-launch kernel runs four times, the dense-h axpy compacts all ff
    rows in several passes)."""
    from powerinfer_amd.ops import SparseFFN
    d, ff, r = 4096, 2048, (512 if route == "one" else 1024)
    L = synth.make_ffn_layer(seed=43, d=d, ff=ff, r=r)
    O = ol.oracle()
    for thr in (1e9, 0.02, -1e9):
        o = ol.ffn_sparse(O, d, ff, r, 1, ol.F16, 1, L["up"], L["gate"], L["down_t"], L["fc1"], L["fc2"], L["x"], L["x"],
                          np.zeros(ff, np.int32), thr, nth=8)
        ffn = SparseFFN(d, ff, r, ol.F16, L["up"], L["gate"], L["down_t"], L["fc1"], L["fc2"], threshold=thr)
        res = (ffn.forward_one_launch if route == "one" else ffn.forward_two_launch)(L["x"][0], L["x"][0])
        mask_g, mask_o = ~(res["logits"] < thr), ~(o["logits"][0] < thr)
        assert res["n_active"] == int(mask_g.sum())
        if thr == 1e9:
            assert res["n_active"] == 0 and (res["out"] == 0).all() and (res["h"] == 0).all()
        if thr == -1e9:
            assert res["n_active"] == ff
        assert (mask_g == mask_o).mean() >= MASK_AGREE
        ou = under(L, d, ff, ol.F16, True, L["x"][0], res["logits"], thr)
        assert np.abs(res["out"] - ou["out"]).max() <= 1e-4 * max(np.abs(ou["out"]).max(), 1e-6)
        ffn.close()


def test_axpy_is_deterministic_and_linear():
    """Size-independent properties at full 7B shape: repeated launches are bit-identical (no float atomics),
    and the block output is linear in the down matrix (down_t * 2 doubles the output exactly)."""
    from powerinfer_amd.ops import SparseFFN
    d, ff, r = 4096, 11008, 1024
    L = synth.make_ffn_layer(seed=51, d=d, ff=ff, r=r)
    a = SparseFFN(d, ff, r, ol.F16, L["up"], L["gate"], L["down_t"], L["fc1"], L["fc2"])
    r1 = a.forward(L["x"][0], L["x"][0], dense_outputs=False)
    r2 = a.forward(L["x"][0], L["x"][0], dense_outputs=False)
    assert np.array_equal(r1["out"], r2["out"]) and np.array_equal(r1["active"], r2["active"])
    b = SparseFFN(d, ff, r, ol.F16, L["up"], L["gate"], (L["down_t"].astype(np.float32) * 2).astype(np.float16), L["fc1"], L["fc2"])
    r3 = b.forward(L["x"][0], L["x"][0], dense_outputs=False)
    assert np.array_equal(r3["out"], 2 * r1["out"])
    a.close(), b.close()
