"""Pins the CPU restatement against what the mathematics fixes, independently of the golden vectors:
library fp16 rounding, an independent numpy Q4_0 codec, fp64 dense algebra with an all-true mask,
the hybrid-split invariant, the RoPE composition invariant of the reference's own tests/test-rope.cpp,
and the loose codec error bounds of tests/test-quantize-fns.cpp."""
import numpy as np
import pytest

import oracle_lib as ol
from oracle_lib import _ptr as P
from powerinfer_amd import synth


def test_fp16_rounding_matches_ieee():
    O = ol.oracle()
    rng = np.random.default_rng(0)
    xs = np.concatenate([
        rng.standard_normal(20000).astype(np.float32) * 10.0 ** rng.uniform(-9, 6, 20000).astype(np.float32),
        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e9, -1e9, 5.96e-8, 2.98e-8, 2.9802322e-8, 2.9802326e-8,
                  6.1035156e-5, 6.097555e-5, np.inf, -np.inf], np.float32),
        # exact ties between adjacent halfs: must round to even
        (np.arange(1024, 2048, dtype=np.float32) + 0.5) / 1024.0,
    ])
    with np.errstate(over="ignore"):
        want = xs.astype(np.float16).view(np.uint16)
    got = np.array([O.pio_f32_to_f16(float(v)) for v in xs], np.uint16)
    assert np.array_equal(got, want)
    row = np.zeros(xs.size, np.uint16)
    O.pio_f32_to_f16_row(P(xs), P(row), xs.size)          # the F16C path the hot loops use
    assert np.array_equal(row, want)
    allh = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    back = np.array([O.pio_f16_to_f32(int(h)) for h in allh], np.float32)
    ref = allh.view(np.float16).astype(np.float32)
    ok = np.isnan(ref) | (back.view(np.uint32) == ref.view(np.uint32))
    assert ok.all()


def test_q4_0_codec_vs_independent_numpy_and_error_bound():
    O = ol.oracle()
    rng = np.random.default_rng(1)
    x = (rng.standard_normal((7, 256)) * 0.3).astype(np.float32)
    x[2, 32:64] = 0
    q = ol.quantize_q4_0(x)
    assert np.array_equal(q, synth.quantize_q4_0(x))
    dq = np.zeros_like(x)
    for i in range(7):
        O.pio_dequantize_row_q4_0(P(q[i]), P(dq[i]), 256)
    assert np.array_equal(dq, synth.dequantize_q4_0(q, 256))
    # tests/test-quantize-fns.cpp:16-20,114-166: cosine signal, RMSE(quantize -> dequantize) < 0.002
    n = 32 * 128
    sig = (0.1 + 2 * np.cos(np.arange(n, dtype=np.float32))).astype(np.float32)
    qs = ol.quantize_q4_0(sig[None])[0]
    ds = np.zeros(n, np.float32)
    O.pio_dequantize_row_q4_0(P(qs), P(ds), n)
    assert np.sqrt(np.mean((ds - sig) ** 2)) / n ** 0.5 < 0.002   # the reference divides the L2 error by n
    # Q8_0: |x - d*q| <= d/2 and q of the largest element is +-127
    q8 = np.zeros(n // 32 * 34, np.uint8)
    O.pio_quantize_row_q8_0(P(sig), P(q8), n)
    b = q8.reshape(-1, 34)
    d = b[:, :2].copy().view(np.float16).astype(np.float32)[:, 0]
    qi = b[:, 2:].view(np.int8).astype(np.float32)
    assert np.abs(qi).max(axis=1).min() == 127
    assert (np.abs(sig.reshape(-1, 32) - qi * d[:, None]) <= d[:, None] * 0.6 + 1e-6).all()   # half a step + the fp16 rounding of d (2^-11 * 127 steps)


def test_vec_dots_vs_float64():
    O = ol.oracle()
    rng = np.random.default_rng(2)
    for n in (32, 96, 200, 4096):
        a = rng.standard_normal(n).astype(np.float16)
        b = rng.standard_normal(n).astype(np.float16)
        want = float(a.astype(np.float64) @ b.astype(np.float64))
        assert abs(O.pio_vec_dot_f16(n, P(a), P(b)) - want) <= 2e-6 * np.abs(a.astype(np.float64) * b.astype(np.float64)).sum()
    n = 4096
    w = (rng.standard_normal(n) * 0.02).astype(np.float32)
    x = rng.standard_normal(n).astype(np.float32)
    qw = ol.quantize_q4_0(w[None])[0]
    q8 = np.zeros(n // 32 * 34, np.uint8)
    O.pio_quantize_row_q8_0(P(x), P(q8), n)
    b = q8.reshape(-1, 34)
    xd = b[:, 2:].view(np.int8).astype(np.float64) * b[:, :2].copy().view(np.float16).astype(np.float64)
    want = float(synth.dequantize_q4_0(qw, n).astype(np.float64) @ xd.reshape(-1))
    assert abs(O.pio_vec_dot_q4_0_q8_0(n, P(qw), P(q8)) - want) < 1e-5 * max(1.0, abs(want))


@pytest.mark.parametrize("wtype", [ol.F16, ol.Q4_0])
@pytest.mark.parametrize("has_gate", [1, 0])
def test_all_true_mask_reduces_to_dense_algebra(wtype, has_gate):
    """threshold = -inf: every row is active, so the block is relu(gate.x) * (up.x) then down^T . h."""
    O = ol.oracle()
    rng = np.random.default_rng(3)
    d, ff, r, T = 128, 1024, 32, 2
    w32 = lambda rows, cols: (rng.standard_normal((rows, cols)) * 0.05).astype(np.float32)  # noqa: E731
    up32, gate32, down32 = w32(ff, d), w32(ff, d), w32(ff, d)
    up, gate, down = (synth.encode(a, wtype) for a in (up32, gate32, down32))
    fc1, fc2 = w32(r, d).astype(np.float16), w32(ff, r).astype(np.float16)
    x = rng.standard_normal((T, d)).astype(np.float32)
    o = ol.ffn_sparse(O, d, ff, r, T, wtype, has_gate, up, gate, down, fc1, fc2, x, x, np.zeros(ff, np.int32), -np.inf)
    if wtype == ol.F16:
        deq = lambda a: a.astype(np.float64)  # noqa: E731
        xr = x.astype(np.float16).astype(np.float64)
    else:
        deq = lambda a: synth.dequantize_q4_0(a, d).astype(np.float64)  # noqa: E731
        q8 = np.zeros((T, d // 32 * 34), np.uint8)
        for t in range(T):
            O.pio_quantize_row_q8_0(P(x[t]), P(q8[t]), d)
        b = q8.reshape(T, -1, 34)
        xr = (b[..., 2:].view(np.int8).astype(np.float64) * b[..., :2].copy().view(np.float16).astype(np.float64)).reshape(T, d)
    upo = xr @ deq(up).T
    np.testing.assert_allclose(o["up"], upo, rtol=1e-5, atol=1e-6)
    h = np.maximum(xr @ deq(gate).T, 0) * upo if has_gate else np.maximum(upo, 0)
    np.testing.assert_allclose(o["h"], h, rtol=2e-5, atol=1e-6)
    # the down projection sees h rounded to its dot type; compare against the oracle's own h to isolate axpy
    hq = o["h"].astype(np.float64)
    if wtype == ol.F16:
        hq = o["h"].astype(np.float16).astype(np.float64)
    else:
        q8 = np.zeros((T, ff // 32 * 34), np.uint8)
        for t in range(T):
            O.pio_quantize_row_q8_0(P(o["h"][t]), P(q8[t]), ff)
        b = q8.reshape(T, -1, 34)
        hq = (b[..., 2:].view(np.int8).astype(np.float64) * b[..., :2].copy().view(np.float16).astype(np.float64)).reshape(T, ff)
    np.testing.assert_allclose(o["out"], hq @ deq(down), rtol=1e-4, atol=2e-6)
    # predictor = two dense layers
    hid = np.maximum(x.astype(np.float16).astype(np.float64) @ fc1.astype(np.float64).T, 0)
    lg = hid.astype(np.float32).astype(np.float16).astype(np.float64) @ fc2.astype(np.float64).T
    np.testing.assert_allclose(o["logits"], lg, rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("wtype", [ol.F16, ol.Q4_0])
def test_hybrid_split_invariant(wtype):
    """CPU share (gpu_idx) + complementary share == everything computed, up to fp32 summation order;
    a share writes exact zeros outside its own neurons."""
    O = ol.oracle()
    L = synth.make_ffn_layer(seed=5, d=128, ff=1024, r=32, wtype=wtype, mean_rate=0.3, T=2)
    gid, bucket = synth.gpu_split(L["p"], 0.6)
    assert gid.sum() == bucket.size == 614 and (np.diff(bucket) > 0).all() and (gid[bucket] == 1).all()
    args = (128, 1024, 32, 2, wtype, 1, L["up"], L["gate"], L["down_t"], L["fc1"], L["fc2"], L["x"], L["x"])
    full = ol.ffn_sparse(O, *args, np.zeros(1024, np.int32), 0.0)
    cold = ol.ffn_sparse(O, *args, gid, 0.0)
    hot = ol.ffn_sparse(O, *args, 1 - gid, 0.0)
    assert (cold["up"][:, gid == 1] == 0).all() and (hot["up"][:, gid == 0] == 0).all()
    assert np.array_equal(cold["up"] + hot["up"], full["up"])
    if wtype == ol.F16:   # Q8_0 block scales of h depend on which neurons share a block, so only F16 is linear
        np.testing.assert_allclose(cold["out"] + hot["out"], full["out"], rtol=1e-4, atol=1e-6)


def test_rope_composition_invariant():
    """tests/test-rope.cpp:137-215: rope(rope(x, p0), p1 - p0) == rope(x, p1)."""
    O = ol.oracle()
    rng = np.random.default_rng(6)
    hd, nh, T = 128, 2, 3
    x = rng.standard_normal((T, nh, hd)).astype(np.float32)
    p0 = np.array([3, 50, 200], np.int32)
    p1 = np.array([40, 51, 333], np.int32)
    for mode in (0, 2):
        a, b, c = (np.zeros_like(x) for _ in range(3))
        O.pio_rope(P(x), hd, nh, T, P(p0), hd, mode, 10000.0, 1.0, P(a))
        O.pio_rope(P(a), hd, nh, T, P(p1 - p0), hd, mode, 10000.0, 1.0, P(b))
        O.pio_rope(P(x), hd, nh, T, P(p1), hd, mode, 10000.0, 1.0, P(c))
        assert np.abs(b - c).max() / np.abs(c).max() < 1e-4
        np.testing.assert_allclose(np.linalg.norm(c, axis=-1), np.linalg.norm(x, axis=-1), rtol=1e-5)
    # position 0 is the identity; closed form for one pair
    O.pio_rope(P(x), hd, nh, T, P(np.zeros(3, np.int32)), hd, 0, 10000.0, 1.0, P(a))
    assert np.array_equal(a, x)
    O.pio_rope(P(x), hd, nh, T, P(p1), hd, 0, 10000.0, 1.0, P(a))
    th = 333 * 10000.0 ** (-2 * 5 / hd)
    want = x[2, 1, 10] * np.cos(th) - x[2, 1, 11] * np.sin(th)
    assert abs(a[2, 1, 10] - want) < 2e-4
    O.pio_rope(P(x), hd, nh, T, P(p1), hd, 2, 10000.0, 1.0, P(a))
    want = x[2, 1, 5] * np.cos(th) - x[2, 1, 5 + hd // 2] * np.sin(th)
    assert abs(a[2, 1, 5] - want) < 2e-4


def test_norms_and_softmax_closed_form():
    O = ol.oracle()
    rng = np.random.default_rng(7)
    x = rng.standard_normal((2, 512)).astype(np.float32) * 3 + 1
    y = np.zeros_like(x)
    O.pio_rms_norm(P(x), 512, 2, 1e-5, P(y))
    np.testing.assert_allclose(y, x / np.sqrt((x.astype(np.float64) ** 2).mean(-1, keepdims=True) + 1e-5), rtol=1e-6)
    O.pio_norm(P(x), 512, 2, 1e-5, P(y))
    xc = x.astype(np.float64) - x.astype(np.float64).mean(-1, keepdims=True)
    np.testing.assert_allclose(y, xc / np.sqrt((xc ** 2).mean(-1, keepdims=True) + 1e-5), rtol=1e-5, atol=1e-6)
    s = rng.standard_normal((3, 100)).astype(np.float32) * 4
    p = np.zeros_like(s)
    O.pio_soft_max(P(s), 100, 3, P(p))
    e = np.exp(s.astype(np.float64) - s.max(-1, keepdims=True))
    np.testing.assert_allclose(p.sum(-1), 1, rtol=1e-6)
    np.testing.assert_allclose(p, e / e.sum(-1, keepdims=True), rtol=1.5e-2, atol=1e-6)   # exp table indexed by fp16(x - max): error grows as |x - max| * 2^-11


def test_active_list_is_ascending_compaction():
    O = ol.oracle()
    rng = np.random.default_rng(8)
    lg = rng.standard_normal(11008).astype(np.float32)
    lg[[3, 77]] = [0.0, -0.0]                                # both count as active: the test is !(x < thr)
    lst = np.zeros(11008, np.int32)
    n = O.pio_active_list(P(lg), 11008, 0.0, P(lst))
    assert np.array_equal(lst[:n], np.nonzero(lg >= 0)[0]) and 3 in lst[:n] and 77 in lst[:n]
    assert O.pio_active_list(P(lg), 0, 0.0, P(lst)) == 0
    assert O.pio_active_list(P(lg), 11008, np.inf, P(lst)) == 0


def test_zipf_predictor_hits_target_rate():
    L = synth.make_ffn_layer(seed=9, d=512, ff=4096, r=128, mean_rate=0.10, T=8)
    O = ol.oracle()
    o = ol.ffn_sparse(O, 512, 4096, 128, 8, ol.F16, 1, L["up"], L["gate"], L["down_t"], L["fc1"], L["fc2"], L["x"], L["x"],
                      np.zeros(4096, np.int32), 0.0, nth=4)
    rate = (o["logits"] >= 0).mean()
    assert 0.07 < rate < 0.13
    hot = np.argsort(-L["p"])[:100]
    assert (o["logits"][:, hot] >= 0).mean() > 0.8


def test_reference_arithmetic_is_chaotic_under_last_bit_noise():
    """Why model-level parity is statistical.  The CPU path rounds activations to fp16 (F16 weights) or to
    int8 blocks (Q4_0 weights) before every dot product, so a perturbation in the LAST BIT of one fp32 input
    is amplified by many orders of magnitude within a couple of layers, and flips neurons whose predictor
    logit sits on the threshold.  Any implementation that sums in a different order than the scalar CPU loop
    differs by more than that last bit, so per-token bit-level agreement of a whole model is not attainable;
    agreement is asserted per operator (tight), per layer on identical inputs (tight) and statistically over
    trajectories."""
    for wt, floor in ((ol.F16, 1e-5), (ol.Q4_0, 1e-4)):
        hp = synth.hparams("llama-tiny", n_ctx=32, seed=3, wtype=wt)
        m = synth.make_model(hp)
        m2 = dict(hp=hp, glob=m["glob"], layers=[dict(L) for L in m["layers"]])
        noise = np.random.default_rng(0).standard_normal(hp.n_embd)
        m2["layers"][0]["attn_norm"] = (m["layers"][0]["attn_norm"] * (1 + 1e-7 * noise)).astype(np.float32)
        a, b = ol.OracleModel(m), ol.OracleModel(m2)
        worst, n = 0.0, 0
        for t in np.random.default_rng(1).integers(0, hp.n_vocab, 6):
            _, la = a.eval([int(t)], n, nth=4)
            _, lb = b.eval([int(t)], n, nth=4)
            n += 1
            worst = max(worst, float(np.abs(la - lb).max() / np.abs(la).max()))
        assert worst > floor, (wt, worst)       # 1e-7 in, > 1e-5 (F16) / > 1e-4 (Q4_0) out
        a.close(), b.close()


def test_q4_reference_departs_from_itself_beyond_the_logit_tolerance():
    """The 1e-2 logits tolerance is not a property the reference's Q4_0 path has against ITSELF over a 72-token trajectory: moving the
    FFN norm weights by one fp32 ulp (less than any other summation order changes) moves some int8 roundings of the activations,
    the difference stays in the KV cache and grows.  Both runs consume the same tokens.  With F16 weights the same experiment stays
    near 1e-3.  Hence the model-level GPU tests hold Q4_0 logits to the tolerance on the median and protect every greedy decision
    by its margin, and hold F16 logits to it on every token."""
    worst = {}
    for wt, seed in ((ol.Q4_0, 25), (ol.F16, 23)):
        hp = synth.hparams("llama-tiny", seed=seed, wtype=wt, pred_margin=True, head_pair=2048)
        m = synth.make_model(hp)
        m2 = dict(hp=hp, glob=m["glob"], layers=[dict(L) for L in m["layers"]])
        rng = np.random.default_rng(5)
        for L in m2["layers"]:
            w = L["ffn_norm"].copy()
            bits = w.view(np.int32)
            bits += rng.integers(-1, 2, bits.shape).astype(np.int32)
            L["ffn_norm"] = w
        a, b = ol.OracleModel(m), ol.OracleModel(m2)
        prompt = np.random.default_rng(seed + 7).integers(0, hp.n_vocab, 8)
        cur, w = None, 0.0
        for s in range(72):
            tok = int(prompt[s]) if s < 8 else cur
            cur, la = a.eval([tok], s, nth=4)
            _, lb = b.eval([tok], s, nth=4)
            w = max(w, float(np.abs(la - lb).max() / np.abs(la).max()))
        worst[wt] = w
        a.close(), b.close()
    assert worst[ol.Q4_0] > 1e-2, worst
    assert worst[ol.F16] < 5e-3, worst


def test_sparse_mul_mat_dispatch_rule_of_the_executor():
    """ggml.c:14904-14927: MUL_MAT_SPARSE goes to the threshold kernel only when the predictor output is wider than 1000; narrower
    nodes take a different kernel (one flag per 128 rows, fixed cut at -7) that no model shape reaches.  The oracle restates the
    first and refuses the second rather than answer with the wrong rule; AXPY without its aux tensor is refused likewise (the
    reference's F16 kernel skips every row then, ggml.c:14424)."""
    O = ol.oracle()
    rng = np.random.default_rng(0)
    for rows, want in ((1000, 4), (1001, 0), (1024, 0)):
        w = (rng.standard_normal((rows, 64)) * 0.1).astype(np.float16)
        x = rng.standard_normal(64).astype(np.float32)
        idx = rng.standard_normal(rows).astype(np.float32)
        out = np.zeros(rows, np.float32)
        rc = O.pio_mul_mat_sparse(ol.F16, ol._ptr(w), rows, 64, ol._ptr(x), 1, ol._ptr(idx), ol._ptr(np.zeros(rows, np.int32)), 0.0, ol._ptr(out), 1)
        assert rc == want, (rows, rc)
        if rc == 0:
            assert np.array_equal(out != 0, idx >= 0)
    h = rng.standard_normal(1024).astype(np.float32)
    wt = (rng.standard_normal((1024, 64)) * 0.1).astype(np.float16)
    assert O.pio_axpy(ol.F16, ol._ptr(wt), 1024, 64, ol._ptr(h), 1, ol._ptr(h), None, 0.0, ol._ptr(np.zeros(64, np.float32)), 1) == 3
