"""The CPU restatement (oracle/pi_oracle.c) against golden vectors written by the compiled reference
(tests/golden/make_fixtures.py, n_threads = 1).  The restatement keeps the reference's lane-wise
accumulation order, so agreement is expected at fp32 round-off; index lists must be identical."""
import numpy as np
import pytest

import oracle_lib as ol
from oracle_lib import _ptr as P

TOL = dict(rtol=2e-6, atol=2e-7)


@pytest.mark.parametrize("name", ["ffn_f16_gate", "ffn_f16_nogate", "ffn_q4_gate", "ffn_q4_nogate"])
def test_ffn_block_matches_reference(golden, name):
    g = golden(name)
    O = ol.oracle()
    d, ff, r, T, wt, hg = (int(g[k]) for k in ("d", "ff", "r", "T", "wtype", "has_gate"))
    args = (d, ff, r, T, wt, hg, g["up"], g["gate"], g["down_t"], g["fc1"], g["fc2"], g["x_ffn"], g["x_pred"])
    zero = np.zeros(ff, np.int32)
    cold = ol.ffn_sparse(O, *args, zero, 0.0)
    np.testing.assert_allclose(cold["logits"], g["logits"], **TOL)
    # index lists: bit-exact
    for t in range(T):
        lst = np.zeros(ff, np.int32)
        n = O.pio_active_list(P(cold["logits"][t]), ff, 0.0, P(lst))
        assert np.array_equal(lst[:n], np.nonzero(g["logits"][t] >= 0.0)[0])
    np.testing.assert_allclose(cold["up"], g["up_out"], **TOL)
    if hg:
        np.testing.assert_allclose(cold["gate"], g["gate_out"], **TOL)
    np.testing.assert_allclose(cold["h"], g["h"], **TOL)
    np.testing.assert_allclose(cold["out"], g["out"], rtol=2e-5, atol=2e-6)
    part = ol.ffn_sparse(O, *args, g["gpu_idx"], 0.0)
    np.testing.assert_allclose(part["up"], g["cpu_part_up"], **TOL)
    np.testing.assert_allclose(part["out"], g["cpu_part_out"], rtol=2e-5, atol=2e-6)
    thr = ol.ffn_sparse(O, *args, zero, 0.05)
    np.testing.assert_allclose(thr["h"], g["thr05_h"], **TOL)
    np.testing.assert_allclose(thr["out"], g["thr05_out"], rtol=2e-5, atol=2e-6)
    assert (thr["h"] != 0).sum() < (cold["h"] != 0).sum()


def test_dense_mul_mat(golden):
    g = golden("ops")
    O = ol.oracle()
    for tag, wt in (("mm_f16", ol.F16), ("mm_q4", ol.Q4_0)):
        w, x, y = g[tag + "_w"], g[tag + "_x"], g[tag + "_y"]
        T, rows = y.shape
        cols = x.shape[1]
        out = np.zeros_like(y)
        assert O.pio_mul_mat(wt, P(w), rows, cols, P(x), T, P(out), 1) == 0
        np.testing.assert_allclose(out, y, **TOL)


def test_norms(golden):
    g = golden("ops")
    O = ol.oracle()
    x = g["norm_x"]
    y = np.zeros_like(x)
    O.pio_rms_norm(P(x), x.shape[1], x.shape[0], 1e-5, P(y))
    assert np.array_equal(y, g["rms_y"])
    O.pio_norm(P(x), x.shape[1], x.shape[0], 1e-5, P(y))
    assert np.array_equal(y, g["ln_y"])


def test_rope(golden):
    g = golden("ops")
    O = ol.oracle()
    x, pos = g["rope_x"], g["rope_pos"]
    T, nh, hd = x.shape
    for mode in (0, 2):
        y = np.zeros_like(x)
        O.pio_rope(P(x), hd, nh, T, P(pos), hd, mode, 10000.0, 1.0, P(y))
        np.testing.assert_allclose(y, g[f"rope{mode}_y"], rtol=0, atol=1e-6)


ROPE_SCALED_CASES = (     # as tests/golden/make_fixtures.py wrote them: (tag, mode, n_orig_ctx, freq_scale, ext_factor, attn_factor, beta_fast, beta_slow)
    ("lin0", 0, 0, 0.25, 0.0, 1.0, 32.0, 1.0), ("lin2", 2, 0, 0.5, 0.0, 1.0, 32.0, 1.0), ("yarn0", 0, 256, 0.25, 1.0, 1.0, 32.0, 1.0),
    ("yarn0b", 0, 128, 0.125, 0.7, 1.3, 16.0, 2.0), ("yarn2", 2, 256, 0.25, 1.0, 1.0, 32.0, 1.0))


def test_rope_with_linear_and_yarn_scaling(golden):
    """ggml_rope_custom's scaling operands against the compiled reference's outputs: linear scaling in both pairings (NeoX applies the
    factor twice, as the reference does), YaRN with its ramp and magnitude correction; and the unscaled call reduces to pio_rope."""
    g = golden("rope_scaled")
    O = ol.oracle()
    x, pos = g["x"], g["pos"]
    T, nh, hd = x.shape
    for tag, mode, n_orig, fs, ext, attn, bf, bs in ROPE_SCALED_CASES:
        y = np.zeros_like(x)
        O.pio_rope_ext(P(x), hd, nh, T, P(pos), hd, mode, n_orig, 10000.0, fs, ext, attn, bf, bs, P(y))
        np.testing.assert_allclose(y, g[tag], rtol=0, atol=2e-6, err_msg=tag)
        assert np.abs(y - x).max() > 0.1                              # the case rotates something
    for mode in (0, 2):
        a, b = np.zeros_like(x), np.zeros_like(x)
        O.pio_rope(P(x), hd, nh, T, P(pos), hd, mode, 10000.0, 1.0, P(a))
        O.pio_rope_ext(P(x), hd, nh, T, P(pos), hd, mode, 0, 10000.0, 1.0, 0.0, 1.0, 32.0, 1.0, P(b))
        assert np.array_equal(a, b)
    # the cases differ from one another and from the unscaled rotation: a dropped operand would not go unnoticed
    a = np.zeros_like(x)
    O.pio_rope(P(x), hd, nh, T, P(pos), hd, 0, 10000.0, 1.0, P(a))
    assert np.abs(g["lin0"] - a).max() > 0.1 and np.abs(g["yarn0"] - g["lin0"]).max() > 0.05 and np.abs(g["yarn0b"] - g["yarn0"]).max() > 0.05


def test_soft_max(golden):
    g = golden("ops")
    O = ol.oracle()
    x = g["sm_x"]
    y = np.zeros_like(x)
    O.pio_soft_max(P(x), x.shape[1], x.shape[0], P(y))
    np.testing.assert_allclose(y, g["sm_y"], rtol=1e-6, atol=0)
    assert (y[:, 60:] == 0).all()


def test_codecs(golden):
    g = golden("ops")
    O = ol.oracle()
    x = g["codec_x"]
    q4 = np.zeros_like(g["codec_q4"])
    q8 = np.zeros_like(g["codec_q8"])
    dq = np.zeros_like(x)
    O.pio_quantize_row_q4_0(P(x), P(q4), x.size)
    O.pio_quantize_row_q8_0(P(x), P(q8), x.size)
    O.pio_dequantize_row_q4_0(P(q4), P(dq), x.size)
    assert np.array_equal(q4, g["codec_q4"])
    assert np.array_equal(q8, g["codec_q8"])
    assert np.array_equal(dq, g["codec_dq4"])


def test_attention_steps(golden):
    g = golden("ops")
    O = ol.oracle()
    hd, nh, nkv, nctx = 32, 4, 2, 48
    kc = np.zeros((nctx, nkv * hd), np.uint16)
    vc = np.zeros((nkv * hd, nctx), np.uint16)
    n_past = 0
    for i in range(3):
        q, k, v, o_ref = (g[f"att{i}_{s}"] for s in "qkvo")
        T = q.shape[0]
        n_kv = n_past + T          # the harness attends exactly the filled cells
        slot = np.arange(n_past, n_past + T, dtype=np.int32)
        mask = np.where(np.arange(n_kv)[None, :] > slot[:, None], -np.inf, 0).astype(np.float32)
        o = np.zeros_like(o_ref)
        assert O.pio_attention(hd, nh, nkv, nctx, n_kv, T, P(slot), P(mask), P(q), P(k), P(v), P(kc), P(vc), P(o)) == 0
        np.testing.assert_allclose(o, o_ref, rtol=2e-6, atol=2e-7)
        n_past += T
    assert np.array_equal(kc, g["att_kc"]) and np.array_equal(vc, g["att_vc"])


def test_layer7b_shape(golden):
    """Config-0 layer at full 7B shape: inputs regenerated from the seed, outputs from the reference."""
    import hashlib
    from powerinfer_amd.synth import make_ffn_layer
    g = golden("layer7b_f16")
    L = make_ffn_layer(seed=1234, d=4096, ff=11008, r=1024, wtype=ol.F16)
    h = hashlib.sha256()
    for k in ("up", "gate", "down_t", "fc1", "fc2", "x"):
        h.update(np.ascontiguousarray(L[k]).tobytes())
    if not np.array_equal(np.frombuffer(h.digest(), np.uint8), g["input_sha"]):
        pytest.skip("numpy generates a different stream here than where the fixture was written")
    O = ol.oracle()
    o = ol.ffn_sparse(O, 4096, 11008, 1024, 1, ol.F16, 1, L["up"], L["gate"], L["down_t"], L["fc1"], L["fc2"],
                      L["x"], L["x"], np.zeros(11008, np.int32), 0.0, nth=4)
    lst = np.zeros(11008, np.int32)
    n = O.pio_active_list(P(o["logits"][0]), 11008, 0.0, P(lst))
    assert np.array_equal(lst[:n], g["active"])
    s = g["sample_idx"]
    np.testing.assert_allclose(o["logits"][0][s], g["logits_sample"], **TOL)
    np.testing.assert_allclose(o["h"][0][s], g["h_sample"], **TOL)
    # 4 threads: same terms, different summation order than the 1-thread reference
    np.testing.assert_allclose(o["out"][0], g["out"], rtol=1e-4, atol=1e-6)


@pytest.mark.parametrize("name", ["ffn_f16_gate", "ffn_f16_nogate", "ffn_q4_gate", "ffn_q4_nogate"])
def test_ffn_under_given_logits_reproduces_the_reference_block(golden, name):
    """oracle_lib.ffn_under_logits (the sparse mat-muls and the axpy driven by GIVEN predictor logits, which the GPU tests feed
    with the GPU's own logits) must return exactly what the compiled reference returned for the whole block when it is given
    the reference's logits."""
    g = golden(name)
    d, ff, T, wt, hg = (int(g[k]) for k in ("d", "ff", "T", "wtype", "has_gate"))
    for t in range(T):
        u = ol.ffn_under_logits(ol.oracle(), d, ff, wt, hg, g["up"], g["gate"] if hg else None, g["down_t"], g["x_ffn"][t], g["logits"][t], 0.0)
        assert np.array_equal(u["up"], g["up_out"][t])
        assert np.array_equal(u["h"], g["h"][t])
        assert np.array_equal(u["out"], g["out"][t])
