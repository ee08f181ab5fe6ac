"""Writes the golden vectors under tests/golden/ by running the COMPILED REFERENCE
(oracle/_ref/libpi_ref.so = /root/reference/{ggml,ggml-quants,ggml-alloc,ggml-backend}.c + oracle/ref_harness.c)
on seeded inputs with n_threads = 1.  Only runs where /root/reference exists; the .npz files it
writes are committed and are what the CPU and GPU test suites read.

    python tests/golden/make_fixtures.py
"""
import hashlib
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import oracle_lib as ol  # noqa: E402
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from powerinfer_amd.synth import make_ffn_layer  # noqa: E402


def sha(*arrs):
    h = hashlib.sha256()
    for a in arrs:
        h.update(np.ascontiguousarray(a).tobytes())
    return h.hexdigest()


def save(name, **kw):
    path = os.path.join(HERE, name + ".npz")
    np.savez_compressed(path, **kw)
    print(f"{name}: {os.path.getsize(path) / 1024:.1f} KiB")


def ffn_case(R, name, seed, d, ff, r, T, wtype, has_gate, hot_frac):
    rng = np.random.default_rng(seed)
    wf = lambda rows, cols, s: (rng.standard_normal((rows, cols)) * s).astype(np.float32)  # noqa: E731
    enc = (lambda a: a.astype(np.float16)) if wtype == ol.F16 else (lambda a: ol.quantize_q4_0(a, R))
    up, gate, down = enc(wf(ff, d, 0.02)), enc(wf(ff, d, 0.02)), enc(wf(ff, d, 0.02))
    fc1 = wf(r, d, 0.05).astype(np.float16)
    fc2 = wf(ff, r, 0.05).astype(np.float16)
    x = rng.standard_normal((T, d)).astype(np.float32)
    xp = rng.standard_normal((T, d)).astype(np.float32)
    gid = (rng.random(ff) < hot_frac).astype(np.int32)
    zero = np.zeros(ff, np.int32)
    cold = ol.ffn_sparse(R, d, ff, r, T, wtype, has_gate, up, gate, down, fc1, fc2, x, xp, zero, 0.0)
    part = ol.ffn_sparse(R, d, ff, r, T, wtype, has_gate, up, gate, down, fc1, fc2, x, xp, gid, 0.0)
    thr = ol.ffn_sparse(R, d, ff, r, T, wtype, has_gate, up, gate, down, fc1, fc2, x, xp, zero, 0.05)
    save(name, d=d, ff=ff, r=r, T=T, wtype=wtype, has_gate=has_gate, up=up, gate=gate, down_t=down, fc1=fc1, fc2=fc2,
         x_ffn=x, x_pred=xp, gpu_idx=gid,
         logits=cold["logits"], up_out=cold["up"], gate_out=cold["gate"], h=cold["h"], out=cold["out"],
         cpu_part_up=part["up"], cpu_part_h=part["h"], cpu_part_out=part["out"],
         thr05_h=thr["h"], thr05_out=thr["out"])


def ops_case(R):
    rng = np.random.default_rng(7)
    P = ol._ptr
    out = {}
    # dense mul_mat, F16 and Q4_0, n not a multiple of 32 for F16 (leftover path)
    for tag, wtype, rows, cols, T in (("mm_f16", ol.F16, 40, 200, 2), ("mm_q4", ol.Q4_0, 24, 256, 2)):
        w32 = (rng.standard_normal((rows, cols)) * 0.1).astype(np.float32)
        w = w32.astype(np.float16) if wtype == ol.F16 else ol.quantize_q4_0(w32, R)
        x = rng.standard_normal((T, cols)).astype(np.float32)
        y = np.zeros((T, rows), np.float32)
        assert R.ref_mul_mat(wtype, P(w), rows, cols, P(x), T, 1, P(y)) == 0
        out.update({tag + "_w": w, tag + "_x": x, tag + "_y": y})
    # norms
    x = (rng.standard_normal((3, 320)) * 2 + 0.3).astype(np.float32)
    for kind, tag in ((0, "rms"), (1, "ln")):
        y = np.zeros_like(x)
        assert R.ref_norm(kind, P(x), 320, 3, 1e-5, P(y)) == 0
        out[tag + "_y"] = y
    out["norm_x"] = x
    # rope, both pairings
    hd, nh, T = 64, 3, 4
    x = rng.standard_normal((T, nh, hd)).astype(np.float32)
    pos = np.array([0, 1, 17, 300], np.int32)
    for mode in (0, 2):
        y = np.zeros_like(x)
        assert R.ref_rope(P(x), hd, nh, T, P(pos), hd, mode, 10000.0, 1.0, P(y)) == 0
        out[f"rope{mode}_y"] = y
    out["rope_x"], out["rope_pos"] = x, pos
    # softmax with masked tail
    x = (rng.standard_normal((5, 77)) * 3).astype(np.float32)
    x[:, 60:] = -np.inf
    y = np.zeros_like(x)
    assert R.ref_soft_max(P(x), 77, 5, P(y)) == 0
    out["sm_x"], out["sm_y"] = x, y
    # codecs
    x = (rng.standard_normal(32 * 9) * np.repeat(10.0 ** rng.uniform(-3, 1, 9), 32)).astype(np.float32)
    x[64:96] = 0.0
    q4 = np.zeros(9 * 18, np.uint8)
    q8 = np.zeros(9 * 34, np.uint8)
    R.ref_quantize_row(ol.Q4_0, P(x), P(q4), x.size)
    R.ref_quantize_row_fast(8, P(x), P(q8), x.size)   # type 8 = Q8_0, the executor's from_float
    dq = np.zeros_like(x)
    R.ref_dequantize_row(ol.Q4_0, P(q4), P(dq), x.size)
    out.update(codec_x=x, codec_q4=q4, codec_q8=q8, codec_dq4=dq)
    # attention with GQA: prefill 5 tokens then one decode token
    hd, nh, nkv, nctx = 32, 4, 2, 48
    kc = np.zeros((nctx, nkv * hd), np.uint16)
    vc = np.zeros((nkv * hd, nctx), np.uint16)
    steps = []
    n_past = 0
    for T in (5, 1, 1):
        q = rng.standard_normal((T, nh, hd)).astype(np.float32)
        k = rng.standard_normal((T, nkv, hd)).astype(np.float32)
        v = rng.standard_normal((T, nkv * hd)).astype(np.float32)
        o = np.zeros((T, nh * hd), np.float32)
        assert R.ref_attention(hd, nh, nkv, nctx, n_past, T, P(q), P(k), P(v), P(kc), P(vc), P(o)) == 0
        steps.append((q, k, v, o))
        n_past += T
    for i, (q, k, v, o) in enumerate(steps):
        out.update({f"att{i}_q": q, f"att{i}_k": k, f"att{i}_v": v, f"att{i}_o": o})
    out["att_kc"], out["att_vc"] = kc, vc
    save("ops", **out)


def layer7b_case(R):
    """One 7B-shaped layer (config 0), inputs regenerated from the seed by powerinfer_amd/synth.py; only the
    outputs (and a hash of the inputs) are stored."""
    L = make_ffn_layer(seed=1234, d=4096, ff=11008, r=1024, wtype=ol.F16)
    zero = np.zeros(L["ff"], np.int32)
    o = ol.ffn_sparse(R, 4096, 11008, 1024, 1, ol.F16, 1, L["up"], L["gate"], L["down_t"], L["fc1"], L["fc2"],
                      L["x"], L["x"], zero, 0.0)
    active = np.nonzero(o["logits"][0] >= 0.0)[0].astype(np.int32)
    sample = np.random.default_rng(5).choice(11008, 512, replace=False).astype(np.int32)
    save("layer7b_f16", input_sha=np.frombuffer(bytes.fromhex(sha(L["up"], L["gate"], L["down_t"], L["fc1"], L["fc2"], L["x"])), np.uint8),
         active=active, sample_idx=sample, logits_sample=o["logits"][0][sample], h_sample=o["h"][0][sample], out=o["out"][0])
    print("layer7b active:", active.size, "of 11008")


ROPE_SCALED_CASES = (     # (tag, mode, n_orig_ctx, freq_scale, ext_factor, attn_factor, beta_fast, beta_slow)
    ("lin0", 0, 0, 0.25, 0.0, 1.0, 32.0, 1.0),            # linear scaling, LLaMA pairs
    ("lin2", 2, 0, 0.5, 0.0, 1.0, 32.0, 1.0),             # linear scaling, NeoX halves (the reference applies the factor twice there)
    ("yarn0", 0, 256, 0.25, 1.0, 1.0, 32.0, 1.0),         # YaRN: ramp between the correction dimensions, magnitude correction
    ("yarn0b", 0, 128, 0.125, 0.7, 1.3, 16.0, 2.0),
    ("yarn2", 2, 256, 0.25, 1.0, 1.0, 32.0, 1.0),
)


def rope_scaled_case(R):
    """ggml_rope_custom with its scaling operands (ggml.c:11124-11161): a file of its own, so that ops.npz keeps its random stream."""
    P = ol._ptr
    rng = np.random.default_rng(77)
    hd, nh, T = 64, 3, 5
    x = rng.standard_normal((T, nh, hd)).astype(np.float32)
    pos = np.array([0, 1, 17, 300, 2047], np.int32)
    out = dict(x=x, pos=pos)
    for tag, mode, n_orig, fs, ext, attn, bf, bs in ROPE_SCALED_CASES:
        y = np.zeros_like(x)
        assert R.ref_rope_ext(P(x), hd, nh, T, P(pos), hd, mode, n_orig, 10000.0, fs, ext, attn, bf, bs, P(y)) == 0
        out[tag] = y
    save("rope_scaled", **out)


if __name__ == "__main__":
    R = ol.ref()
    assert R is not None, "needs /root/reference"
    if len(sys.argv) > 1 and sys.argv[1] == "rope_scaled":
        rope_scaled_case(R)
        sys.exit(0)
    ffn_case(R, "ffn_f16_gate", 11, 64, 1024, 32, 3, ol.F16, 1, 0.6)
    ffn_case(R, "ffn_f16_nogate", 12, 64, 1024, 32, 2, ol.F16, 0, 0.6)
    ffn_case(R, "ffn_q4_gate", 13, 64, 1024, 32, 3, ol.Q4_0, 1, 0.6)
    ffn_case(R, "ffn_q4_nogate", 14, 128, 1056, 32, 1, ol.Q4_0, 0, 0.6)
    ops_case(R)
    rope_scaled_case(R)
    layer7b_case(R)
