"""Seeded synthetic PowerInfer models (random-init weights of a given shape).

The reference ships no checkpoints; its loaders expect the tensors listed at llama.cpp:403-461
(`blk.N.{attn_q,...,ffn_gate,ffn_up,ffn_down_t,fc1,fc2}.weight`).  This module produces arrays with
those roles and shapes, in ggml's row-major layout (`[rows][ne0]`, ne0 contiguous).

Predictor.  The reference predictor is weight-only: logits = fc2 . relu(fc1 . x), neuron j is active
iff logit_j >= threshold (llama.cpp:4688-4695, ggml.c:14256).  To give neuron j a chosen firing rate
p_j without a bias tensor, fc2 row j is built as  b_j * u + eps_j  with u the unit all-ones direction and
eps_j ~ N(0, sigma^2 I).  For h = relu(fc1 . x) with Gaussian pre-activations, (u.h)/|h| concentrates
at 1/sqrt(pi), so P(logit_j >= 0) = Phi(b_j / (sigma * sqrt(pi))), independent of the scale of x and
fc1:  b_j = sigma * sqrt(pi) * Phi^-1(p_j).  Rates follow a Zipf(1.2) law over a seeded random ranking of
the neurons, clipped to [p_min, p_max] and normalised to the requested mean.
"""
import numpy as np
from scipy.special import ndtri

F32, F16, Q4_0, I32 = 0, 1, 2, 18   # enum ggml_type values (ggml.h:333-355)


def zipf_rates(ff, mean, rng, s=1.2, p_max=0.98, p_min=1e-4):
    """Per-neuron firing rates p_j ∝ rank_j^-s with the given mean; returns (p, rank)."""
    rank = rng.permutation(ff) + 1                    # rank 1 = hottest
    w = rank.astype(np.float64) ** (-s)
    p = np.minimum(w * (mean * ff / w.sum()), p_max)
    for _ in range(64):                               # water-filling: rescale the unclipped part
        free = p < p_max
        need = mean * ff - p_max * (~free).sum()
        scale = need / p[free].sum()
        if abs(scale - 1) < 1e-12:
            break
        p[free] = np.minimum(p[free] * scale, p_max)
    return np.maximum(p, p_min), rank


def predictor_fc2(ff, r, p, rng, sigma=0.02):
    b = sigma * np.sqrt(np.pi) * ndtri(p)
    eps = rng.standard_normal((ff, r), dtype=np.float32) * np.float32(sigma)
    return (eps + (b / np.sqrt(r)).astype(np.float32)[:, None]).astype(np.float16)


def predictor_fc2_margin(ff, r, p, rng, sigma=0.02, kappa=0.5):
    """A predictor whose decisions keep a margin from the threshold 0: row j = b_j * u + eps_j with |eps_j|_inf <= kappa * |b_j| / sqrt(r)
    and u the unit all-ones direction.  For the non-negative hidden vector h = relu(.) this gives |eps_j . h| <= kappa * |b_j| * (u . h),
    so logit_j = b_j * (u . h) + eps_j . h has the sign of b_j with a relative margin of 1 - kappa whatever the input: the round(mean * ff)
    neurons of highest rate p are active for every token, the others never, and a difference in the last places of the arithmetic
    cannot flip one.  The logits themselves still vary with the input."""
    n_on = int(round(float(np.mean(p)) * ff))
    on = np.zeros(ff, bool)
    on[np.argsort(-p, kind="stable")[:n_on]] = True
    b = np.where(on, 1.0, -1.0) * sigma * np.sqrt(np.pi) * (0.5 + rng.random(ff))          # |b_j| in sigma * sqrt(pi) * [0.5, 1.5)
    eps = (rng.random((ff, r), dtype=np.float32) * 2 - 1) * (kappa * np.abs(b) / np.sqrt(r)).astype(np.float32)[:, None]
    return (eps + (b / np.sqrt(r)).astype(np.float32)[:, None]).astype(np.float16)


# ---- a predictor whose active set moves with the token and still keeps a margin -------------------------------------------------
# Five coordinates of the residual stream are a side channel (MARK_DIMS): coordinate d-5 carries a constant for every token, coordinates
# d-4 .. d-1 carry a constant for token 0 .. 3 only (make_model writes them into the embeddings, keeps the attention output and the
# down projection away from them and hides them from the output matrix).  Five rows of fc1 read those coordinates, so the last five
# hidden units are MARK_GAIN * MARK_VALUE for the constant one and for the current token's own one (tokens 0..3), about zero otherwise.
MARK_DIMS, MARK_VALUE, MARK_GAIN = 5, 1.0, 8.0          # small enough to leave the norms alone (nothing else writes the channel: no noise to beat)


def predictor_fc2_moving(ff, r, p, rng, sigma=0.02, kappa=0.5, group_div=48):
    """Two classes of rows.  Four groups of ff // group_div neurons read only the marker units: row = g * (e_t - e_c / 2) for
    group t, so logit = g * MARK_GAIN * MARK_VALUE * (+1/2 if the current token is t, -1/2 otherwise): the group is active exactly
    while token t is being decoded (tokens 0..3, which is where the greedy path of a head_pair model lives), with a margin that does
    not depend on the layer or the input.  The other rows are predictor_fc2_margin's static-sign rows over the ordinary units, of
    which round(mean * ff) - ff // group_div are active for every token, so that a decoding step fires about mean * ff neurons.
    (With larger groups the token's own group dominates the block's output and the greedy path of a synthetic model settles on one
    token at once.)  Returns (fc2 fp16 [ff][r], rates [ff]): the rate of a moving neuron is 1/4 in groups 0 and 1 and next to nothing
    in groups 2 and 3, so that a split by rate (gpu_split) puts the first two on the device and the other two with the host share,
    which then has rows to compute whenever token 2 or 3 is decoded."""
    g = ff // group_div
    moving = np.sort(rng.permutation(ff)[:4 * g])
    static = np.setdiff1d(np.arange(ff), moving)
    n_on = max(int(round(float(np.mean(p)) * ff)) - g, 1)
    on = np.zeros(ff, bool)
    on[static[np.argsort(-p[static], kind="stable")[:n_on]]] = True
    ro = r - MARK_DIMS                                                     # ordinary hidden units
    b = np.where(on, 1.0, -1.0) * sigma * np.sqrt(np.pi) * (0.5 + rng.random(ff))
    eps = (rng.random((ff, ro), dtype=np.float32) * 2 - 1) * (kappa * np.abs(b) / np.sqrt(ro)).astype(np.float32)[:, None]
    w = np.zeros((ff, r), np.float32)
    w[:, :ro] = eps + (b / np.sqrt(ro)).astype(np.float32)[:, None]
    gain = np.float32(0.25)
    for t in range(4):
        rows = moving[t * g:(t + 1) * g]
        w[rows] = 0.0
        w[rows, ro] = -0.5 * gain                                          # the constant marker
        w[rows, ro + 1 + t] = gain                                         # token t's marker
    rates = np.where(on, 0.98, 1e-4)
    rates[moving[:2 * g]] = 0.25
    rates[moving[2 * g:]] = 1e-5            # groups 2 and 3 pass for rarely active: a hot/cold split by rate leaves them to the host
    return w.astype(np.float16), rates


def quantize_q4_0(x):
    """ggml Q4_0 (ggml-quants.c:428-463) in numpy: float32 [..., n] -> uint8 [..., n/32*18]."""
    x = np.ascontiguousarray(x, np.float32)
    n = x.shape[-1]
    b = x.reshape(-1, n // 32, 32)
    i = np.argmax(np.abs(b), axis=-1)                 # first element of largest magnitude
    mx = np.take_along_axis(b, i[..., None], -1)[..., 0]
    d = (mx / np.float32(-8)).astype(np.float32)
    idv = np.where(d != 0, np.float32(1) / np.where(d != 0, d, 1), 0).astype(np.float32)
    q = np.minimum(15, (b * idv[..., None] + np.float32(8.5)).astype(np.int8)).astype(np.uint8)
    out = np.empty(b.shape[:2] + (18,), np.uint8)
    out[..., :2] = d.astype(np.float16).view(np.uint8).reshape(b.shape[:2] + (2,))
    out[..., 2:] = q[..., :16] | (q[..., 16:] << 4)
    return out.reshape(x.shape[:-1] + (n // 32 * 18,))


def dequantize_q4_0(q, n):
    b = q.reshape(-1, n // 32, 18)
    d = b[..., :2].copy().view(np.float16).astype(np.float32)
    lo = (b[..., 2:] & 0x0F).astype(np.int8) - 8
    hi = (b[..., 2:] >> 4).astype(np.int8) - 8
    y = np.concatenate([lo, hi], -1).astype(np.float32) * d
    return y.reshape(q.shape[:-1] + (n,))


def encode(w32, wtype):
    return w32.astype(np.float16) if wtype == F16 else quantize_q4_0(w32)


def gpu_split(p, hot_frac):
    """Top `hot_frac` of neurons by firing rate go to the GPU (export_split.py:24-52 given the per-layer
    count): gpu_idx int32[ff] (1 = on GPU), gpu_bucket = sorted original indices of the GPU neurons."""
    ff = p.size
    n_hot = int(round(hot_frac * ff))
    hot = np.argsort(-p, kind="stable")[:n_hot]
    gpu_idx = np.zeros(ff, np.int32)
    gpu_idx[hot] = 1
    return gpu_idx, np.sort(hot).astype(np.int32)


def make_ffn_layer(seed, d, ff, r, wtype=F16, has_gate=True, mean_rate=0.10, T=1):
    """Config-0 style single sparse FFN layer: weights ~N(0, 0.02), activations ~N(0, 1)."""
    rng = np.random.default_rng(seed)
    nrm = lambda rows, cols, s: rng.standard_normal((rows, cols), dtype=np.float32) * np.float32(s)  # noqa: E731
    L = dict(d=d, ff=ff, r=r, wtype=wtype, has_gate=has_gate)
    L["up"] = encode(nrm(ff, d, 0.02), wtype)
    L["gate"] = encode(nrm(ff, d, 0.02), wtype) if has_gate else None
    L["down_t"] = encode(nrm(ff, d, 0.02), wtype)
    L["fc1"] = nrm(r, d, 0.02).astype(np.float16)
    L["p"], L["rank"] = zipf_rates(ff, mean_rate, rng)
    L["fc2"] = predictor_fc2(ff, r, L["p"], rng)
    L["x"] = rng.standard_normal((T, d), dtype=np.float32)
    return L


class HParams(dict):
    __getattr__ = dict.__getitem__


def hparams(name, **over):
    """Shapes of the benchmark configurations (d, ff, rank, heads, layers, vocab)."""
    base = {
        "llama-7b": dict(arch="llama", n_embd=4096, n_ff=11008, n_rank=1024, n_head=32, n_head_kv=32, n_layer=32,
                         n_vocab=32000, mean_rate=0.10),
        "llama-13b": dict(arch="llama", n_embd=5120, n_ff=13824, n_rank=1280, n_head=40, n_head_kv=40, n_layer=40,
                          n_vocab=32000, mean_rate=0.11),
        "falcon-40b": dict(arch="falcon", n_embd=8192, n_ff=32768, n_rank=1024, n_head=128, n_head_kv=8, n_layer=60,
                           n_vocab=65024, mean_rate=0.08),
        "llama-tiny": dict(arch="llama", n_embd=512, n_ff=4096, n_rank=128, n_head=8, n_head_kv=8, n_layer=3,
                           n_vocab=1024, mean_rate=0.15),
        "falcon-tiny": dict(arch="falcon", n_embd=512, n_ff=4096, n_rank=128, n_head=8, n_head_kv=2, n_layer=3,
                            n_vocab=1024, mean_rate=0.15),
    }[name]
    hp = HParams(base, name=name, n_ctx=512, wtype=F16, norm_eps=1e-5, rope_freq_base=10000.0, rope_freq_scale=1.0, sparse_threshold=0.0,
                 hot_frac=1.0, seed=0)
    hp.update(over)
    return hp


def make_model(hp):
    """All tensors of a synthetic model as numpy arrays: dict(glob={...}, layers=[{...}], hp=hp).
    Norm weights are 1 (biases 0); everything else ~N(0, 0.02) rounded to fp16 and then, for
    wtype == Q4_0, quantised (attention, FFN and output matrices; predictors stay fp16)."""
    rng = np.random.default_rng(hp.seed)
    d, ff, r = hp.n_embd, hp.n_ff, hp.n_rank
    gqa = d // hp.n_head * hp.n_head_kv
    wt = hp.wtype
    nrm = lambda rows, cols: (rng.standard_normal((rows, cols), dtype=np.float32) * np.float32(0.02)).astype(np.float16)  # noqa: E731
    enc = (lambda a: a) if wt == F16 else (lambda a: quantize_q4_0(a.astype(np.float32)))
    falcon = hp.arch == "falcon"
    tok_embd, output = nrm(hp.n_vocab, d), nrm(hp.n_vocab, d)
    if hp.get("head_pair"):
        # A greedy decision with a margin: output rows 0..3 are +c*w0, -c*w0, +c*w1, -c*w1 with c far above every other row, so
        # the next token is one of those four, chosen by which of the two projections w0 . x, w1 . x of the final state is larger
        # in magnitude and by its sign -- still a function of the whole network's state.  The winning logit is c * max(|w0 . x|,
        # |w1 . x|): both projections vanishing at once is quadratically rare, so the largest logit stays well conditioned, and
        # the runner-up comes close only where the two magnitudes happen to agree, which a test rules out for its seed by
        # measuring it.  (With i.i.d. random rows the two largest of tens of thousands of logits are within 0.4 % of the maximum
        # for one token in twenty, and any two correct implementations whose sums run in a different order then disagree on the
        # greedy token.)  The embeddings of tokens 0..3 are scaled down, so that once the path runs on those tokens the residual
        # stream comes from what attention and the FFNs add rather than from the current token's own embedding, and the path does
        # not settle on one token.
        for k in range(2):
            w = rng.standard_normal(d, dtype=np.float32) * np.float32(0.02 * hp.head_pair)
            output[2 * k], output[2 * k + 1] = w.astype(np.float16), (-w).astype(np.float16)
        for t in range(4):
            tok_embd[t] = (tok_embd[t].astype(np.float32) * np.float32(0.05)).astype(np.float16)
    moving = bool(hp.get("pred_moving"))
    if moving:
        assert hp.get("head_pair"), "pred_moving marks tokens 0..3, the tokens a head_pair model decodes"
        tok_embd[:, d - MARK_DIMS:] = 0
        tok_embd[:, d - MARK_DIMS] = MARK_VALUE
        for t in range(4):
            tok_embd[t, d - MARK_DIMS + 1 + t] = MARK_VALUE
        output[:, d - MARK_DIMS:] = 0                                      # the greedy choice does not look at the side channel
    glob = dict(tok_embd=enc(tok_embd), output_norm=np.ones(d, np.float32), output=enc(output))
    if falcon:
        glob["output_norm_b"] = np.zeros(d, np.float32)
    layers = []
    for _ in range(hp.n_layer):
        L = dict(attn_norm=np.ones(d, np.float32))
        def blind(w):                                                      # a matrix that does not read the side channel
            if moving:
                w[:, d - MARK_DIMS:] = 0
            return w
        if falcon:
            L["attn_norm_b"] = np.zeros(d, np.float32)
            if hp.n_head_kv != hp.n_head and hp.get("two_norms", True):
                L["attn_norm_2"] = np.ones(d, np.float32)
                L["attn_norm_2_b"] = np.zeros(d, np.float32)
            L["wqkv"] = enc(blind(nrm(d + 2 * gqa, d)))
        else:
            L["wq"], L["wk"], L["wv"] = enc(blind(nrm(d, d))), enc(blind(nrm(gqa, d))), enc(blind(nrm(gqa, d)))
            L["ffn_norm"] = np.ones(d, np.float32)
            L["ffn_gate"] = enc(blind(nrm(ff, d)))
        wo, up, down_t, fc1 = nrm(d, d), blind(nrm(ff, d)), nrm(ff, d), blind(nrm(r, d))
        if moving:                                                         # nothing writes into the side channel; only fc1's last rows read it
            wo[d - MARK_DIMS:, :] = 0
            down_t[:, d - MARK_DIMS:] = 0
            fc1[r - MARK_DIMS:, :] = 0
            for k in range(MARK_DIMS):
                fc1[r - MARK_DIMS + k, d - MARK_DIMS + k] = MARK_GAIN
        L["wo"] = enc(wo)
        L["ffn_up"] = enc(up)
        L["ffn_down_t"] = enc(down_t)
        L["fc1"] = fc1
        p, _ = zipf_rates(ff, hp.mean_rate, rng)
        if moving:
            L["fc2"], p = predictor_fc2_moving(ff, r, p, rng)
        else:
            L["fc2"] = predictor_fc2_margin(ff, r, p, rng) if hp.get("pred_margin") else predictor_fc2(ff, r, p, rng)
        L["p"] = p
        if hp.hot_frac < 1.0:
            L["gpu_idx"], L["gpu_bucket"] = gpu_split(p, hp.hot_frac)
        layers.append(L)
    if hp.get("vram_budget_gb") is not None:
        # --vram-budget: the planner decides how many neurons of each layer stay on the GPU (powerinfer_amd.split)
        from . import split
        splits, rep = split.plan_split(hp, [L["p"] for L in layers], hp.vram_budget_gb, hp.n_ctx, batch=hp.get("split_batch", 256))
        for L, (gi, gb) in zip(layers, splits):
            if gb.size:
                L["gpu_idx"], L["gpu_bucket"] = gi, gb
        hp["split_report"] = rep
    return dict(hp=hp, glob=glob, layers=layers)
