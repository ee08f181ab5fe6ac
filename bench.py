#!/usr/bin/env python3
"""Benchmark of the sparse decode token loop on one MI355X.

Workload (BASELINE.json configs[1]): 32-layer ReLU-LLaMA-2-7B-shaped model, random-init FP16 weights generated
in HBM, per-layer rank-1024 predictors with Zipf(1.2) firing rates (~10 % of neurons active), all neurons on
the GPU; a 64-token random prompt, then greedy decode at batch 1.  One "step" = one decoded token.

    python bench.py [--gpus 1] [--steps 256] [--warmup 8]

Prints ONE JSON line: decode tok/s, the HBM roofline of the kernel that moves the most bytes per token
(measured here with HIP events on the engine's stream), the touched-bytes accounting of the whole token
loop, and a CPU baseline (the repo's CPU port of the reference path, timed on the host cores on a bounded
sample of the same workload).
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0


def build_synthetic_on_device(hp, keep):
    """Random-init weights generated directly in HBM (pi_fill_normal_f16 / pi_fill_normal_q4_0), predictor fc2 rows
    carrying the Zipf firing-rate bias computed on the host (powerinfer_amd.synth).  With hp.hot_frac < 1 the FFN
    matrices are copied back to the host, which keeps the cold neurons, and the engine gathers the hot rows
    (gpu_bucket) into compact device matrices."""
    from powerinfer_amd import lib as pl, synth
    from powerinfer_amd.model import Model
    from scipy.special import ndtri
    L = pl.init()
    m = Model(hp)
    d, ff, r = hp.n_embd, hp.n_ff, hp.n_rank
    gqa = d // hp.n_head * hp.n_head_kv
    falcon = hp.arch == "falcon"
    q4 = hp.wtype == pl.Q4_0
    hybrid = hp.hot_frac < 1.0
    seed = [hp.seed * 1000003 + 17]

    def normal(rows, cols, bias=None, f16=False):
        seed[0] += 1
        if q4 and not f16:
            buf = pl.DevBuf(rows * cols // 32 * 18)
            pl.check(L.pi_fill_normal_q4_0(buf.ptr, rows * cols, seed[0], 0.02, None), "fill")
        else:
            buf = pl.DevBuf(rows * cols * 2)
            pl.check(L.pi_fill_normal_f16(buf.ptr, rows * cols, seed[0], 0.02, bias.ptr if bias is not None else None, cols, None), "fill")
        keep.append(buf)
        return buf

    def put(layer, kind, buf, rows, cols, f16=False):
        m.set_tensor_device(layer, kind, buf.ptr, pl.F16 if (f16 or not q4) else pl.Q4_0, cols, rows)

    def put_ffn(layer, kind, buf, rows, cols):
        if not hybrid:
            return put(layer, kind, buf, rows, cols)
        pl.sync()
        host = buf.download(np.uint8).reshape(rows, -1) if q4 else buf.download(np.float16).reshape(rows, cols)
        m.set_tensor(layer, kind, host)

    tok_embd, output = normal(hp.n_vocab, d), normal(hp.n_vocab, d)
    rng = np.random.default_rng(hp.seed)
    if hp.get("head_pair"):
        # the greedy decision with a margin of powerinfer_amd.synth.make_model: four dominant output rows +-w0, +-w1, and the
        # embeddings of those four tokens scaled down
        assert not q4
        pl.sync()
        rows = np.empty((4, d), np.float16)
        for k in range(2):
            w = rng.standard_normal(d, dtype=np.float32) * np.float32(0.02 * hp.head_pair)
            rows[2 * k], rows[2 * k + 1] = w.astype(np.float16), (-w).astype(np.float16)
        output.upload(rows)
        tok_embd.upload((tok_embd.download(np.float16, 4 * d).astype(np.float32) * np.float32(0.05)).astype(np.float16))
    put(-1, "tok_embd", tok_embd, hp.n_vocab, d)
    put(-1, "output", output, hp.n_vocab, d)
    m.set_tensor(-1, "output_norm", np.ones(d, np.float32))
    if falcon:
        m.set_tensor(-1, "output_norm_b", np.zeros(d, np.float32))
    for il in range(hp.n_layer):
        m.set_tensor(il, "attn_norm", np.ones(d, np.float32))
        if falcon:
            m.set_tensor(il, "attn_norm_b", np.zeros(d, np.float32))
            if hp.n_head_kv != hp.n_head:
                m.set_tensor(il, "attn_norm_2", np.ones(d, np.float32))
                m.set_tensor(il, "attn_norm_2_b", np.zeros(d, np.float32))
        else:
            m.set_tensor(il, "ffn_norm", np.ones(d, np.float32))
        put(il, "wqkv", normal(d + 2 * gqa, d), d + 2 * gqa, d)
        put(il, "wo", normal(d, d), d, d)
        if not falcon:
            put_ffn(il, "ffn_gate", normal(ff, d), ff, d)
        put_ffn(il, "ffn_up", normal(ff, d), ff, d)
        put_ffn(il, "ffn_down_t", normal(ff, d), ff, d)
        put(il, "fc1", normal(r, d, f16=True), r, d, f16=True)
        p, _ = synth.zipf_rates(ff, hp.mean_rate, rng)
        if hp.get("pred_margin"):                  # a predictor whose decisions keep a margin (synth.predictor_fc2_margin), made on the host
            fc2 = pl.DevBuf(host=synth.predictor_fc2_margin(ff, r, p, rng))
            keep.append(fc2)
        else:
            b = (0.02 * np.sqrt(np.pi) * ndtri(p) / np.sqrt(r)).astype(np.float32)
            bias = pl.DevBuf(host=b)
            fc2 = normal(ff, r, bias, f16=True)
        put(il, "fc2", fc2, ff, r, f16=True)
        m.set_tensor(il, "neuron_rate", p.astype(np.float32))      # the activation statistics the split planner works from
        if hybrid:
            gi, gb = synth.gpu_split(p, hp.hot_frac)
            m.set_tensor(il, "gpu_idx", gi)
            m.set_tensor(il, "gpu_bucket", gb)
    pl.sync()
    m.finalize()
    return m


def download_model(hp, keep):
    """Host copies of the device-generated tensors of the default workload (F16 LLaMA shape, all neurons on the GPU), in
    the dict layout powerinfer_amd.synth.make_model uses (feeds the CPU port for the cpu_baseline leg)."""
    d, ff, r = hp.n_embd, hp.n_ff, hp.n_rank
    gqa = d // hp.n_head * hp.n_head_kv
    it = iter(keep)
    grab = lambda rows, cols: next(it).download(np.float16).reshape(rows, cols)  # noqa: E731
    glob = dict(tok_embd=grab(hp.n_vocab, d), output=grab(hp.n_vocab, d), output_norm=np.ones(d, np.float32))
    layers = []
    for _ in range(hp.n_layer):
        Lr = dict(attn_norm=np.ones(d, np.float32), ffn_norm=np.ones(d, np.float32))
        wqkv = grab(d + 2 * gqa, d)
        Lr["wq"], Lr["wk"], Lr["wv"] = (np.ascontiguousarray(a) for a in (wqkv[:d], wqkv[d:d + gqa], wqkv[d + gqa:]))
        Lr["wo"], Lr["ffn_gate"], Lr["ffn_up"], Lr["ffn_down_t"] = grab(d, d), grab(ff, d), grab(ff, d), grab(ff, d)
        Lr["fc1"], Lr["fc2"] = grab(r, d), grab(ff, r)
        layers.append(Lr)
    return dict(hp=hp, glob=glob, layers=layers)


def rnd(v, n):
    return None if v != v else round(v, n)


def touched_bytes_per_token(hp, active_sum, n_kv_mean):
    """Algorithmic bytes of one decoded token:  sum_l [ W_attn + W_pred + A_l * n_mats * R + 2 * n_kv * n_embd_gqa * 2 ]
    + W_lmhead + d * 2, with the measured per-token sum of active rows (the GPU's share for a hybrid split)."""
    d, ff, r, Lr = hp.n_embd, hp.n_ff, hp.n_rank, hp.n_layer
    gqa = d // hp.n_head * hp.n_head_kv
    s = 2.0 if hp.wtype == 1 else 18.0 / 32.0
    n_mats = 2 if hp.arch == "falcon" else 3
    w_attn = (d * (d + 2 * gqa) + d * d) * s
    w_pred = (d * r + r * ff) * 2.0
    row = d * s
    return Lr * (w_attn + w_pred + 2 * n_kv_mean * gqa * 2.0) + active_sum * n_mats * row + hp.n_vocab * d * s + d * 2.0


def cpu_baseline(hp, keep, prompt, n_prompt, n_decode, threads, model=None):
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import oracle_lib as ol
    model = model or download_model(hp, keep)
    om = ol.OracleModel(model)
    n_past = 0
    tok = 0
    for t in prompt[:n_prompt]:
        tok, _ = om.eval([int(t)], n_past, nth=threads)
        n_past += 1
    t0 = time.perf_counter()
    for _ in range(n_decode):
        tok, _ = om.eval([tok], n_past, nth=threads)
        n_past += 1
    dt = time.perf_counter() - t0
    om.close()
    return n_decode / dt


def cpu_reference(model, prompt, n_prompt, n_decode, threads):
    """The reference's own CPU path on the same weights: the model is written as a PowerInfer GGUF into memory-backed storage and
    oracle/_ref/ref_llama - the reference's llama.cpp and ggml.c compiled without an accelerator (oracle/Makefile) - decodes
    n_prompt prompt tokens and n_decode greedy tokens with `threads` threads.  Returns tok/s over the decode tokens, or None when the
    binary or the space for the file is missing."""
    import shutil
    import subprocess
    import tempfile
    from powerinfer_amd import gguf
    exe = os.path.join(ROOT, "oracle", "_ref", "ref_llama")
    if not os.path.exists(exe):
        return None
    hp = model["hp"]
    need = sum(a.nbytes for a in model["glob"].values()) + sum(a.nbytes for L in model["layers"] for a in L.values() if a is not None)
    base = next((d for d in ("/dev/shm", tempfile.gettempdir()) if os.path.isdir(d) and shutil.disk_usage(d).free > need * 1.2 + (1 << 30)), None)
    if base is None:
        return None
    td = tempfile.mkdtemp(prefix="pi_cpu_ref_", dir=base)
    try:
        path, out = os.path.join(td, "m.powerinfer.gguf"), os.path.join(td, "out.bin")
        gguf.write_model(path, model, gguf.synthetic_tokenizer_kv(hp.n_vocab))
        toks = [str(int(t)) for t in prompt[:n_prompt]]
        r = subprocess.run([exe, path, str(n_prompt + n_decode + 8), str(threads), str(n_decode), out] + toks, capture_output=True, text=True, timeout=600)
        ms = [float(l.split()[1]) for l in r.stdout.splitlines() if l.startswith("decode_ms_per_token")]
        return 1e3 / ms[0] if r.returncode == 0 and ms and ms[0] > 0 else None
    finally:
        shutil.rmtree(td, ignore_errors=True)


def reference_host_on_this_backend(n_prompt=8, n_gen=48):
    """The drop-in path as a number: the reference's own llama.cpp (loader, ggml-alloc, graph builder, executor) compiled against this
    library in place of ggml-cuda.cu (oracle/_ref/ref_llama_gpu, test infrastructure) decodes 7B-wide synthetic models of 4 and of 8
    layers with every tensor on the GPU, one ggml_cuda_compute_forward call per graph node.  The difference between the two runs is
    what one more layer costs; the 4-layer figure also carries what the host does once per token (graph construction, the
    inputs' upload, the lm-head and the logits' way back)."""
    import subprocess
    import tempfile
    from powerinfer_amd import gguf, split, synth
    exe = os.path.join(ROOT, "oracle", "_ref", "ref_llama_gpu")
    if not os.path.exists(exe):
        return None
    ms_of, stats = {}, {}
    for n_layer in (4, 8):
        hp = synth.hparams("llama-7b", n_layer=n_layer, n_ctx=128, seed=3)
        model = synth.make_model(hp)
        with tempfile.TemporaryDirectory() as td:
            path, out = os.path.join(td, "m.powerinfer.gguf"), os.path.join(td, "out.bin")
            gguf.write_model(path, model, gguf.synthetic_tokenizer_kv(hp.n_vocab))
            splits = [(np.ones(hp.n_ff, np.int32), np.arange(hp.n_ff, dtype=np.int32)) for _ in range(hp.n_layer)]
            split.write_gpuidx(path + ".generated.gpuidx", splits, split.required_bytes(hp, splits))
            del model
            toks = [str(int(t)) for t in np.random.default_rng(5).integers(0, hp.n_vocab, n_prompt)]
            r = subprocess.run([exe, path, "128", "1", str(n_gen), out] + toks, env=dict(os.environ, REF_VRAM_GB="16"),
                               capture_output=True, text=True, timeout=240)
        if r.returncode != 0:
            return {"error": (r.stdout + r.stderr)[-300:]}
        ms = [float(l.split()[1]) for l in r.stdout.splitlines() if l.startswith("decode_ms_per_token")]
        if not ms:
            return {"error": "no timing line"}
        ms_of[n_layer] = ms[0]
        for l in r.stdout.splitlines():
            if l.startswith("backend_stats"):
                w = l.split()
                stats[n_layer] = {w[i]: int(w[i + 1]) for i in range(1, len(w), 2)}
    return {"ms_per_token": round(ms_of[4], 3), "n_layer": 4, "ms_per_token_per_layer": round(ms_of[4] / 4, 4),
            "ms_per_token_8_layers": round(ms_of[8], 3), "ms_per_additional_layer": round((ms_of[8] - ms_of[4]) / 4, 4),
            "backend_stats_8_layers": stats.get(8), "host_threads": 1,
            "what": "reference llama.cpp + ggml executor linked to libpowerinfer_hip.so (oracle/_ref/ref_llama_gpu), 7B-wide layers, "
                    "all tensors and the KV cache on the GPU, one backend call per graph node (single-token nodes wait in a window: an "
                    "attention block runs as three launches, an FFN block as three); ms_per_token includes the lm-head and the host's "
                    "per-token work once, ms_per_additional_layer is (8 layers - 4 layers) / 4"}


def bench_batched(args):
    """configs[3]: 13B shape, 16 sequences advancing one token per step; the whole-job rate counts every sequence's token."""
    from powerinfer_amd import lib as pl, synth
    n_seq = 16
    n_prompt = 512 if args.prompt == 64 else args.prompt
    steps = 128 if args.steps == 256 else args.steps
    over = {} if args.mean_rate is None else {"mean_rate": args.mean_rate}
    q4 = args.batch_model == "llama-7b-q4"
    if q4:      # the Q4_0 model of configs[2] with every neuron on the GPU, sixteen sequences in lockstep
        hp = synth.hparams("llama-7b", n_layer=args.layers, n_ctx=n_prompt + args.warmup + steps + 8, seed=1, wtype=pl.Q4_0, **over)
    else:
        hp = synth.hparams("llama-13b", n_layer=40 if args.layers == 32 else args.layers, n_ctx=n_prompt + args.warmup + steps + 8, seed=1, **over)
    keep = []
    m = build_synthetic_on_device(hp, keep)
    m.batch_init(n_seq)
    if args.dense_above is not None:
        m.batch_set_dense_above(args.dense_above)
    rng = np.random.default_rng(2024)
    prompt = rng.integers(0, hp.n_vocab, (n_prompt, n_seq)).astype(np.int32)
    for s in range(n_prompt):                                   # prompt phase (not timed): one position of every sequence per step
        m.batch_decode(prompt[s], np.full(n_seq, s, np.int32), want_logits=False)
    if args.warmup > 0:
        m.batch_generate(args.warmup)
    pl.sync()
    t0 = time.perf_counter()
    toks, ms_dev = m.batch_generate(steps)
    pl.sync()
    wall = time.perf_counter() - t0
    union = m.batch_union().astype(np.float64)
    d, ff, r = hp.n_embd, hp.n_ff, hp.n_rank
    n_kv = n_prompt + args.warmup + (steps + 1) / 2.0
    step_bytes = hp.n_layer * (4 * d * d * 2.0 + (d * r + r * ff) * 2.0 + n_seq * 2 * n_kv * d * 2.0) + union.sum() * 3 * d * 2.0 + hp.n_vocab * d * 2.0
    ms_step = wall * 1e3 / steps
    out = {
        "metric": "decode tok/s, 16 sequences, " + ("ReluLLaMA-7B shape Q4_0 (integer matrix-core kernels on Q4_0 x Q8_0 blocks)" if q4 else "ProSparse-Llama2-13B shape FP16"), "value": round(n_seq * 1e3 / ms_step, 1), "unit": "tok/s",
        "n_gpus": 1, "steps": steps, "warmup": args.warmup, "ms_per_step": round(ms_step, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "q4_0 x q8_0 (int8 MFMA, fp32 scale)" if q4 else "f16", "data": "synthetic",
        "config": {"workload": ("configs[2]'s model in lockstep: ReluLLaMA-7B shape (d 4096, ff 11008, 32 heads, vocab 32000, predictor rank 1024), " if q4 else
                                "configs[3]: ProSparse-LLaMA-2-13B shape (d 5120, ff 13824, 40 heads, vocab 32000, predictor rank 1280), ") +
                               f"{hp.n_layer} layers, random-init {'Q4_0' if q4 else 'FP16'} weights, all neurons on the GPU, {n_seq} sequences with {n_prompt}-token random "
                               "prompts, greedy decode in lockstep (one token per sequence per step)",
                   "n_layer": hp.n_layer, "n_seq": n_seq, "prompt_tokens": n_prompt, "n_ctx": hp.n_ctx,
                   "mean_union_rows_per_layer": round(union.mean(), 1), "union_fraction": round(union.mean() / hp.n_ff, 3),
                   "layers_run_dense": m.batch_dense_layers(), "device": pl.device_name()},
        "token_loop": {"device_ms_per_step": round(ms_dev / steps, 4), "touched_GB_per_step": round(step_bytes / 1e9, 3),
                       "effective_GBps": round(step_bytes / (ms_step * 1e-3) / 1e9, 1),
                       "hbm_frac_touched": round(step_bytes / (ms_step * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)},
    }
    m.close()
    print(json.dumps(out), flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--prompt", type=int, default=64)
    ap.add_argument("--layers", type=int, default=32, help="only for quick trials; the reported workload uses 32")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--prompt-bench", type=int, default=1024, help="length of the prompt timed for the prompt_phase entry (0 = skip)")
    ap.add_argument("--no-q4", action="store_true", help="config 1: skip the extra object with the Q4_0 split model (configs[2]) measured in a child process (about 25 s)")
    ap.add_argument("--no-ref-host", action="store_true", help="skip the leg that runs the reference's llama.cpp on this backend (about 40 s)")
    ap.add_argument("--cpu-tokens", type=int, default=320, help="decode tokens timed on the host for the cpu_baseline leg (about 10 s of CPU work)")
    ap.add_argument("--config", type=int, default=1, choices=[1, 2, 3, 4],
                    help="BASELINE configs index: 1 (default, the reported metric) 7B FP16 all on the GPU; 2 the same shape in "
                         "Q4_0 with the hottest 60 %% of neurons on the GPU and the rest on host threads; 3 ProSparse-LLaMA-2-13B shape FP16, "
                         "16 sequences decoded in lockstep; 4 Falcon-40B shape FP16")
    ap.add_argument("--n-seq", type=int, default=16, choices=[1, 16], help="config 3: 16 sequences in lockstep (configs[3]) or the same model at batch 1")
    ap.add_argument("--batch-model", default="llama-13b", choices=["llama-13b", "llama-7b-q4"], help="config 3 with 16 sequences: configs[3]'s model, or the Q4_0 7B model in lockstep")
    ap.add_argument("--mean-rate", type=float, default=None, help="config 3: mean firing rate of the synthetic predictors (default: the model's own, 0.11)")
    ap.add_argument("--dense-above", type=float, default=None, help="config 3: union fraction above which a layer's FFN runs dense (0 always, 1 never: the library's default)")
    ap.add_argument("--rest-on-gpu", action="store_true", help="config 2: the GPU reads the non-resident neurons' rows from pinned host memory itself instead of handing those neurons to host threads")
    ap.add_argument("--hot-frac", type=float, default=None, help="configs 1 and 2: share of each layer's neurons on the GPU (default 1.0 and 0.6)")
    ap.add_argument("--pmc-probe", action="store_true",
                    help="counter-collection aid: run only one section of a 4-layer model a few times plus one "
                         "device-to-device copy of the q|k|v matrix's byte count (the known-size reference for FETCH_SIZE / WRITE_SIZE)")
    ap.add_argument("--pmc-section", type=int, default=0, choices=[0, 1],
                    help="section replayed by --pmc-probe: 0 the q|k|v mat-vec, 1 the sparse FFN block (fc1, fused predictor + FFN, reduction)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs the token loop on ONE GPU; --gpus must be 1 "
                 "(more GPUs would split the FFN by neuron and attention by head, one [n_embd] exchange per layer)")

    from powerinfer_amd import lib as pl, synth
    if args.pmc_probe:
        hp = synth.hparams("llama-7b", n_layer=4, n_ctx=64, seed=1)
        keep = []
        m = build_synthetic_on_device(hp, keep)
        m.decode(np.array([1, 2], np.int32), 0, want_logits=False)
        d = hp.n_embd
        nbytes = 3 * d * d * 2
        src, dst = pl.DevBuf(nbytes), pl.DevBuf(nbytes)
        pl.check(pl.load().pi_memset(src.ptr, 1, nbytes), "memset")
        pl.sync()
        pl.check(pl.load().pi_memcpy_d2d(dst.ptr, src.ptr, nbytes), "copy")     # reads nbytes, writes nbytes
        pl.sync()
        ms, n = m.time_section(args.pmc_section, 4)
        act = [int(v) for v in m.get_capture()[2]] if args.pmc_section == 1 else None      # active rows per layer of the replayed block
        print(json.dumps({"pmc_probe": True, "section": args.pmc_section, "copy_bytes": nbytes, "launches": n, "us_per_launch": ms * 1e3,
                          "active_per_layer": act}))
        m.close()
        return
    n_ctx = args.prompt + args.warmup + args.steps + 8
    if args.config == 1:
        hp = synth.hparams("llama-7b", n_layer=args.layers, n_ctx=n_ctx, seed=1, hot_frac=1.0 if args.hot_frac is None else args.hot_frac)
    elif args.config == 2:
        hp = synth.hparams("llama-7b", n_layer=args.layers, n_ctx=n_ctx, seed=1, wtype=pl.Q4_0, hot_frac=0.6 if args.hot_frac is None else args.hot_frac,
                           rest_on_gpu=bool(args.rest_on_gpu))
    elif args.config == 3:
        hp = None if args.n_seq != 1 else synth.hparams("llama-13b", n_layer=40 if args.layers == 32 else args.layers, n_ctx=n_ctx, seed=1)
    else:
        hp = synth.hparams("falcon-40b", n_layer=60 if args.layers == 32 else args.layers, n_ctx=n_ctx, seed=1)
    if args.config == 3 and args.n_seq != 1:
        return bench_batched(args)
    hybrid = hp.hot_frac < 1.0
    keep = []
    t0 = time.perf_counter()
    m = build_synthetic_on_device(hp, keep)
    t_build = time.perf_counter() - t0

    rng = np.random.default_rng(2024)
    prompt = rng.integers(0, hp.n_vocab, args.prompt).astype(np.int32)
    m.decode(prompt, 0, want_logits=False)                    # prompt phase (not timed)
    if args.warmup > 0:
        m.generate(args.warmup)                               # warm-up steps (captures the HIP graph)
    pl.sync()
    t0 = time.perf_counter()
    toks, ms_dev = m.generate(args.steps)                     # timed: exactly K decode steps, device events inside
    pl.sync()
    wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / args.steps
    act = m.step_active(args.steps).astype(np.float64)
    n_kv_mean = args.prompt + args.warmup + (args.steps + 1) / 2.0
    tok_bytes = touched_bytes_per_token(hp, act.mean(), n_kv_mean)

    # roofline of the dominant kernel: the q|k|v projection mat-vec (gemv_f16_kernel<4>), one launch per layer
    d = hp.n_embd
    gqa = d // hp.n_head * hp.n_head_kv
    wbytes = 2.0 if hp.wtype == pl.F16 else 18.0 / 32.0
    qkv_bytes = (d + 2 * gqa) * d * wbytes + d * 4 + (d + 2 * gqa) * 4       # weights + activation in + result out
    if hybrid:                                                               # the section timers replay full-GPU layers only
        ms_qkv, n_qkv, ms_ffn, ms_head = float("nan"), 0, float("nan"), float("nan")
        ms_pf, n_pf, ms_fr = float("nan"), 0, float("nan")
    else:
        ms_qkv, n_qkv = m.time_section(0, 8)
        ms_ffn, _ = m.time_section(1, 8)
        ms_head, _ = m.time_section(2, 8)
        try:
            ms_pf, n_pf = m.time_section(3, 8)            # the fused predictor + FFN kernel alone, and the reduction behind it
            ms_fr, _ = m.time_section(4, 8)
        except Exception:
            ms_pf, n_pf, ms_fr = float("nan"), 0, float("nan")
    achieved = qkv_bytes / (ms_qkv * 1e-3) / 1e9
    n_mats = 2 if hp.arch == "falcon" else 3
    ffn_bytes = (d * hp.n_rank + hp.n_rank * hp.n_ff) * 2.0 + (act.mean() / hp.n_layer) * n_mats * d * wbytes

    # the fused sparse-FFN launch: ALGORITHMIC bytes only - the fc2 rows of every neuron and the gate / up / down rows of the active
    # ones (fc2 + A * n_mats * R); the partial output vectors it writes for the reduction are overhead, not work
    a_layer = act.mean() / hp.n_layer
    pf_bytes = hp.n_rank * hp.n_ff * 2.0 + a_layer * n_mats * d * 2.0

    def profiled_traffic(name, shape):
        """HBM bytes per launch from the FETCH_SIZE / WRITE_SIZE counter runs kept under profiles/ (a separate rocprofv3 --pmc run of
        `bench.py --pmc-probe`, not measured by this run); None when no profile of this shape is there."""
        try:
            with open(os.path.join(ROOT, "profiles", name + ".json")) as f:
                pj = json.load(f)
            if pj.get("shape") == shape and args.config == 1:
                return pj["traffic_bytes_per_launch"], "profiles/" + name + ".md (rocprofv3 --pmc FETCH_SIZE, WRITE_SIZE; a constant from that run, not measured here)"
        except (OSError, ValueError, KeyError):
            pass
        return None, None

    pf_traffic, pf_src = profiled_traffic("sparse_ffn_hbm_traffic", [hp.n_ff, d, hp.n_rank])
    traffic, qkv_src = profiled_traffic("qkv_gemv_hbm_traffic", [d + 2 * gqa, d])
    n_cu_form = d == 4096 and pl.load().pi_k_sparse_ffn_workgroups(hp.n_ff, hp.n_rank, d) != hp.n_ff // 32
    roof_qkv = {
        "bound": "hbm",
        "kernel": {1: "gemv_f16_reg_kernel<8,1,0> (q|k|v projection, 12288 x 4096 fp16, fused RMSNorm)",
                   2: "gemv_q4_kernel (q|k|v projection, 12288 x 4096 Q4_0, fused RMSNorm; not timed for a hybrid model)",
                   3: "gemv_f16_reg_kernel<10,1,0> (q|k|v projection, 15360 x 5120 fp16, fused RMSNorm)",
                   4: "gemv_f16_reg_kernel<16,2,0> (q|k|v projection, 9216 x 8192 fp16, fused LayerNorm)"}[args.config],
        "achieved": rnd(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": rnd(achieved / HBM_PEAK_GBPS, 4),
        "traffic": traffic, "traffic_source": qkv_src,
        "bytes_per_launch": qkv_bytes, "bytes_are": "weights + input vector + result (algorithmic)",
        "us_per_launch": rnd(ms_qkv * 1e3, 2), "launches_timed": n_qkv,
    }
    roof_ffn = {
        "bound": "hbm",
        "kernel": {1: ("ffn_cu_f16_kernel<8,1024,true,6,1>" if n_cu_form else "pred_ffn_f16_kernel<1,2,true,1,false>") +
                      " (predictor fc2 11008 x 1024 + mask + gate/up/down rows of the active neurons, 7B layer)",
                   2: "pred_upgate_q4_kernel (not timed for a hybrid model)",
                   3: "ffn_cu_f16_kernel<10,1280,true,6,1> (predictor fc2 13824 x 1280 + mask + gate/up/down rows of the active neurons, 13B layer)",
                   4: "pred_ffn_f16_kernel<2,2,false,4,false> (predictor fc2 32768 x 1024 + mask + up/down rows of the active neurons, Falcon-40B layer)"}[args.config],
        "achieved": rnd(pf_bytes / (ms_pf * 1e-3) / 1e9, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
        "frac": rnd(pf_bytes / (ms_pf * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
        "traffic": pf_traffic, "traffic_source": pf_src,
        "bytes_per_launch": round(pf_bytes),
        "bytes_are": "fc2 rows of every neuron + gate/up/down rows of the measured mean of active neurons (algorithmic; the partial vectors written for the reduction are excluded)",
        "us_per_launch": rnd(ms_pf * 1e3, 2), "reduce_us_per_launch": rnd(ms_fr * 1e3, 2), "launches_timed": n_pf,
    }
    # `roofline` names the kernel that takes the most time per token (one launch per layer each): whichever of the two is slower in this run
    ffn_dominates = ms_pf == ms_pf and ms_pf >= ms_qkv

    out = {
        "metric": {1: "decode tok/s bs=1 ReLU-Llama2-7B FP16", 2: "decode tok/s bs=1 ReLU-Llama2-7B Q4_0 (60 % of neurons on the GPU)",
                   3: "decode tok/s bs=1 ProSparse-Llama2-13B shape FP16", 4: "decode tok/s bs=1 ReLU-Falcon-40B FP16"}[args.config],
        "value": round(1e3 / ms_per_step, 2),
        "unit": "tok/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16" if hp.wtype == pl.F16 else "q4_0 x q8_0 (int8 dot, fp32 scale)",
        "data": "synthetic",
        "config": {
            "workload": {
                1: "configs[1]: ReLU-LLaMA-2-7B shape (d 4096, ff 11008, 32 heads, vocab 32000, predictor rank 1024), "
                   f"{hp.n_layer} layers, random-init FP16 weights, all neurons on the GPU, {args.prompt}-token random prompt, "
                   "greedy decode at batch 1",
                2: "configs[2]: ReLU-LLaMA-2-7B shape, random-init weights quantised to Q4_0 (predictors FP16), per layer the hottest "
                   f"60 % of neurons on the GPU and the rest " + ("in pinned host memory, their active rows read by the GPU itself" if hp.get("rest_on_gpu") else "on host threads")
                   + f", {hp.n_layer} layers, {args.prompt}-token random prompt, greedy decode at batch 1",
                3: "configs[3]'s model at batch 1: ProSparse-LLaMA-2-13B shape (d 5120, ff 13824, 40 heads, vocab 32000, predictor rank 1280), "
                   f"{hp.n_layer} layers, random-init FP16 weights, all neurons on the GPU, {args.prompt}-token random prompt, greedy decode at batch 1",
                4: "configs[4]: ReLU-Falcon-40B shape (d 8192, ff 32768 up/down only, 128 heads / 8 KV heads, vocab 65024, predictor "
                   f"rank 1024), {hp.n_layer} layers, random-init FP16 weights, all neurons on the GPU, {args.prompt}-token random "
                   "prompt, greedy decode at batch 1"}[args.config],
            "n_layer": hp.n_layer, "prompt_tokens": args.prompt, "n_ctx": hp.n_ctx,
            "mean_active_per_layer": round(act.mean() / hp.n_layer, 1),
            "device": pl.device_name(),
        },
        "roofline": dict(roof_ffn if ffn_dominates else roof_qkv),
        "roofline_qkv": roof_qkv,
        "roofline_sparse_ffn": roof_ffn,
        "token_loop": {
            "device_ms_per_step": round(ms_dev / args.steps, 4),
            "touched_GB_per_token": round(tok_bytes / 1e9, 4),
            "effective_GBps": round(tok_bytes / (ms_per_step * 1e-3) / 1e9, 1),
            "hbm_frac_touched": round(tok_bytes / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
            "sparse_ffn_us_per_layer": rnd(ms_ffn * 1e3, 2),
            "sparse_ffn_effective_GBps": rnd(ffn_bytes / (ms_ffn * 1e-3) / 1e9, 1),
            "lm_head_us": rnd(ms_head * 1e3, 2),
            "build_s": round(t_build, 1),
        },
    }
    if not args.no_cpu and args.config == 1:
        threads = min(16, os.cpu_count() or 1)
        n_prompt = 8
        cpu_tokens = max(1, min(args.cpu_tokens, hp.n_ctx - n_prompt))
        host_model = download_model(hp, keep)
        v = cpu_baseline(hp, keep, prompt, n_prompt, cpu_tokens, threads, model=host_model)
        port = {"value": round(v, 3), "unit": "tok/s", "cores": threads, "kind": "port",
                "sample": f"same {hp.n_layer}-layer model and weights (copied back from HBM), {n_prompt}-token prompt then "
                          f"{cpu_tokens} greedy decode tokens timed, oracle/pi_oracle.c with OpenMP (on the build container this port runs "
                          f"the 7B sparse FFN block alone in 0.67x (1 thread) / 0.36x (8 threads) the time of the reference's own ggml.c, "
                          f"oracle/calibrate_cpu.py; the reference's whole token loop is timed beside it when its binary is present)"}
        ref_tokens = 48
        try:
            vr = cpu_reference(host_model, prompt, n_prompt, ref_tokens, threads)
        except Exception:               # a missing binary or a full disk leaves the port's figure
            vr = None
        if vr is not None:
            out["cpu_baseline"] = {"value": round(vr, 3), "unit": "tok/s", "cores": threads, "kind": "reference",
                                   "sample": f"same {hp.n_layer}-layer model and weights (copied back from HBM and written as a PowerInfer GGUF into "
                                             f"memory-backed storage), {n_prompt}-token prompt then {ref_tokens} greedy decode tokens timed, the reference's "
                                             f"own llama.cpp + ggml.c CPU path (oracle/_ref/ref_llama, -ngl 0) with {threads} threads",
                                   "port": port}
        else:
            out["cpu_baseline"] = port
        del host_model
    m.close()
    del keep
    if args.config == 2 and hybrid and not hp.get("rest_on_gpu"):
        # the same split with the non-resident rows in pinned host memory and the GPU reading the active ones itself: no host
        # threads in the loop, one graph replay per token; same model, prompt and steps, tokens compared with the run above
        try:
            hp2 = synth.HParams(hp)
            hp2["rest_on_gpu"] = True
            keep2 = []
            m2 = build_synthetic_on_device(hp2, keep2)
            m2.decode(prompt, 0, want_logits=False)
            if args.warmup > 0:
                m2.generate(args.warmup)
            pl.sync()
            t0 = time.perf_counter()
            toks2, _ = m2.generate(args.steps)
            pl.sync()
            dt = time.perf_counter() - t0
            out["rest_read_by_gpu"] = {"value": round(args.steps / dt, 2), "unit": "tok/s", "ms_per_step": round(dt * 1e3 / args.steps, 4),
                                       "tokens_identical_to_host_threads": bool(np.array_equal(np.asarray(toks), np.asarray(toks2))),
                                       "what": "same 60 % split: the non-resident 40 % of each layer's rows stay in pinned host memory, the kernels that "
                                               "compute the resident neurons also read the rows of active non-resident neurons over the host link "
                                               "(pi_model_set_rest_on_gpu), one HIP graph replay per token"}
            m2.close()
            del keep2
        except Exception as e:
            out["rest_read_by_gpu"] = {"error": repr(e)[:200]}
    if args.prompt_bench > 0:
        # prompt phase on its own: a fresh instance of the same model with room for the prompt, one untimed pass (allocations, the
        # transposed down projections, the library's mat-mul plans), then the timed pass from an empty cache; chunks of up to 512 tokens
        # per weight pass
        try:
            hp2 = synth.hparams({1: "llama-7b", 2: "llama-7b", 4: "falcon-40b"}[args.config], n_layer=hp.n_layer, n_ctx=args.prompt_bench + 8, seed=1,
                                wtype=hp.wtype, hot_frac=hp.hot_frac)
            keep2 = []
            m2 = build_synthetic_on_device(hp2, keep2)
            ptoks = rng.integers(0, hp2.n_vocab, args.prompt_bench).astype(np.int32)
            m2.decode(ptoks, 0, want_logits=False)
            m2.kv_clear()
            pl.sync()
            t0 = time.perf_counter()
            m2.decode(ptoks, 0, want_logits=False)
            pl.sync()
            dt = time.perf_counter() - t0
            out["prompt_phase"] = {"tokens": args.prompt_bench, "ms": round(dt * 1e3, 2), "tok_per_s": round(args.prompt_bench / dt, 1),
                                   "gemm": "own LDS-tiled MFMA kernel" if os.environ.get("PI_PREFILL_GEMM") == "own" else "hipBLASLt plans",
                                   "what": "pi_model_decode of the whole prompt: chunks of up to 512 tokens (dense mat-muls through hipBLASLt plans, or on this library's own kernel with PI_PREFILL_GEMM=own; each weight "
                                           "row read once per chunk, predictor mask applied to h), last token through the single-token path"
                                           + ("; Q4_0 matrices expanded to fp16 per chunk, activations through Q8_0 blocks" if hp.wtype != pl.F16 else "")
                                           + ("; non-resident FFN rows read from pinned host memory once per chunk" if hybrid else "")}
            m2.close()
            del keep2
        except Exception as e:
            out["prompt_phase"] = {"error": repr(e)[:200]}
    if args.config == 1 and not hybrid and not args.no_q4:
        # the Q4_0 half of the metric (configs[2]: hottest 60 % of neurons on the GPU, the rest on host threads) as an extra object:
        # the same script in a child process, so that this process's line stays the FP16 one
        try:
            import subprocess
            r = subprocess.run([sys.executable, os.path.abspath(__file__), "--config", "2", "--no-cpu", "--no-ref-host", "--steps", str(args.steps),
                                "--warmup", str(args.warmup), "--prompt", str(args.prompt), "--layers", str(args.layers), "--prompt-bench", str(args.prompt_bench)],
                               capture_output=True, text=True, timeout=600)
            q = json.loads(r.stdout.strip().splitlines()[-1])
            out["q4_0_split"] = {"value": q["value"], "unit": q["unit"], "ms_per_step": q["ms_per_step"], "workload": q["config"]["workload"],
                                 "mean_active_per_layer": q["config"]["mean_active_per_layer"], "hbm_frac_touched": q["token_loop"]["hbm_frac_touched"],
                                 "rest_read_by_gpu": {k: q["rest_read_by_gpu"].get(k) for k in ("value", "unit", "ms_per_step")} if "rest_read_by_gpu" in q else None,
                                 "prompt_phase": {k: q["prompt_phase"].get(k) for k in ("tokens", "ms", "tok_per_s")} if "prompt_phase" in q else None}
        except Exception as e:          # a reporting extra: never costs the bench line
            out["q4_0_split"] = {"error": repr(e)[:200]}
    if not args.no_ref_host and args.config == 1:
        try:
            rh = reference_host_on_this_backend()
        except Exception as e:          # a reporting extra: never costs the bench line
            rh = {"error": repr(e)[:200]}
        if rh is not None:
            out["reference_host_on_this_backend"] = rh
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
