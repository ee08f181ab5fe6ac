"""Model-level golden vectors from the REFERENCE's own llama.cpp CPU path (oracle/_ref/ref_llama = llama.cpp + ggml
compiled from /root/reference by oracle/Makefile): a synthetic PowerInfer GGUF ("PWRI" magic, tokenizer entries taken
from the reference's models/ggml-vocab-*.gguf data files) is written to a temporary directory, evaluated token by
token with one thread, and the greedy tokens plus a fixed sample of the logits of every step are stored.
The model itself is regenerated from its seed by powerinfer_amd.synth (a hash of the tensors guards the stream).

    python tests/golden/make_llama_fixture.py
"""
import hashlib
import os
import subprocess
import sys
import tempfile

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
from powerinfer_amd import gguf, synth  # noqa: E402

REF = "/root/reference"
BIN = os.path.join(ROOT, "oracle", "_ref", "ref_llama")

CASES = {
    "llama_f16": dict(base="llama-tiny", vocab="ggml-vocab-llama.gguf", over=dict(n_embd=256, n_ff=1024, n_rank=64, n_head=4, n_head_kv=4, n_layer=2, n_vocab=32000, n_ctx=64, seed=21)),
    "llama_q4": dict(base="llama-tiny", vocab="ggml-vocab-llama.gguf", over=dict(n_embd=256, n_ff=1024, n_rank=64, n_head=4, n_head_kv=4, n_layer=2, n_vocab=32000, n_ctx=64, seed=22, wtype=synth.Q4_0)),
    # the same models with a context shift before step 12 (llama_kv_cache_seq_rm + llama_kv_cache_seq_shift: K-shift, ring slots)
    "llama_f16_shift": dict(base="llama-tiny", vocab="ggml-vocab-llama.gguf", shift=(12, 2, 4), n_gen=14, over=dict(n_embd=256, n_ff=1024, n_rank=64, n_head=4, n_head_kv=4, n_layer=2, n_vocab=32000, n_ctx=64, seed=21)),
    "falcon_f16_shift": dict(base="falcon-tiny", vocab="ggml-vocab-falcon.gguf", shift=(12, 2, 4), n_gen=14, over=dict(n_embd=256, n_ff=1024, n_rank=64, n_head=8, n_head_kv=2, n_layer=2, n_vocab=65024, n_ctx=64, seed=23)),
    # linear RoPE scaling (the file's rope.scaling.factor = 2, so rope_freq_scale = 0.5) through prompt, decode and a context shift:
    # rope_yarn with ext_factor 0 (ggml.c:11124-11146), NeoX mode's second product (ggml.c:11292, 11447), the scaled K-shift
    "llama_f16_scaled_shift": dict(base="llama-tiny", vocab="ggml-vocab-llama.gguf", shift=(12, 2, 4), n_gen=14, over=dict(n_embd=256, n_ff=1024, n_rank=64, n_head=4, n_head_kv=4, n_layer=2, n_vocab=32000, n_ctx=64, seed=24, rope_freq_scale=0.5)),
    "falcon_f16_scaled_shift": dict(base="falcon-tiny", vocab="ggml-vocab-falcon.gguf", shift=(12, 2, 4), n_gen=14, over=dict(n_embd=256, n_ff=1024, n_rank=64, n_head=8, n_head_kv=2, n_layer=2, n_vocab=65024, n_ctx=64, seed=25, rope_freq_scale=0.5)),
    "falcon_f16": dict(base="falcon-tiny", vocab="ggml-vocab-falcon.gguf", over=dict(n_embd=256, n_ff=1024, n_rank=64, n_head=8, n_head_kv=2, n_layer=2, n_vocab=65024, n_ctx=64, seed=23)),
}


def model_sha(model):
    h = hashlib.sha256()
    for a in model["glob"].values():
        h.update(np.ascontiguousarray(a).tobytes())
    for L in model["layers"]:
        for k in sorted(L):
            if L[k] is not None and k != "p":
                h.update(np.ascontiguousarray(L[k]).tobytes())
    return np.frombuffer(h.digest(), np.uint8)


def case_model(name):
    c = CASES[name]
    hp = synth.hparams(c["base"], **c["over"])
    return hp, synth.make_model(hp)


def seq_edit_case():
    """Three sequences in lockstep, then llama_kv_cache_seq_rm / _seq_shift / _seq_cp on them (the history of
    tests/test_gpu_batch.py::test_batch_kv_sequence_edits), driven through the reference's own KV-cell bookkeeping."""
    hp = synth.hparams("llama-tiny", seed=9, n_ctx=48, sparse_threshold=-1e30)
    n_seq, n0 = 3, 8
    toks = np.random.default_rng(21).integers(0, hp.n_vocab, (n0 + 1, n_seq)).astype(np.int32)
    lines = []
    for s in range(n0):
        lines.append("decode %d " % n_seq + " ".join("%d %d %d" % (toks[s, q], s, q) for q in range(n_seq)))
    lines += ["rm 0 2 5", "shift 0 5 8 -3", "rm 2 0 -1", "cp 1 2 0 6"]
    last_pos = (5, 8, 6)
    lines.append("decode %d " % n_seq + " ".join("%d %d %d" % (toks[n0, q], last_pos[q], q) for q in range(n_seq)))
    return hp, toks, last_pos, lines


def make_seq_edit_fixture():
    hp, toks, last_pos, lines = seq_edit_case()
    model = synth.make_model(hp)
    with tempfile.TemporaryDirectory() as td:
        path, out, script = os.path.join(td, "m.powerinfer.gguf"), os.path.join(td, "out.bin"), os.path.join(td, "script.txt")
        gguf.write_model(path, model, gguf.synthetic_tokenizer_kv(hp.n_vocab))
        with open(script, "w") as f:
            f.write("\n".join(lines) + "\n")
        subprocess.check_call([BIN, path, str(hp.n_ctx), "1", "0", out, "0"], stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL,
                              env=dict(os.environ, REF_SCRIPT=script))
        raw = np.fromfile(out, np.uint8)
    n_rows, n_vocab = (int(v) for v in raw[:8].view(np.int32))
    logits = raw[8:].view(np.float32).reshape(n_rows, n_vocab)
    assert n_rows == 3 * 9
    np.savez_compressed(os.path.join(HERE, "ref_llama_seq_edits.npz"), tokens=toks, last_pos=np.asarray(last_pos, np.int32),
                        logits_last=logits[-3:], logits_step0=logits[:3], model_sha=model_sha(model))
    print("seq edits: greedy of the last step", logits[-3:].argmax(1).tolist())


def main(only=()):
    if not only:
        make_seq_edit_fixture()
    for name, c in CASES.items():
        if only and name not in only:
            continue
        hp, model = case_model(name)
        _, vkv, _ = gguf.read_gguf(os.path.join(REF, "models", c["vocab"]))
        tok_kv = {k: v for k, v in vkv.items() if k.startswith("tokenizer.")}
        assert len(tok_kv["tokenizer.ggml.tokens"][1][1]) == hp.n_vocab
        prompt = np.random.default_rng(hp.seed).integers(0, hp.n_vocab, 6)
        n_gen = c.get("n_gen", 10)
        env = dict(os.environ)
        shift = c.get("shift")
        if shift:
            env.update(REF_SHIFT_AT=str(shift[0]), REF_N_KEEP=str(shift[1]), REF_N_DISCARD=str(shift[2]))
        with tempfile.TemporaryDirectory() as td:
            path, out = os.path.join(td, "m.powerinfer.gguf"), os.path.join(td, "out.bin")
            gguf.write_model(path, model, tok_kv)
            subprocess.check_call([BIN, path, str(hp.n_ctx), "1", str(n_gen), out] + [str(int(t)) for t in prompt],
                                  stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL, env=env)
            raw = np.fromfile(out, np.uint8)
        n_steps, n_vocab = raw[:8].view(np.int32)
        rec = raw[8:].reshape(n_steps, 8 + 4 * n_vocab)
        consumed = rec[:, :4].copy().view(np.int32)[:, 0]
        greedy = rec[:, 4:8].copy().view(np.int32)[:, 0]
        logits = rec[:, 8:].copy().view(np.float32)
        sample = np.sort(np.random.default_rng(1).choice(n_vocab, 1024, replace=False)).astype(np.int32)
        np.savez_compressed(os.path.join(HERE, f"ref_{name}.npz"), prompt=prompt.astype(np.int32), consumed=consumed, greedy=greedy,
                            sample_idx=sample, logits_sample=logits[:, sample], logits_max=logits.max(1), logits_absmax=np.abs(logits).max(1),
                            model_sha=model_sha(model), shift=np.asarray(shift if shift else (-1, 0, 0), np.int32))
        print(name, "greedy", greedy.tolist())


if __name__ == "__main__":
    main(sys.argv[1:])                                   # case names to write; none = every fixture
