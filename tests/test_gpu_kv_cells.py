"""One KV cache with cells shared between sequences (pi_model_kv_cells_*): the cells' bookkeeping against the restatement of
llama_kv_cache (oracle_lib.KVCells), and the logits of sequences that share cells against the CPU oracle evaluating every
sequence on its own."""
import numpy as np
import pytest

import oracle_lib as ol
from powerinfer_amd import synth

pytestmark = pytest.mark.gpu


def rel_err(a, b):
    return float(np.abs(np.asarray(a, np.float64) - np.asarray(b, np.float64)).max() / max(np.abs(np.asarray(b, np.float64)).max(), 1e-30))


def test_cells_follow_the_reference_bookkeeping():
    """A random walk of steps (one to six tokens, one or several sequences per token), removals, copies, keeps and position shifts on a
    64-cell cache:
    after every operation the cells' positions, sequence sets and the ring's head equal the restatement's, and a step finds no slot
    exactly when the restatement finds none."""
    from powerinfer_amd import lib as pl
    from powerinfer_amd.model import Model
    hp = synth.hparams("llama-tiny", seed=3, n_ctx=64)
    gm = Model(hp).load(synth.make_model(hp))
    gm.kv_cells_init(64)
    ref = ol.KVCells(64)
    rng = np.random.default_rng(7)
    next_pos = [0] * 6
    n_fail = 0
    for it in range(140):
        op = rng.choice(["step", "step", "step", "rm", "cp", "keep", "shift"], p=[0.3, 0.3, 0.15, 0.1, 0.07, 0.03, 0.05])
        if op == "step":
            n = int(rng.integers(1, 7))
            seqs, pos = [], []
            for _ in range(n):
                s = int(rng.integers(0, 6))
                ids = [s] if rng.random() < 0.8 else sorted({s, int(rng.integers(0, 6))})
                seqs.append(ids)
                pos.append(next_pos[ids[0]])
                for v in ids:
                    next_pos[v] = max(next_pos[v], pos[-1] + 1)
            want = ref.decode(pos, seqs)
            toks = rng.integers(0, hp.n_vocab, n)
            if want is None:
                n_fail += 1
                with pytest.raises(pl.PiError):
                    gm.kv_cells_decode(toks, pos, seqs, want_logits=False)
            else:
                gm.kv_cells_decode(toks, pos, seqs, want_logits=False)
        elif op == "rm":
            s, p0 = int(rng.integers(-1, 6)), int(rng.integers(-1, 6))
            p1 = -1 if rng.random() < 0.5 else p0 + int(rng.integers(1, 8))
            ref.seq_rm(s, p0, p1)
            gm.kv_cells_seq_rm(s, p0, p1)
        elif op == "cp":
            a, b = (int(v) for v in rng.choice(6, 2, replace=False))
            ref.seq_cp(a, b, 0, -1)
            gm.kv_cells_seq_cp(a, b, 0, -1)
        elif op == "shift":
            s, p0, dl = int(rng.integers(0, 6)), int(rng.integers(0, 6)), int(rng.integers(-4, 3))
            ref.seq_shift(s, p0, -1, dl)
            gm.kv_cells_seq_shift(s, p0, -1, dl)
            next_pos[s] = max(0, next_pos[s] + dl)
        else:
            s = int(rng.integers(0, 6))
            ref.seq_keep(s)
            gm.kv_cells_seq_keep(s)
        gp, gs, gh = gm.kv_cells_state()
        rp, rs, rh = ref.state()
        assert np.array_equal(gp, rp) and np.array_equal(gs, rs) and gh == rh, (it, op)
    assert n_fail > 0                                            # the walk reached a cache without a free run
    gm.kv_cells_clear()
    assert np.all(gm.kv_cells_state()[0] == -1)
    gm.close()


@pytest.mark.parametrize("wtype", [synth.F16, synth.Q4_0], ids=["f16", "q4_0"])
@pytest.mark.parametrize("arch", ["llama-tiny", "falcon-tiny"])
def test_a_prompt_evaluated_once_serves_every_continuation(arch, wtype):
    """examples/batched/batched.cpp: the prompt is evaluated once for sequence 0, llama_kv_cache_seq_cp makes its cells visible to the
    other sequences (nothing is copied), and the continuations advance in lockstep, each attending the shared prompt cells and its own.
    Every continuation's logits against the CPU oracle evaluating prompt + continuation as a sequence of its own (median 1e-2, nine
    greedy tokens in ten equal); then one sequence is removed, its cells are found again by a new sequence (the ring), and the
    others are undisturbed."""
    from powerinfer_amd.model import Model
    q4 = wtype != synth.F16
    hp = synth.hparams(arch, seed=5, n_ctx=64, wtype=wtype, **(dict(pred_margin=True, head_pair=2048) if q4 else {}))
    model = synth.make_model(hp)
    rng = np.random.default_rng(21)
    n_prompt, n_seq, n_steps = 6, 3, 5
    prompt = rng.integers(0, hp.n_vocab, n_prompt)
    cont = rng.integers(0, hp.n_vocab, (n_steps, n_seq))
    gm = Model(hp).load(model)
    gm.kv_cells_init(32)
    _, lg = gm.kv_cells_decode(prompt, np.arange(n_prompt), [0] * n_prompt)
    oms = [ol.OracleModel(model) for _ in range(n_seq)]
    errs, same = [], 0
    for s in range(n_seq):
        tok_o, lg_o = oms[s].eval([int(t) for t in prompt], 0)
        if s == 0:
            errs.append(rel_err(lg[-1], lg_o))
    for s in range(1, n_seq):
        gm.kv_cells_seq_cp(0, s, 0, -1)
    pos, seq, head = gm.kv_cells_state()
    assert np.all(seq[:n_prompt] == 0b111) and np.all(pos[n_prompt:] == -1) and head == 0
    for i in range(n_steps):
        nxt, lg = gm.kv_cells_decode(cont[i], np.full(n_seq, n_prompt + i), list(range(n_seq)))
        for s in range(n_seq):
            tok_o, lg_o = oms[s].eval([int(cont[i, s])], n_prompt + i)
            errs.append(rel_err(lg[s], lg_o))
            same += int(nxt[s] == tok_o)
    assert np.median(errs) < 1e-2 and max(errs) < (1e-1 if q4 else 5e-2), errs
    assert same >= 0.9 * n_seq * n_steps, same
    # sequence 1 leaves: its own cells are freed, the shared prompt stays; sequence 3 starts from the prompt in the freed cells
    gm.kv_cells_seq_rm(1, -1, -1)
    pos, seq, head = gm.kv_cells_state()
    assert np.all(seq[:n_prompt] == 0b101) and head == n_prompt + 1          # the first cell sequence 1 owned alone
    gm.kv_cells_seq_cp(0, 3, 0, n_prompt)
    om3 = ol.OracleModel(model)
    om3.eval([int(t) for t in prompt], 0)
    toks = rng.integers(0, hp.n_vocab, 3)
    for i in range(3):
        steps = [(int(toks[i]), n_prompt + i, 3), (int(cont[0, 0]), n_prompt + n_steps + i, 0)]
        nxt, lg = gm.kv_cells_decode([t for t, _, _ in steps], [p for _, p, _ in steps], [q for _, _, q in steps])
        tok_o, lg_o = om3.eval([int(toks[i])], n_prompt + i)
        tok_0, lg_0 = oms[0].eval([int(cont[0, 0])], n_prompt + n_steps + i)
        assert rel_err(lg[0], lg_o) < (1e-1 if q4 else 5e-2) and rel_err(lg[1], lg_0) < (1e-1 if q4 else 5e-2)
        assert int(nxt[0]) == tok_o or q4
    pos, seq, _ = gm.kv_cells_state()
    assert np.count_nonzero(seq >> 3 & 1) == n_prompt + 3
    for om in oms + [om3]:
        om.close()
    gm.close()


@pytest.mark.parametrize("arch", ["llama-tiny", "falcon-tiny"])
def test_a_context_shift_in_the_shared_cell_cache(arch):
    """The context shift of examples/main (llama_kv_cache_seq_rm of a range, llama_kv_cache_seq_shift of what lies behind it): the
    positions move at once, the K rows are rotated at the start of the next step (llm_build_k_shift on the reference's cache layout).
    The steps after the shift against this library's per-sequence cache doing the same edit (pi_model_kv_seq_rm / _seq_shift, which
    the reference's own context-shift logits pin, tests/test_gpu_model.py), and a second sequence that shares the shifted cells."""
    from powerinfer_amd.model import Model
    hp = synth.hparams(arch, seed=9, n_ctx=64, pred_margin=True, head_pair=2048)      # no neuron on the threshold: the two attention kernels round differently
    model = synth.make_model(hp)
    rng = np.random.default_rng(5)
    toks = rng.integers(0, hp.n_vocab, 20)
    ga, gb = Model(hp).load(model), Model(hp).load(model)
    gb.kv_cells_init(32)
    for i in range(12):
        _, la = ga.decode([int(toks[i])], i)
        _, lb = gb.kv_cells_decode([toks[i]], [i], [0])
        assert rel_err(lb[0], la) < 1e-2, (i, rel_err(lb[0], la))
    gb.kv_cells_seq_cp(0, 1, 0, -1)                              # sequence 1 shares every cell: the shift below moves them for both
    ga.kv_seq_rm(2, 6)
    ga.kv_seq_shift(6, -1, -4)
    gb.kv_cells_seq_rm(0, 2, 6)
    gb.kv_cells_seq_rm(1, 2, 6)
    gb.kv_cells_seq_shift(0, 6, -1, -4)
    pos, seq, head = gb.kv_cells_state()
    assert list(pos[:12]) == [0, 1, -1, -1, -1, -1, 2, 3, 4, 5, 6, 7] and np.all(seq[6:12] == 0b11) and head == 0
    for i in range(12, 16):
        _, la = ga.decode([int(toks[i])], i - 4)
        nxt, lb = gb.kv_cells_decode([toks[i], toks[i]], [i - 4, i - 4], [0, 1])      # both sequences take the same token: same logits
        assert rel_err(lb[0], la) < 1e-2 and rel_err(lb[1], la) < 1e-2, (i, rel_err(lb[0], la), rel_err(lb[1], la))
    pos, _, _ = gb.kv_cells_state()
    assert list(pos[2:6]) == [8, 8, 9, 9]                        # the freed cells were found again, two per step
    ga.close(), gb.close()


def test_kv_cells_refuse_what_they_cannot_hold():
    from powerinfer_amd import lib as pl
    from powerinfer_amd.model import Model
    hp = synth.hparams("llama-tiny", seed=2, n_ctx=32)
    gm = Model(hp).load(synth.make_model(hp))
    with pytest.raises(pl.PiError):
        gm.kv_cells_decode([1], [0], [0])                        # not initialised
    with pytest.raises(pl.PiError):
        gm.kv_cells_init(40)                                     # not a multiple of 32
    gm.kv_cells_init(32)
    with pytest.raises(pl.PiError):
        gm.kv_cells_decode(list(range(17)), list(range(17)), [0] * 17)
    gm.close()
    hp = synth.hparams("llama-tiny", seed=2, n_ctx=32, hot_frac=0.5)
    gm = Model(hp).load(synth.make_model(hp))
    with pytest.raises(pl.PiError):
        gm.kv_cells_init(32)                                     # a VRAM split: the host computes part of every layer
    gm.close()
