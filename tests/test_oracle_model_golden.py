"""The oracle's whole-model evaluation (pio_model_eval: the wiring of build_llama_variants / build_falcon with
llm_build_ffn_sparse, attention, norms, RoPE, KV cache, lm-head) against golden vectors produced by the REFERENCE's
own llama.cpp CPU path on a synthetic PowerInfer GGUF (tests/golden/make_llama_fixture.py, one thread)."""
import importlib.util
import os

import numpy as np
import pytest

import oracle_lib as ol
from powerinfer_amd import synth

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
spec = importlib.util.spec_from_file_location("make_llama_fixture", os.path.join(ROOT, "tests", "golden", "make_llama_fixture.py"))
fx = importlib.util.module_from_spec(spec)
spec.loader.exec_module(fx)


@pytest.mark.parametrize("name", ["llama_f16", "llama_q4", "falcon_f16"])
def test_model_eval_matches_reference_llama_cpp(name):
    g = dict(np.load(os.path.join(ROOT, "tests", "golden", f"ref_{name}.npz")))
    hp, model = fx.case_model(name)
    if not np.array_equal(fx.model_sha(model), g["model_sha"]):
        pytest.skip("numpy generates a different stream here than where the fixture was written")
    om = ol.OracleModel(model)
    worst = 0.0
    for s, tok in enumerate(g["consumed"]):
        best, lg = om.eval([int(tok)], s, nth=1)
        err = np.abs(lg[g["sample_idx"]] - g["logits_sample"][s]).max() / g["logits_absmax"][s]
        worst = max(worst, float(err))
        assert best == g["greedy"][s], (s, best, g["greedy"][s])
        assert abs(lg.max() - g["logits_max"][s]) <= 1e-5 * g["logits_absmax"][s]
    # same arithmetic, same order (single thread): agreement at fp32 round-off
    assert worst < 1e-5, worst
    om.close()


@pytest.mark.parametrize("name", ["llama_f16_shift", "falcon_f16_shift", "llama_f16_scaled_shift", "falcon_f16_scaled_shift"])
def test_context_shift_matches_reference_llama_cpp(name):
    """KV ring slots, cell mask and K-shift: before step 12 the reference removed positions [2, 6) and shifted the later cells by
    -4 (llama_kv_cache_seq_rm + llama_kv_cache_seq_shift); the next llama_decode rotated the cached K rows (llm_build_k_shift)
    and stored new tokens in the freed cells.  The oracle repeats that with the reference's cell bookkeeping."""
    g = dict(np.load(os.path.join(ROOT, "tests", "golden", f"ref_{name}.npz")))
    hp, model = fx.case_model(name)
    if not np.array_equal(fx.model_sha(model), g["model_sha"]):
        pytest.skip("numpy generates a different stream here than where the fixture was written")
    shift_at, n_keep, n_discard = (int(v) for v in g["shift"])
    om = ol.OracleModel(model)
    cells = ol.KVCells(hp.n_ctx)
    n_past, worst = 0, 0.0
    for s, tok in enumerate(g["consumed"]):
        if s == shift_at:
            cells.seq_rm(0, n_keep, n_keep + n_discard)
            cells.seq_shift(0, n_keep + n_discard, n_past, -n_discard)
            n_past -= n_discard
        if cells.has_shift:                              # llama_decode_internal applies pending shifts first (llama.cpp:5494-5500, 6921-6929)
            om.k_shift(cells.delta)
            cells.has_shift = False
            cells.delta[:] = 0
        slot = cells.find_slot([n_past])
        n_kv = min(hp.n_ctx, max(32, cells.cell_max()))                      # llama.cpp:6842
        best, lg = om.eval_cells([int(tok)], [n_past], [slot], n_kv, cells.mask([n_past], n_kv))
        if s == shift_at:
            assert slot == n_keep and slot != n_past     # the ring reuses the freed cells
        err = np.abs(lg[g["sample_idx"]] - g["logits_sample"][s]).max() / g["logits_absmax"][s]
        worst = max(worst, float(err))
        assert best == g["greedy"][s], (s, best, g["greedy"][s])
        n_past += 1
    assert worst < 1e-5, worst
    om.close()


def test_sequence_edits_match_reference_llama_cpp():
    """Three sequences sharing one KV cache (llama_batch entries with sequence ids), then llama_kv_cache_seq_rm, _seq_shift and
    _seq_cp: one sequence takes a context shift, one is emptied and handed the first six cells of its neighbour.  The reference
    wrote the logits of the last lockstep step (tests/golden/ref_llama_seq_edits.npz); the oracle repeats the history with the
    reference's cell bookkeeping (ring slots, owners per cell, pending K-shift, per-token mask)."""
    g = dict(np.load(os.path.join(ROOT, "tests", "golden", "ref_llama_seq_edits.npz")))
    hp, toks, last_pos, _ = fx.seq_edit_case()
    model = synth.make_model(hp)
    if not np.array_equal(fx.model_sha(model), g["model_sha"]):
        pytest.skip("numpy generates a different stream here than where the fixture was written")
    assert np.array_equal(toks, g["tokens"])
    om = ol.OracleModel(model)
    cells = ol.KVCells(hp.n_ctx)
    n_seq, n0 = toks.shape[1], toks.shape[0] - 1
    seqs = list(range(n_seq))

    def step(tokens, positions):
        if cells.has_shift:
            om.k_shift(cells.delta)
            cells.has_shift = False
            cells.delta[:] = 0
        slot = cells.find_slot(positions, seqs)
        n_kv = min(hp.n_ctx, max(32, cells.cell_max()))
        return om.eval_cells(tokens, positions, [slot + i for i in range(n_seq)], n_kv, cells.mask(positions, n_kv, seqs), all_logits=True)[1]

    for s in range(n0):
        lg = step(toks[s], [s] * n_seq)
        if s == 0:
            assert np.abs(lg - g["logits_step0"]).max() <= 1e-5 * np.abs(g["logits_step0"]).max()
    cells.seq_rm(0, 2, 5)
    cells.seq_shift(0, 5, 8, -3)
    cells.seq_rm(2, 0, -1)
    cells.seq_cp(1, 2, 0, 6)
    lg = step(toks[n0], list(g["last_pos"]))
    assert np.abs(lg - g["logits_last"]).max() <= 1e-5 * np.abs(g["logits_last"]).max()
    assert np.array_equal(lg.argmax(1), g["logits_last"].argmax(1))
    om.close()
