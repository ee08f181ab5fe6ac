"""The decode engine against vectors produced by the REFERENCE's own llama.cpp CPU path (tests/golden/ref_*.npz,
written by tests/golden/make_llama_fixture.py).  The model travels the way a user's would: synthetic weights are
written as a PowerInfer GGUF file, read back with powerinfer_amd.gguf.read_model and loaded through the C ABI.
Both sides consume the reference's token sequence (teacher forcing), so one early flip does not decide the rest."""
import importlib.util
import os

import numpy as np
import pytest

from powerinfer_amd import gguf

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
spec = importlib.util.spec_from_file_location("make_llama_fixture", os.path.join(ROOT, "tests", "golden", "make_llama_fixture.py"))
fx = importlib.util.module_from_spec(spec)
spec.loader.exec_module(fx)


@pytest.mark.parametrize("name", ["llama_f16", "llama_q4", "falcon_f16"])
def test_engine_from_gguf_matches_reference_llama_cpp(name, tmp_path):
    from powerinfer_amd.model import Model
    g = dict(np.load(os.path.join(ROOT, "tests", "golden", f"ref_{name}.npz")))
    hp0, model = fx.case_model(name)
    if not np.array_equal(fx.model_sha(model), g["model_sha"]):
        pytest.skip("numpy generates a different stream here than where the fixture was written")
    path = str(tmp_path / "m.powerinfer.gguf")
    gguf.write_model(path, model, {})                       # the engine needs no tokenizer entries
    hp, loaded = gguf.read_model(path, n_ctx=hp0.n_ctx)
    for k in ("n_embd", "n_ff", "n_head", "n_head_kv", "n_layer", "n_vocab", "n_rank", "wtype", "arch"):
        assert hp[k] == hp0[k], k
    gm = Model(hp).load(loaded)
    errs, same = [], 0
    for s, tok in enumerate(g["consumed"]):
        best, lg = gm.decode([int(tok)], s)
        errs.append(float(np.abs(lg[g["sample_idx"]] - g["logits_sample"][s]).max() / g["logits_absmax"][s]))
        same += int(best == g["greedy"][s])
    errs = np.array(errs)
    # logits tolerance of the north star (1e-2 relative); the median shows the typical agreement
    assert errs.max() < 1e-2, errs
    assert np.median(errs) < 2e-3, errs
    assert same >= len(errs) - 1, (same, len(errs))


@pytest.mark.parametrize("name", ["llama_f16_shift", "falcon_f16_shift", "llama_f16_scaled_shift", "falcon_f16_scaled_shift"])
def test_context_shift_matches_reference_llama_cpp(name):
    """llama_kv_cache_seq_rm + llama_kv_cache_seq_shift before step 12 (what examples/main does when the context is full): the
    engine squeezes the removed cells out and rotates the shifted K rows; the reference's logits after the shift are the check."""
    from powerinfer_amd.model import Model
    g = dict(np.load(os.path.join(ROOT, "tests", "golden", f"ref_{name}.npz")))
    hp, model = fx.case_model(name)
    if not np.array_equal(fx.model_sha(model), g["model_sha"]):
        pytest.skip("numpy generates a different stream here than where the fixture was written")
    shift_at, n_keep, n_discard = (int(v) for v in g["shift"])
    gm = Model(hp).load(model)
    errs, same, n_past = [], 0, 0
    for s, tok in enumerate(g["consumed"]):
        if s == shift_at:
            assert gm.kv_seq_rm(n_keep, n_keep + n_discard) == n_past - n_discard
            with pytest.raises(Exception):                   # positions 0,1,6,7,.. : a gap is open
                gm.decode([int(tok)], n_past)
            assert gm.kv_seq_shift(n_keep + n_discard, n_past, -n_discard) == n_past - n_discard
            n_past -= n_discard
        best, lg = gm.decode([int(tok)], n_past)
        errs.append(float(np.abs(lg[g["sample_idx"]] - g["logits_sample"][s]).max() / g["logits_absmax"][s]))
        same += int(best == g["greedy"][s])
        n_past += 1
    errs = np.array(errs)
    assert errs.max() < 1e-2, errs
    assert np.median(errs) < 2e-3, errs
    assert np.median(errs[shift_at:]) < 2e-3, errs
    assert same >= len(errs) - 1, (same, len(errs))


def test_generate_continues_behind_a_context_shift():
    """pi_model_generate picks up at the shifted position: tokens after rm + shift equal those of explicit decode calls."""
    from powerinfer_amd.model import Model
    hp, model = fx.case_model("llama_f16_shift")
    prompt = np.random.default_rng(3).integers(0, hp.n_vocab, 12)

    def run(use_generate):
        gm = Model(hp).load(model)
        tok, _ = gm.decode(prompt, 0)
        gm.kv_seq_rm(2, 6)
        assert gm.kv_seq_shift(6, 12, -4) == 8
        if use_generate:
            return [tok] + [int(t) for t in gm.generate(5)[0]]
        out, n_past = [tok], 8
        for _ in range(5):
            tok, _ = gm.decode([tok], n_past)
            out.append(tok)
            n_past += 1
        return out

    a, b = run(True), run(False)
    assert a == b, (a, b)
