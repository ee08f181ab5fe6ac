"""The oracle's whole-model evaluation (pio_model_eval: the wiring of build_llama_variants / build_falcon with
llm_build_ffn_sparse, attention, norms, RoPE, KV cache, lm-head) against golden vectors produced by the REFERENCE's
own llama.cpp CPU path on a synthetic PowerInfer GGUF (tests/golden/make_llama_fixture.py, one thread)."""
import importlib.util
import os

import numpy as np
import pytest

import oracle_lib as ol

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
