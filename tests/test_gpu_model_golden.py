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
