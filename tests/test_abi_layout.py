"""include/ggml_backend_abi.h must lay out struct ggml_tensor / ggml_compute_params and number the enumerators
exactly as the reference's ggml.h does (tests/golden/ggml_abi.json was produced by compiling a probe against the
reference's own header, tests/golden/make_abi_fixture.py)."""
import importlib.util
import json
import os

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_tensor_layout_and_enums_match_reference_header():
    spec = importlib.util.spec_from_file_location("make_abi_fixture", os.path.join(ROOT, "tests", "golden", "make_abi_fixture.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    mine = mod.probe("ggml_backend_abi.h", os.path.join(ROOT, "include"))
    with open(os.path.join(ROOT, "tests", "golden", "ggml_abi.json")) as f:
        ref = json.load(f)
    assert mine == ref, {k: (mine.get(k), ref.get(k)) for k in ref if mine.get(k) != ref.get(k)}
    assert ref["GGML_OP_MUL_MAT_SPARSE"] == 24 and ref["GGML_OP_AXPY"] == 25
