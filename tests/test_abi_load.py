"""CPU-side check of the boundary: the shared library loads and exports every entry point that
include/*.h declares (no device call is made)."""
import os
import re

from powerinfer_amd import lib as pl

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_in_headers():
    names = set()
    for fn in os.listdir(os.path.join(ROOT, "include")):
        if fn.endswith(".h"):
            src = open(os.path.join(ROOT, "include", fn)).read()
            src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
            src = re.sub(r"#define[^\n]*", "", src)
            names |= set(re.findall(r"(?:PI_API|GGML_API)\s+[^;{]*?\b(\w+)\s*\(", src))
    return names


def test_library_exports_every_declared_symbol():
    L = pl.load()
    names = declared_in_headers()
    assert len(names) >= 20
    missing = [n for n in sorted(names) if not hasattr(L, n)]
    assert not missing, missing


def test_python_binding_covers_the_header():
    names = {n for n in declared_in_headers() if n.startswith("pi_")}
    assert names <= set(pl.declared_symbols()), names - set(pl.declared_symbols())
