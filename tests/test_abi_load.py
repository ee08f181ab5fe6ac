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


def test_attention_route_follows_the_kernels_own_lds_budget():
    """Host-side logic only: the decode loop takes the fused RoPE + attention kernel exactly where that kernel's launcher accepts
    the context (both keep every cell's score in LDS next to one partial row per group of lanes; the fused kernel's workgroup is
    four times larger), and the rope_kv_store + attn_decode pair beyond it."""
    L = pl.load()
    # head size 128 (7B, 13B): 60 KiB = 15360 floats = n_ctx + groups * 128 (+ q, k, v of the new cell for the fused kernel)
    assert L.pi_k_attn_fused_supported(128, 6784) == 1 and L.pi_k_attn_fused_supported(128, 6785) == 0
    assert L.pi_k_attn_decode_supported(128, 13312) == 1 and L.pi_k_attn_decode_supported(128, 13313) == 0
    assert L.pi_k_attn_fused_supported(128, 8192) == 0 and L.pi_k_attn_decode_supported(128, 8192) == 1     # takes the unfused pair
    # head size 64 (Falcon-40B)
    assert L.pi_k_attn_fused_supported(64, 6976) == 1 and L.pi_k_attn_fused_supported(64, 6977) == 0
    # head sizes outside 8 * (a divisor of 64)
    assert L.pi_k_attn_fused_supported(96, 512) == 0 and L.pi_k_attn_fused_supported(0, 512) == 0 and L.pi_k_attn_fused_supported(128, 0) == 0
