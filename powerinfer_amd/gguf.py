"""GGUF v3 container reader/writer (ggml.c:19384-19672 of the reference), including the PowerInfer variant whose
magic is "PWRI" (ggml.h:246-247), and the mapping between a `*.powerinfer.gguf` file and the tensor dict the engine
loads (tensor names: llama.cpp:403-461).

    magic[4] | u32 version = 3 | u64 n_tensors | u64 n_kv | kv... | tensor infos... | pad to alignment | tensor data

A kv is: string key (u64 length + bytes), u32 value type, value; arrays are u32 element type, u64 count, payload.
A tensor info is: string name, u32 n_dims, u64 ne[n_dims], u32 ggml type, u64 offset into the data section.
"""
import struct

import numpy as np

F32, F16, Q4_0, I32 = 0, 1, 2, 18
T_U8, T_I8, T_U16, T_I16, T_U32, T_I32, T_F32, T_BOOL, T_STR, T_ARR, T_U64, T_I64, T_F64 = range(13)
_SCALAR = {T_U8: "<B", T_I8: "<b", T_U16: "<H", T_I16: "<h", T_U32: "<I", T_I32: "<i", T_F32: "<f", T_BOOL: "<?", T_U64: "<Q", T_I64: "<q", T_F64: "<d"}
_NP = {F32: np.float32, F16: np.float16, Q4_0: np.uint8, I32: np.int32}


def _row_bytes(t, ne0):
    return {F32: 4 * ne0, I32: 4 * ne0, F16: 2 * ne0, Q4_0: ne0 // 32 * 18}[t]


class _Reader:
    def __init__(self, buf):
        self.b, self.o = buf, 0

    def take(self, fmt):
        v = struct.unpack_from(fmt, self.b, self.o)
        self.o += struct.calcsize(fmt)
        return v[0] if len(v) == 1 else v

    def string(self):
        n = self.take("<Q")
        s = bytes(self.b[self.o:self.o + n])
        self.o += n
        return s

    def value(self, t):
        if t == T_STR:
            return self.string()
        if t == T_ARR:
            et, n = self.take("<I"), self.take("<Q")
            if et in _SCALAR and et != T_BOOL:
                dt = np.dtype(_SCALAR[et])
                a = np.frombuffer(self.b, dt, n, self.o).copy()
                self.o += n * dt.itemsize
                return (et, a)
            return (et, [self.value(et) for _ in range(n)])
        return self.take(_SCALAR[t])


def read_gguf(path):
    """Returns (magic, kv, tensors): kv maps key -> (type, value); tensors maps name -> (ggml_type, ne tuple, numpy view
    onto a read-only memory map, shaped [rows..., row_bytes-or-ne0])."""
    mm = np.memmap(path, np.uint8, "r")
    r = _Reader(mm)
    magic = bytes(mm[:4])
    r.o = 4
    if magic not in (b"GGUF", b"PWRI"):
        raise ValueError(f"{path}: not a GGUF file (magic {magic!r})")
    version, n_tensors, n_kv = r.take("<I"), r.take("<Q"), r.take("<Q")
    if version not in (2, 3):      # v2 and v3 share the little-endian layout (64-bit counts); v1 used 32-bit counts
        raise ValueError(f"{path}: GGUF version {version} is not supported (2 or 3 expected)")
    kv = {}
    for _ in range(n_kv):
        k = r.string().decode()
        t = r.take("<I")
        kv[k] = (t, r.value(t))
    infos = []
    for _ in range(n_tensors):
        name = r.string().decode()
        nd = r.take("<I")
        ne = tuple(r.take("<Q") for _ in range(nd))
        t, off = r.take("<I"), r.take("<Q")
        infos.append((name, t, ne, off))
    align = kv.get("general.alignment", (T_U32, 32))[1]
    base = (r.o + align - 1) // align * align
    tensors = {}
    for name, t, ne, off in infos:
        if t not in _NP:
            raise ValueError(f"{path}: tensor {name} has unsupported ggml type {t}")
        rows = int(np.prod(ne[1:])) if len(ne) > 1 else 1
        rb = _row_bytes(t, ne[0])
        raw = mm[base + off: base + off + rb * rows]
        tensors[name] = (t, ne, raw.view(_NP[t]).reshape(rows, -1) if rows > 1 else raw.view(_NP[t]))
    return magic, kv, tensors


def _w_str(out, s):
    s = s if isinstance(s, bytes) else s.encode()
    out.append(struct.pack("<Q", len(s)))
    out.append(s)


def _w_val(out, t, v):
    if t == T_STR:
        _w_str(out, v)
    elif t == T_ARR:
        et, items = v
        out.append(struct.pack("<IQ", et, len(items)))
        if et in _SCALAR and et != T_BOOL:
            out.append(np.asarray(items, np.dtype(_SCALAR[et])).tobytes())
        else:
            for it in items:
                _w_val(out, et, it)
    else:
        out.append(struct.pack(_SCALAR[t], v))


def write_gguf(path, kv, tensors, magic=b"PWRI", align=32):
    """kv: key -> (type, value); tensors: name -> (ggml_type, ne tuple, numpy array holding the raw rows)."""
    out = [magic, struct.pack("<IQQ", 3, len(tensors), len(kv))]
    for k, (t, v) in kv.items():
        _w_str(out, k)
        out.append(struct.pack("<I", t))
        _w_val(out, t, v)
    off, blobs = 0, []
    for name, (t, ne, arr) in tensors.items():
        raw = np.ascontiguousarray(arr).view(np.uint8).reshape(-1)
        _w_str(out, name)
        out.append(struct.pack("<I", len(ne)))
        out.append(struct.pack("<%dQ" % len(ne), *ne))
        out.append(struct.pack("<IQ", t, off))
        pad = (-raw.size) % align
        blobs.append((raw, pad))
        off += raw.size + pad
    head = b"".join(out)
    with open(path, "wb") as f:
        f.write(head)
        f.write(b"\0" * ((-len(head)) % align))
        for raw, pad in blobs:
            f.write(raw.tobytes())
            f.write(b"\0" * pad)


# ---- model <-> file ------------------------------------------------------------------------------------
_LAYER_NAMES = {  # role in powerinfer_amd.model.KINDS -> tensor name suffix (llama.cpp:403-461)
    "attn_norm": "attn_norm.weight", "attn_norm_b": "attn_norm.bias", "attn_norm_2": "attn_norm_2.weight", "attn_norm_2_b": "attn_norm_2.bias",
    "wq": "attn_q.weight", "wk": "attn_k.weight", "wv": "attn_v.weight", "wqkv": "attn_qkv.weight", "wo": "attn_output.weight",
    "ffn_norm": "ffn_norm.weight", "ffn_gate": "ffn_gate.weight", "ffn_up": "ffn_up.weight", "ffn_down_t": "ffn_down_t.weight",
    "fc1": "fc1.weight", "fc2": "fc2.weight",
}
_GLOBAL_NAMES = {"tok_embd": "token_embd.weight", "output_norm": "output_norm.weight", "output_norm_b": "output_norm.bias", "output": "output.weight"}


def _ne_of(arr, t):
    if arr.ndim == 1:
        return (arr.shape[0],)
    return ((arr.shape[1] // 18 * 32) if t == Q4_0 else arr.shape[1], arr.shape[0])


def _gtype(arr):
    return {np.dtype(np.float32): F32, np.dtype(np.float16): F16, np.dtype(np.uint8): Q4_0, np.dtype(np.int32): I32}[arr.dtype]


def synthetic_tokenizer_kv(n_vocab):
    """`tokenizer.*` entries of a made-up SentencePiece-type vocabulary of n_vocab distinct strings, enough for the reference's
    loader (llm_load_vocab, llama.cpp:2473-2700) to accept a synthetic model of either architecture: ids 0..2 are <unk> <s> </s>,
    3..258 the byte tokens <0x00>..<0xFF> (the loader looks the newline up as <0x0A>), the rest plain words.  Logits do not
    depend on any of it."""
    if n_vocab < 259:
        raise ValueError("a SentencePiece vocabulary needs the 3 control and 256 byte tokens")
    words = [b"<unk>", b"<s>", b"</s>"] + [b"<0x%02X>" % i for i in range(256)] + [b"w%d" % i for i in range(259, n_vocab)]
    types = np.ones(n_vocab, np.int32)              # normal
    types[0], types[1:3], types[3:259] = 2, 3, 6    # unknown, control, byte
    return {
        "tokenizer.ggml.model": (T_STR, b"llama"),
        "tokenizer.ggml.tokens": (T_ARR, (T_STR, words)),
        "tokenizer.ggml.scores": (T_ARR, (T_F32, np.zeros(n_vocab, np.float32))),
        "tokenizer.ggml.token_type": (T_ARR, (T_I32, types)),
        "tokenizer.ggml.bos_token_id": (T_U32, 1), "tokenizer.ggml.eos_token_id": (T_U32, 2), "tokenizer.ggml.unknown_token_id": (T_U32, 0),
    }


def write_model(path, model, tokenizer_kv):
    """Writes a synthetic model (powerinfer_amd.synth.make_model) as a PowerInfer GGUF.  tokenizer_kv: the
    `tokenizer.*` entries of a vocabulary file whose token count equals hp.n_vocab."""
    hp = model["hp"]
    arch = hp.arch
    kv = {
        "general.architecture": (T_STR, arch), "general.name": (T_STR, "synthetic-" + hp.name),
        f"{arch}.context_length": (T_U32, hp.n_ctx), f"{arch}.embedding_length": (T_U32, hp.n_embd),
        f"{arch}.feed_forward_length": (T_U32, hp.n_ff), f"{arch}.block_count": (T_U32, hp.n_layer),
        f"{arch}.attention.head_count": (T_U32, hp.n_head), f"{arch}.attention.head_count_kv": (T_U32, hp.n_head_kv),
        f"{arch}.rope.dimension_count": (T_U32, hp.n_embd // hp.n_head), f"{arch}.rope.freq_base": (T_F32, hp.rope_freq_base),
        (f"{arch}.attention.layer_norm_rms_epsilon" if arch == "llama" else f"{arch}.attention.layer_norm_epsilon"): (T_F32, hp.norm_eps),
        "powerinfer.sparse_threshold": (T_F32, hp.sparse_threshold),
    }
    if hp.get("rope_freq_scale", 1.0) != 1.0:             # stored as its inverse, with the scaling type the loader defaults to (llama.cpp:2316-2328)
        kv[f"{arch}.rope.scaling.type"] = (T_STR, "linear")
        kv[f"{arch}.rope.scaling.factor"] = (T_F32, 1.0 / hp.rope_freq_scale)
    kv.update(tokenizer_kv)
    tensors = {}
    for k, a in model["glob"].items():
        tensors[_GLOBAL_NAMES[k]] = (_gtype(a), _ne_of(a, _gtype(a)), a)
    for il, L in enumerate(model["layers"]):
        for k, a in L.items():
            if k in _LAYER_NAMES and a is not None:
                tensors[f"blk.{il}.{_LAYER_NAMES[k]}"] = (_gtype(a), _ne_of(a, _gtype(a)), a)
    write_gguf(path, kv, tensors, b"PWRI")


def read_model(path, n_ctx=512):
    """Reads a PowerInfer GGUF (LLaMA or Falcon architecture) into (hp, model dict) for powerinfer_amd.model.Model.load."""
    from . import synth
    magic, kv, tensors = read_gguf(path)
    arch = kv["general.architecture"][1].decode()
    if arch not in ("llama", "falcon"):
        raise ValueError(f"{path}: architecture {arch!r} is outside this path (llama and falcon only)")
    g = lambda k, d=None: kv[k][1] if k in kv else d  # noqa: E731
    n_head = g(f"{arch}.attention.head_count")
    # linear RoPE scaling: the file holds 1 / freq_scale under the new key or the old one (llama.cpp:2316-2328); type "none"
    # switches it off (llama.cpp:9869-9871) and YaRN is outside the fused token loop
    scaling = g(f"{arch}.rope.scaling.type", b"linear").decode()
    if scaling not in ("linear", "none"):
        raise ValueError(f"{path}: rope scaling type {scaling!r} is outside this path (linear only)")
    factor = g(f"{arch}.rope.scaling.factor", 0.0) or g(f"{arch}.rope.scale_linear", 0.0)
    freq_scale = 1.0 if scaling == "none" or factor == 0.0 else float(np.float32(1.0) / np.float32(factor))
    hp = synth.HParams(arch=arch, name=g("general.name", b"?").decode(), n_embd=g(f"{arch}.embedding_length"),
                       n_ff=g(f"{arch}.feed_forward_length"), n_head=n_head, n_head_kv=g(f"{arch}.attention.head_count_kv", n_head),
                       n_layer=g(f"{arch}.block_count"), n_vocab=tensors["token_embd.weight"][1][1], n_ctx=n_ctx,
                       norm_eps=g(f"{arch}.attention.layer_norm_rms_epsilon", g(f"{arch}.attention.layer_norm_epsilon", 1e-5)),
                       rope_freq_base=g(f"{arch}.rope.freq_base", 10000.0), rope_freq_scale=freq_scale, sparse_threshold=g("powerinfer.sparse_threshold", 0.0),
                       sparse=(magic == b"PWRI"))
    hp["n_rank"] = tensors["blk.0.fc1.weight"][1][1]
    hp["wtype"] = tensors["blk.0.ffn_up.weight"][0]
    glob = {k: tensors[n][2] for k, n in _GLOBAL_NAMES.items() if n in tensors}
    layers = []
    for il in range(hp.n_layer):
        layers.append({k: tensors[f"blk.{il}.{n}"][2] for k, n in _LAYER_NAMES.items() if f"blk.{il}.{n}" in tensors})
    return hp, dict(hp=hp, glob=glob, layers=layers)


def read_gpu_split(path, n_layer):
    """`*.generated.gpuidx` (export_split.py:54-76): GGUF with arch generic.gpu_index, tensors blk.N.gpu_idx /
    blk.N.gpu_bucket.  Returns a list of (gpu_idx, gpu_bucket) per layer."""
    _, kv, tensors = read_gguf(path)
    out = []
    for il in range(n_layer):
        out.append((np.asarray(tensors[f"blk.{il}.gpu_idx"][2], np.int32), np.asarray(tensors[f"blk.{il}.gpu_bucket"][2], np.int32)))
    return out
