"""VRAM-budget planning of the hot/cold split (host side).

What the reference does between `--vram-budget` and the `gpu_idx` / `gpu_bucket` tensors of every layer:

1. dense tensors are offloaded by priority while the budget lasts: attention (weights and norms), then the predictors,
   then ffn_norm, then output + output_norm, each level in layer order; the first tensor that does not fit ends the
   offload (buffered_tensor_allocator::flush, llama.cpp:3047-3078; levels llama.cpp:644-676);
2. if everything above fits, the K and the V cache are reserved (llama.cpp:3400-3420);
3. what is left buys hot neurons: capacity = floor(budget / (slice * (4.5 with a gate | 2 without))) * 4 neurons with
   slice = ne[1](ffn_up) * type_size / block_size (llm_load_gpu_split_with_budget, llama.cpp:3115-3118);
4. `python -m powerinfer` distributes that capacity over the layers by an integer program over batches of 256 neurons sorted
   by activation count (solver.py:8-100) and writes, per layer, the top-k neurons as gpu_idx (1 = on the GPU) and their
   sorted indices as gpu_bucket (export_split.py:24-52) into `<model>.generated.gpuidx`.

Step 4's solver needs cvxopt/GLPK; `solve_counts` solves the same program exactly by dynamic programming instead (a selected
batch is worth its summed activation count, a layer takes none or at least `threshold` neurons, at most `capacity` in total).
"""
import numpy as np

from . import gguf

TYPE_BYTES = {gguf.F32: (4, 1), gguf.F16: (2, 1), gguf.Q4_0: (18, 32), gguf.I32: (4, 1)}     # (type size, block size)


def nbytes(t, *ne):
    size, blk = TYPE_BYTES[t]
    return int(np.prod(ne)) // blk * size


def dense_tensor_queue(hp):
    """(level, layer, name, bytes) of every tensor the allocator queues, in its flush order."""
    d, ff, r, wt = hp.n_embd, hp.n_ff, hp.n_rank, hp.wtype
    gqa = d // hp.n_head * hp.n_head_kv
    falcon = hp.arch == "falcon"
    attn, pred, ffn_io = [], [], []
    for il in range(hp.n_layer):
        attn.append((il, "attn_norm", nbytes(gguf.F32, d) * (2 if falcon else 1)))
        if falcon and hp.n_head_kv != hp.n_head:
            attn.append((il, "attn_norm_2", 2 * nbytes(gguf.F32, d)))
        if falcon:
            attn.append((il, "attn_qkv", nbytes(wt, d, d + 2 * gqa)))
        else:
            attn += [(il, "attn_q", nbytes(wt, d, d)), (il, "attn_k", nbytes(wt, d, gqa)), (il, "attn_v", nbytes(wt, d, gqa))]
        attn.append((il, "attn_output", nbytes(wt, d, d)))
        pred += [(il, "fc1", nbytes(gguf.F16, d, r)), (il, "fc2", nbytes(gguf.F16, r, ff))]
        if not falcon:
            ffn_io.append((il, "ffn_norm", nbytes(gguf.F32, d)))
    out = [(-1, "output_norm", nbytes(gguf.F32, d) * (2 if falcon else 1)), (-1, "output", nbytes(wt, d, hp.n_vocab))]
    q = [("attn", *t) for t in attn] + [("mlp_pred", *t) for t in pred] + [("ffn_io", *t) for t in ffn_io] + [("output", *t) for t in out]
    return q


def offload_plan(hp, budget_bytes, n_ctx, f16_kv=True):
    """Walks the budget the way the loader does.  Returns dict(offloaded_layers, complete, kv_on_gpu, dense_bytes,
    remaining_bytes, neuron_capacity)."""
    left = int(budget_bytes)
    offloaded_layers, complete, dense = 0, True, 0
    for level, il, name, size in dense_tensor_queue(hp):
        if size > left:
            complete = False
            break
        left -= size
        dense += size
        if level == "attn" and name == "attn_output":
            offloaded_layers = il + 1
        elif level == "output":
            offloaded_layers = hp.n_layer + 1
    kv = 0
    if complete:
        gqa = hp.n_embd // hp.n_head * hp.n_head_kv
        cache = gqa * hp.n_layer * n_ctx * (2 if f16_kv else 4)
        for _ in range(2):
            if cache > left:
                break
            left -= cache
            kv += 1
    if not complete:
        cap = 0
    else:
        size, blk = TYPE_BYTES[hp.wtype]
        slice_size = hp.n_ff * size // blk                      # ne[1] of ffn_up, as the reference computes it
        per_slice = int(slice_size * (2 if hp.arch == "falcon" else 4.5))
        cap = left // per_slice * 4
    return dict(offloaded_layers=offloaded_layers, complete=complete, kv_on_gpu=kv == 2, dense_bytes=dense, remaining_bytes=left,
                neuron_capacity=int(cap))


def solve_counts(rates, capacity, batch=256, threshold=0):
    """Neurons per layer to keep on the GPU.  rates: one array of activation counts (or firing rates) per layer.
    Layers are cut into batches of `batch` neurons in descending order of rate; choosing the j hottest batches of layer i is
    worth the sum of their rates; at most capacity // batch batches in total; a layer gets none or at least
    threshold // batch.  Exact (dynamic programming over layers), ties resolved towards lower layers."""
    L = len(rates)
    cap = int(capacity) // batch
    thr = int(threshold) // batch
    pref = []
    for r in rates:
        s = np.sort(np.asarray(r, np.float64))[::-1]
        nb = s.size // batch
        v = s[:nb * batch].reshape(nb, batch).sum(1)
        pref.append(np.concatenate([[0.0], np.cumsum(v)]))          # pref[k] = value of the k hottest batches
    NEG = -1e300
    best = np.full(cap + 1, NEG)
    best[0] = 0.0
    choice = []
    for i in range(L):
        nb = pref[i].size - 1
        new = best.copy()                                          # k = 0
        ch = np.zeros(cap + 1, np.int64)
        for k in range(max(thr, 1), min(nb, cap) + 1):
            cand = np.full(cap + 1, NEG)
            cand[k:] = best[:cap + 1 - k] + pref[i][k]
            better = cand > new
            new[better] = cand[better]
            ch[better] = k
        choice.append(ch)
        best = new
    c = int(np.argmax(best))
    counts = [0] * L
    for i in range(L - 1, -1, -1):
        k = int(choice[i][c])
        counts[i] = k * batch
        c -= k
    return counts


def split_from_counts(rates, counts):
    """export_split.py:24-52: per layer the `count` hottest neurons; gpu_idx int32 [ff] (1 = on the GPU), gpu_bucket = their
    sorted indices."""
    out = []
    for r, k in zip(rates, counts):
        r = np.asarray(r)
        hot = np.argsort(-r, kind="stable")[:int(k)]
        gi = np.zeros(r.size, np.int32)
        gi[hot] = 1
        out.append((gi, np.sort(hot).astype(np.int32)))
    return out


def write_gpuidx(path, splits, vram_capacity):
    """`<model>.generated.gpuidx`: GGUF container with the PowerInfer magic, architecture generic.gpu_index, tensors
    blk.N.gpu_idx / blk.N.gpu_bucket and the key split.vram_capacity (export_split.py:54-76)."""
    kv = {"general.architecture": (gguf.T_STR, "generic.gpu_index"), "generic.gpu_index.block_count": (gguf.T_U32, len(splits)),
          "split.vram_capacity": (gguf.T_U64, int(vram_capacity))}
    tensors = {}
    for il, (gi, gb) in enumerate(splits):
        tensors[f"blk.{il}.gpu_idx"] = (gguf.I32, (gi.size,), gi.astype(np.int32))
        tensors[f"blk.{il}.gpu_bucket"] = (gguf.I32, (gb.size,), gb.astype(np.int32))
    gguf.write_gguf(path, kv, tensors, b"PWRI")


def required_bytes(hp, splits):
    """VRAM the split's FFN rows need (gate, up, down_t rows of every bucket)."""
    size, blk = TYPE_BYTES[hp.wtype]
    row = hp.n_embd * size // blk
    n_mats = 2 if hp.arch == "falcon" else 3
    return sum(int(gb.size) for _, gb in splits) * row * n_mats


def plan_split(hp, rates, budget_gb, n_ctx, batch=256, threshold=0):
    """--vram-budget in GiB -> (splits, report).  Raises if the dense tensors the engine keeps on the GPU do not fit."""
    budget = int(budget_gb * 1024 ** 3)
    rep = offload_plan(hp, budget, n_ctx)
    if not rep["complete"] or not rep["kv_on_gpu"]:
        raise ValueError("the VRAM budget does not hold the attention, predictor and output tensors plus the KV cache; "
                         "this engine keeps those on the GPU (offloaded_layers %d of %d)" % (rep["offloaded_layers"], hp.n_layer + 1))
    cap = min(rep["neuron_capacity"], hp.n_ff * hp.n_layer)
    counts = solve_counts(rates, cap, batch=batch, threshold=threshold)
    splits = split_from_counts(rates, counts)
    rep.update(counts=counts, ffn_bytes=required_bytes(hp, splits))
    return splits, rep
