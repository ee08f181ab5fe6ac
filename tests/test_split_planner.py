"""VRAM-budget planner (host logic): offload order, neuron capacity, the per-layer distribution program and the split file."""
import itertools
import os

import numpy as np
import pytest

from powerinfer_amd import gguf, split, synth


def brute_force(rates, capacity, batch, threshold):
    L = len(rates)
    vals = []
    for r in rates:
        s = np.sort(np.asarray(r, np.float64))[::-1]
        nb = s.size // batch
        vals.append(np.concatenate([[0.0], np.cumsum(s[:nb * batch].reshape(nb, batch).sum(1))]))
    best, arg = -1.0, None
    for ks in itertools.product(*[range(v.size) for v in vals]):
        if sum(ks) > capacity // batch or any(0 < k < threshold // batch for k in ks):
            continue
        v = sum(vals[i][k] for i, k in enumerate(ks))
        if v > best + 1e-12:
            best, arg = v, ks
    return best, arg


@pytest.mark.parametrize("threshold", [0, 4, 6])
def test_solver_is_optimal_on_small_instances(threshold):
    rng = np.random.default_rng(threshold)
    for trial in range(20):
        L, nb, batch = 3, 5, 2
        rates = [rng.random(nb * batch) ** 3 * (1 + i) for i in range(L)]
        cap = int(rng.integers(0, L * nb * batch + 1))
        counts = split.solve_counts(rates, cap, batch=batch, threshold=threshold)
        assert sum(counts) <= cap and all(c % batch == 0 for c in counts)
        assert all(c == 0 or c >= threshold // batch * batch for c in counts)
        best, _ = brute_force(rates, cap, batch, threshold)
        got = sum(np.sort(r)[::-1][:c].sum() for r, c in zip(rates, counts))
        assert abs(got - best) < 1e-9, (trial, counts, got, best)


def test_solver_without_threshold_takes_the_globally_hottest_batches():
    rng = np.random.default_rng(1)
    rates = [synth.zipf_rates(2048, 0.1, rng)[0] for _ in range(4)]
    batch, cap = 256, 10 * 256
    counts = split.solve_counts(rates, cap, batch=batch)
    vals = sorted(((np.sort(r)[::-1].reshape(-1, batch).sum(1)[k], i) for i, r in enumerate(rates) for k in range(2048 // batch)), reverse=True)
    want = sum(v for v, _ in vals[:cap // batch])                  # layers share one rate distribution here, so counts may tie
    got = sum(np.sort(r)[::-1][:c].sum() for r, c in zip(rates, counts))
    assert sum(counts) == cap and abs(got - want) < 1e-9 * want


def test_offload_order_and_capacity():
    hp = synth.hparams("llama-7b", wtype=gguf.Q4_0)
    d, ff, r, L = hp.n_embd, hp.n_ff, hp.n_rank, hp.n_layer
    q4 = lambda n: n // 32 * 18  # noqa: E731
    attn = L * (4 * q4(d * d) + 4 * d)
    pred = L * (d * r + r * ff) * 2
    ffn_io = L * 4 * d
    out = q4(d * hp.n_vocab) + 4 * d
    kv = 2 * d * L * 512 * 2
    # attention only: stops inside the predictor level
    rep = split.offload_plan(hp, attn + 1000, 512)
    assert rep["offloaded_layers"] == L and not rep["complete"] and rep["neuron_capacity"] == 0
    # half of the attention: the layer count follows attn_output
    rep = split.offload_plan(hp, attn // 2, 512)
    assert 0 < rep["offloaded_layers"] < L and not rep["complete"]
    # everything dense + KV + room for neurons
    extra = 1 << 30
    rep = split.offload_plan(hp, attn + pred + ffn_io + out + kv + extra, 512)
    assert rep["complete"] and rep["kv_on_gpu"] and rep["offloaded_layers"] == L + 1 and rep["remaining_bytes"] == extra
    per_slice = int(q4(ff) * 4.5)                                # the reference's slice: ne[1] of ffn_up, x 4.5 with a gate
    assert rep["neuron_capacity"] == extra // per_slice * 4
    # Falcon: factor 2
    hf = synth.hparams("falcon-40b")
    rep = split.offload_plan(hf, 200 << 30, 512)
    assert rep["complete"] and rep["neuron_capacity"] == rep["remaining_bytes"] // int(hf.n_ff * 2 * 2) * 4


def test_plan_split_roundtrip_through_the_split_file(tmp_path):
    hp = synth.hparams("llama-tiny", n_layer=3)
    rng = np.random.default_rng(3)
    rates = [synth.zipf_rates(hp.n_ff, 0.15, rng)[0] for _ in range(hp.n_layer)]
    dense = split.offload_plan(hp, 1 << 40, 64)
    base = dense["dense_bytes"] + 2 * hp.n_embd * hp.n_layer * 64 * 2
    budget_gb = (base + int(2.5e6)) / 1024 ** 3
    splits, rep = split.plan_split(hp, rates, budget_gb, 64, batch=256)
    assert 0 < sum(rep["counts"]) <= rep["neuron_capacity"]
    for (gi, gb), r, k in zip(splits, rates, rep["counts"]):
        assert gi.sum() == k == gb.size and np.all(np.diff(gb) > 0) and np.all(gi[gb] == 1)
        if 0 < k < r.size:
            assert r[gb].min() >= np.delete(r, gb).max()             # the bucket holds the hottest neurons
    path = str(tmp_path / "m.generated.gpuidx")
    split.write_gpuidx(path, splits, int(budget_gb * 1024 ** 3))
    with open(path, "rb") as f:
        assert f.read(4) == b"PWRI"
    back = gguf.read_gpu_split(path, hp.n_layer)
    for (gi, gb), (gi2, gb2) in zip(splits, back):
        assert np.array_equal(gi, gi2) and np.array_equal(gb, gb2)
    _, kv, _ = gguf.read_gguf(path)
    assert kv["general.architecture"][1] == b"generic.gpu_index" and kv["split.vram_capacity"][1] == int(budget_gb * 1024 ** 3)
    with pytest.raises(ValueError):
        split.plan_split(hp, rates, base / 2 / 1024 ** 3, 64)


def test_rope_scaling_keys_of_a_model_file(tmp_path):
    """Linear RoPE scaling travels in the model file as the inverse of rope_freq_scale, under `rope.scaling.factor` or the
    older `rope.scale_linear`; scaling type "none" switches it off and other types are refused (llama.cpp:2316-2328, 9857-9871).
    That the reference's loader reads what write_model writes is shown by the compiled reference itself: the fixtures
    ref_*_scaled_shift.npz come from such files."""
    hp = synth.hparams("llama-tiny", n_layer=1, n_ctx=32, seed=3, rope_freq_scale=0.25)
    model = synth.make_model(hp)
    path = str(tmp_path / "m.powerinfer.gguf")
    gguf.write_model(path, model, {})
    _, kv, _ = gguf.read_gguf(path)
    assert kv["llama.rope.scaling.factor"][1] == 4.0 and kv["llama.rope.scaling.type"][1] == b"linear"
    assert gguf.read_model(path, n_ctx=32)[0].rope_freq_scale == 0.25
    hp1 = synth.hparams("llama-tiny", n_layer=1, n_ctx=32, seed=3)
    gguf.write_model(path, synth.make_model(hp1), {})
    _, kv, _ = gguf.read_gguf(path)
    assert "llama.rope.scaling.factor" not in kv
    assert gguf.read_model(path, n_ctx=32)[0].rope_freq_scale == 1.0
    for extra, want in (({"llama.rope.scale_linear": (gguf.T_F32, 2.0)}, 0.5),
                        ({"llama.rope.scaling.type": (gguf.T_STR, "none"), "llama.rope.scaling.factor": (gguf.T_F32, 2.0)}, 1.0)):
        gguf.write_model(path, synth.make_model(hp1), extra)
        assert gguf.read_model(path, n_ctx=32)[0].rope_freq_scale == want
    gguf.write_model(path, synth.make_model(hp1), {"llama.rope.scaling.type": (gguf.T_STR, "yarn")})
    with pytest.raises(ValueError):
        gguf.read_model(path, n_ctx=32)
