"""Bobevik on the CPU: limiting cases of the plain implementation's mechanisms (each checked against
a form that is obviously right), config.json in and out, what the architecture refuses, the cache
layout (pages for the attention layers, a state for the others), and the loader's tensor names."""

import math

import numpy as np
import pytest
import torch

import bobevik_cases as cases
import plain_bobevik as P
from mini_gpt_inference_amd.config.model_config import ConfigError, read_config_json
from mini_gpt_inference_amd.config.registry import architecture_of
from mini_gpt_inference_amd.models import bobevik
from mini_gpt_inference_amd.parts.base import KVNeed, StateNeed
from mini_gpt_inference_amd.parts.model import DecoderModel


def _rnd(g, *shape):
    return torch.randn(*shape, generator=g, dtype=P.DTYPE)


# ---------------------------------------------------------------- the plain mechanisms
def test_rotation_depends_on_the_distance_only_and_keeps_lengths():
    g = torch.Generator().manual_seed(0)
    q, k = _rnd(g, 1, 1, 12), _rnd(g, 1, 1, 12)
    scores = []
    for shift in (0, 5, 40):
        seq_q = torch.zeros(shift + 8, 1, 12, dtype=P.DTYPE)
        seq_k = torch.zeros(shift + 8, 1, 12, dtype=P.DTYPE)
        seq_q[shift + 7], seq_k[shift + 3] = q[0], k[0]
        rq, rk = P.rotate_half(seq_q, 8, 100.0, 2.0), P.rotate_half(seq_k, 8, 100.0, 2.0)
        scores.append(float((rq[shift + 7, 0] * rk[shift + 3, 0]).sum()))
        assert math.isclose(float(rq[shift + 7].norm()), float(q.norm()), rel_tol=1e-12)
        assert torch.equal(rq[shift + 7, 0, 8:], q[0, 0, 8:])          # channels beyond `dims` pass
    assert max(scores) - min(scores) < 1e-9
    # position 0 is not rotated; a factor of 2 halves every angle
    x = _rnd(g, 9, 2, 8)
    assert torch.allclose(P.rotate_half(x, 8, 50.0)[0], x[0])
    same_row = torch.cat([x[8:9]] * 9)
    assert torch.allclose(P.rotate_half(same_row, 8, 50.0, 2.0)[8], P.rotate_half(same_row, 8, 50.0)[4])


def test_decaying_state_is_a_weighted_sum_over_the_past():
    g = torch.Generator().manual_seed(1)
    T, H, D, E = 9, 2, 4, 3
    q, k, v = _rnd(g, T, H, D), _rnd(g, T, H, D), _rnd(g, T, H, E)
    decay = [0.8, 1.0]
    got = P.decaying_state(q, k, v, decay)
    for a in range(H):
        for t in range(T):
            want = sum(decay[a] ** (t - s) * float(q[t, a] @ k[s, a]) * v[s, a] for s in range(t + 1))
            assert torch.allclose(got[t, a], want, atol=1e-12)


def test_grouped_attention_equals_attention_with_repeated_heads_and_the_cap_bounds_scores():
    g = torch.Generator().manual_seed(2)
    T, H, G, D, E = 11, 4, 2, 6, 5
    q, k, v = _rnd(g, T, H, D), _rnd(g, T, G, D), _rnd(g, T, G, E)
    grouped = P.causal_softmax_attention(q, k, v, 0.3)
    full = P.causal_softmax_attention(q, k.repeat_interleave(2, dim=1), v.repeat_interleave(2, dim=1), 0.3)
    assert torch.allclose(grouped, full, atol=1e-12)
    assert torch.allclose(grouped[0], v[0].repeat_interleave(2, dim=0))       # the first token sees itself only
    # a tiny cap makes every score nearly equal: the output is nearly the running mean of the values
    capped = P.causal_softmax_attention(q, k, v, 0.3, softcap=1e-6)
    means = torch.cumsum(v, 0) / torch.arange(1, T + 1, dtype=P.DTYPE)[:, None, None]
    assert torch.allclose(capped, means.repeat_interleave(2, dim=1), atol=1e-5)


def test_norms():
    g = torch.Generator().manual_seed(3)
    x = _rnd(g, 4, 10)
    unit = P.unit_rms(x, 0.0)
    assert torch.allclose((unit * unit).mean(-1), torch.ones(4, dtype=P.DTYPE))
    gain = _rnd(g, 10)
    assert torch.allclose(P.rms_norm(x, gain, 1e-5, True), P.rms_norm(x, gain + 1.0, 1e-5, False))
    assert torch.allclose(P.unit_rms(torch.zeros(1, 4, dtype=P.DTYPE), 0.25), torch.zeros(1, 4, dtype=P.DTYPE))


def test_what_the_test_models_are_sensitive_to(tmp_path):
    """Changing the value-mixing weight, a decay, the cap, the scaling of positions, a gate, a norm
    behind a sublayer or the residual multiplier moves the logits by far more than the tolerances."""
    folder = cases.write_model(str(tmp_path / "A"), "A")
    cfg, w = P.read_model_folder(folder)
    ids = list(np.random.default_rng(0).integers(0, cfg["vocab"], 60))
    base = P.forward(cfg, w, ids)

    def moved(cfg2=None, w2=None):
        return float((P.forward(cfg2 or cfg, w2 or w, ids) - base).abs().max())

    def with_mixer(i, change):
        layers = [dict(l) for l in cfg["layers"]]
        layers[i] = {**layers[i], "mixer": change(layers[i]["mixer"])}
        return {**cfg, "layers": layers}

    assert moved(w2={**w, "l4.mix.vmix": w["l4.mix.vmix"] + 0.5}) > 0.05
    assert moved(w2={**w, "l2.mix.vmix": w["l2.mix.vmix"] + 0.5}) == 0.0            # the first such layer's is unused
    assert moved(with_mixer(1, lambda m: {**m, "decay": [0.5, 0.999]})) > 0.05
    assert moved(with_mixer(0, lambda m: {**m, "left": {**m["left"], "softcap": 40.0}})) > 0.01
    assert moved(with_mixer(0, lambda m: {**m, "left": {**m["left"], "rot": {"dims": 8, "base": 1000.0}}})) > 0.01
    assert moved(with_mixer(0, lambda m: {**m, "right": {**m["right"], "decay": [0.9, 0.9]}})) > 0.01
    assert moved(w2={**w, "l2.mix.g": w["l2.mix.g"] * 0.0}) > 0.05
    assert moved(w2={**w, "l1.norm1b": w["l1.norm1b"] + 0.5}) > 0.05
    assert moved({**cfg, "residual_mult": 1.0}) > 0.05
    assert moved(w2={**w, "l0.mix.left.out": w["l0.mix.left.out"] * 2.0}) > 0.01
    assert moved(w2={**w, "l0.mix.left.k.b": w["l0.mix.left.k.b"] + 1.0}) > 0.001


# ---------------------------------------------------------------- configuration
@pytest.mark.parametrize("name", sorted(cases.RAW))
def test_config_round_trip(name, tmp_path):
    cfg = cases.config(name)
    assert bobevik.config_from_json(bobevik.config_to_json(cfg)) == cfg
    folder = cases.write_model(str(tmp_path / name), name)
    raw = read_config_json(folder)
    assert architecture_of(raw).name == "Bobevik" and bobevik.config_from_json(raw) == cfg


def test_random_configurations_are_accepted_and_round_trip():
    rng = np.random.default_rng(4)
    for _ in range(30):
        raw = cases.random_raw(rng)
        cfg = bobevik.config_from_json(raw)
        assert bobevik.config_from_json(bobevik.config_to_json(cfg)) == cfg
        DecoderModel(bobevik.model_spec(cfg))


def _edited(name, edit):
    import copy
    raw = copy.deepcopy(cases.RAW[name])
    edit(raw)
    return raw


@pytest.mark.parametrize("edit", [
    lambda r: r["layers"][0].update(type="convolution"),
    lambda r: r["layers"][1]["mixer"].update(decay=[0.9]),
    lambda r: r["layers"][2]["mixer"].update(kv_heads=3),
    lambda r: r["layers"][2]["mixer"]["rot"].update(dims=7),
    lambda r: r["layers"][2]["mixer"]["rot"].update(dims=64),
    lambda r: r["layers"][0]["mixer"]["left"].update(softcap=0.0),
    lambda r: r["layers"][4]["mixer"].update(vdim=32),
    lambda r: r["layers"][0]["mlp"].update(kind="moe"),
    lambda r: r.update(layers=[]),
    lambda r: r.update(width=0),
])
def test_refusals(edit):
    with pytest.raises(ConfigError):
        bobevik.config_from_json(_edited("A", edit))


# ---------------------------------------------------------------- model as data
def test_cache_layout_and_tensor_names():
    model = DecoderModel(bobevik.model_spec(cases.config("A")))
    layout = model.cache_layout
    # attention layers (and the left halves) keep pages of max(dim, vdim) rounded up to 32 channels
    # a head, the others a float32 state of heads * dim * vdim
    assert [(g.n_kv_head, g.head_dim, g.n_pools) for g in layout.groups] == [(2, 32, 1), (1, 32, 2)]
    assert layout.state_numels == [2 * 16 * 24, 2 * 32 * 16, 3 * 8 * 40]
    kinds = [{role: b.kind for role, b in run.items()} for run in layout.run_bindings]
    assert kinds == [{"mixer0": "kv", "mixer1": "state"}, {"mixer": "state"}, {"mixer": "kv"}, {"mixer": "state"},
                     {"mixer": "kv"}]
    needs = [p.cache_need() for layer in model.layers for r, p in layer.parts.items() if r.startswith("mixer")]
    assert sum(isinstance(n, KVNeed) for n in needs) == 3 and sum(isinstance(n, StateNeed) for n in needs) == 3
    wanted = model.weight_requests()
    plan_names = {name: tuple(shape) for name, shape, _, _ in bobevik.init_plan(cases.config("A"))}
    assert {n: tuple(r.shape) for n, r in wanted.items()} == plan_names
    assert wanted["l2.mix.vmix"].shape == () and "l0.mix.left.q.b" in wanted and "l2.norm2" not in wanted
    assert "l0.mix.right.norm" in wanted and "l0.mix.left.out" in wanted and "embed.norm" in wanted
    # the first layer that mixes values keeps them, the later ones mix
    assert [model.layers[i].parts["mixer"].value_mix for i in (2, 4)] == ["keep", "mix"]
    assert model.graph_safe and model.plan_safe
