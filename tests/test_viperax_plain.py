"""Viperax on the CPU: the plain implementation's mechanisms against their limiting cases, the
configuration's way in and out of config.json, the cache layout of layers that share latents, and
the loader's names and shapes."""

import json
import os

import pytest
import torch

import plain_viperax as V
import viperax_cases as cases
from mini_gpt_inference_amd.config.model_config import ConfigError, read_config_json
from mini_gpt_inference_amd.config.registry import architecture_of
from mini_gpt_inference_amd.models import viperax
from mini_gpt_inference_amd.parts.model import DecoderModel
from mini_gpt_inference_amd.weights.loader import load_tensors


def test_sink_attention_limits():
    g = torch.Generator().manual_seed(0)
    q, k, v = (torch.randn(12, 2, 8, generator=g) for _ in range(3))
    # a sink far below every score changes nothing; a window as long as the sequence is no window
    plain = V.sink_attention(q, k, v, None, 0.4, 0)
    assert torch.allclose(V.sink_attention(q, k, v, torch.tensor([-80.0, -80.0]), 0.4, 12), plain, atol=1e-6)
    # a sink takes weight away: the output is the ordinary one times (1 - the sink's share)
    sunk = V.sink_attention(q, k, v, torch.tensor([0.5, 2.0]), 0.4, 0)
    for i in range(12):
        for a, s in enumerate((0.5, 2.0)):
            scores = (k[:i + 1, a] @ q[i, a]) * 0.4
            share = torch.exp(torch.tensor(s)) / (torch.exp(scores).sum() + torch.exp(torch.tensor(s)))
            assert torch.allclose(sunk[i, a], plain[i, a] * (1 - share), atol=1e-5)
    # window 1: a query sees itself only, so its output is its own value times (1 - share)
    one = V.sink_attention(q, k, v, None, 0.4, 1)
    assert torch.allclose(one, v, atol=1e-6)
    # window w: key i - w is out, key i - w + 1 is in
    k2, v2 = k.clone(), v.clone()
    k2[3], v2[3] = 50.0 * q[8] / q[8].norm(), 7.0
    assert (V.sink_attention(q, k2, v2, None, 0.4, 6)[8] - 7.0).abs().max() < 1e-3      # 8 - 3 < 6
    assert (V.sink_attention(q, k2, v2, None, 0.4, 5)[8] - 7.0).abs().min() > 1.0       # 8 - 3 = 5: out


def test_hyper_connections_with_one_stream_are_the_plain_residual():
    x = torch.randn(1, 5, 6)
    y = torch.randn(5, 6)
    assert torch.equal(V.hyper_read(x, torch.ones(1)), x[0])
    assert torch.allclose(V.hyper_write(x, torch.ones(1, 1), torch.ones(1), y), (x[0] + y)[None])
    # the mixing matrix is indexed [from, to]
    x3 = torch.randn(3, 2, 4)
    mix = torch.zeros(3, 3)
    mix[0, 2] = 1.0
    out = V.hyper_write(x3, mix, torch.zeros(3), torch.zeros(2, 4))
    assert torch.equal(out[2], x3[0]) and out[:2].abs().max() == 0


def test_table_experts_weights_and_shared():
    g = torch.Generator().manual_seed(1)
    h = torch.randn(4, 6, generator=g)
    experts = [tuple(torch.randn(*s, generator=g) for s in ((5, 6), (5, 6), (6, 5))) for _ in range(3)]
    shared = tuple(torch.randn(*s, generator=g) for s in ((3, 6), (3, 6), (6, 3)))
    table = torch.tensor([[0, 2], [1, 0], [2, 1]])
    out = V.table_moe(h, [1, 1, 0, 2], table, experts, shared)
    want0 = (V.gated_mlp(h[:1], *experts[1]) + V.gated_mlp(h[:1], *experts[0])) / 2 + V.gated_mlp(h[:1], *shared)
    assert torch.allclose(out[:1], want0, atol=1e-5)


@pytest.mark.parametrize("name", sorted(cases.RAW))
def test_config_goes_through_config_json_unchanged(name, tmp_path):
    cfg = cases.config(name)
    again = viperax.config_from_json(json.loads(json.dumps(viperax.config_to_json(cfg))))
    assert again == cfg
    spec = viperax.model_spec(cfg)
    assert spec.streams == (cfg.streams or 1) and len(spec.layers) == len(cfg.layers)


def test_config_refuses_what_the_design_does_not_have():
    raw = json.loads(json.dumps(cases.RAW["Q"]))
    raw["layers"][2]["mixer"]["kv_from"] = 2
    with pytest.raises(ConfigError):
        viperax.config_from_json(raw)
    raw = json.loads(json.dumps(cases.RAW["Q"]))
    raw["layers"][2]["mixer"]["kv_rank"] = 16       # not the size of the latents it would read
    with pytest.raises(ConfigError):
        viperax.config_from_json(raw)
    raw = json.loads(json.dumps(cases.RAW["Q"]))
    raw["layers"][0]["type"] = "something_else"
    with pytest.raises(ConfigError):
        viperax.config_from_json(raw)


def test_pages_keep_the_widest_window_among_the_layers_that_read_them():
    model = DecoderModel(viperax.model_spec(cases.config("P")))
    layout = model.cache_layout
    # layer 0's latents are read by layer 3 without a mask: kept whole; layer 1's by layer 2 through 33
    assert sorted((g.window, g.n_pools, g.joint, g.head_dim) for g in layout.groups) == [(0, 1, True, 32), (33, 1, True, 32)]
    b = [next(iter(x.values())) for x in layout.run_bindings]
    assert [x.writes for x in b] == [True, True, False, False]
    assert (b[2].group, b[2].index) == (b[1].group, b[1].index) and (b[3].group, b[3].index) == (b[0].group, b[0].index)
    # a reader with a shorter window than the writer's leaves the writer's window in force
    model = DecoderModel(viperax.model_spec(cases.config("S")))
    assert [(g.window, g.n_pools) for g in model.cache_layout.groups] == [(70, 1)]


@pytest.mark.parametrize("name", sorted(cases.RAW))
def test_loader_finds_every_tensor_and_the_joined_matrices_are_the_loaded_ones(name, tmp_path):
    folder = cases.write_model(str(tmp_path / name), name)
    raw = read_config_json(folder)
    arch = architecture_of(raw)
    model = DecoderModel(arch.model_spec(arch.config_from_json(raw)))
    tensors = load_tensors(folder, model.weight_requests(), torch.float32, torch.device("cpu"))
    model.bind(tensors)
    _, plain = V.read_model_folder(folder)
    for i, layer in enumerate(model.layers):
        mixer = layer.parts["mixer"]
        assert torch.equal(mixer.in_weight[:mixer.q_width], plain[f"l{i}.mix.q"])
        h, d, r = mixer.n_head, mixer.head_dim, mixer.rank
        assert torch.equal(mixer.uk_folded.transpose(1, 2).reshape(h * d, r), plain[f"l{i}.mix.uk"])
        ff = layer.parts.get("feed_forward")
        if ff is not None and hasattr(ff, "in_weights"):
            assert ff.table.dtype == torch.int32
            assert torch.equal(ff.in_weights[1, ff.hidden:], plain[f"l{i}.mlp.e1.up"])
            assert torch.equal(ff.down_weights[0], plain[f"l{i}.mlp.e0.down"])
    cost = model.cost()
    assert cost.run_matrix_elements > 0 and all(run.tensors == 1 for run in cost.kv_runs)


def test_a_missing_tensor_is_named(tmp_path):
    from mini_gpt_inference_amd.weights.loader import WeightError

    folder = cases.write_model(str(tmp_path / "Q"), "Q", edit=lambda t: t.pop("l1.mix.sink"))
    raw = read_config_json(folder)
    arch = architecture_of(raw)
    model = DecoderModel(arch.model_spec(arch.config_from_json(raw)))
    with pytest.raises(WeightError, match="l1.mix.sink"):
        load_tensors(folder, model.weight_requests(), torch.float32, torch.device("cpu"))


def test_plain_forward_does_not_look_ahead(tmp_path):
    folder = cases.write_model(str(tmp_path / "P"), "P")
    cfg, w = V.read_model_folder(folder)
    ids = [5, 9, 100, 3, 77, 41, 12, 8, 8, 130, 2, 64]
    whole, layers = V.forward(cfg, w, ids)
    assert layers.shape == (len(cfg["layers"]), len(ids), cfg["width"])
    assert torch.allclose(V.forward(cfg, w, ids[:7])[0], whole[:7], atol=1e-5)
    assert float(whole.abs().max()) <= cfg["logit_softcap"]
    # without the key there is no cap
    loose = {k: v for k, v in cfg.items() if k != "logit_softcap"}
    assert torch.allclose(torch.tanh(V.forward(loose, w, ids)[0] / 10.0) * 10.0, whole, atol=1e-5)
