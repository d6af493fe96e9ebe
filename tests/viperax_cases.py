"""Small Viperax configurations and model folders with random weights for the tests.

The configurations differ from each other in every size and option: streams (several, one, none),
heads (also one), query/key size against value size, latent sizes that the bfloat16 tile kernel
takes (32, 64) and that it does not (40, 24), windows (none, 1, a few tokens, longer than the
prompts), layers that read another layer's latents through a longer or a shorter window than the
layer that writes them, feed-forwards (none, dense, experts with top 1 and 2, with and without a
shared expert), logit scale and cap."""

from __future__ import annotations

import os
from typing import Callable, Dict, Optional

import torch
from safetensors.torch import save_file

from mini_gpt_inference_amd.config.model_config import write_config_json
from mini_gpt_inference_amd.models import viperax
from mini_gpt_inference_amd.weights.random_init import random_tensors


def _mixer(heads, dim, vdim, rank, scale, window=None, kv_from=None):
    m = {"heads": heads, "dim": dim, "vdim": vdim, "kv_rank": rank, "scale": scale}
    if window is not None:
        m["mask"] = {"size": window}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return m


def _layer(mixer, mlp):
    return {"type": "latent_attention", "mixer": mixer, "mlp": mlp}


def _moe(ff, experts, top, shared=None):
    mlp = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if shared:
        mlp["shared"] = {"ff": shared}
    return mlp


RAW: Dict[str, dict] = {
    # several streams; a layer that reads layer 1's latents through a longer window than layer 1's own,
    # one without a feed-forward, one that reads layer 0's without any mask
    "P": {"architecture": "Viperax", "vocab": 131, "width": 64, "streams": 2, "norm": {"eps": 1e-5},
          "embedding": {"scale": 8.0}, "logit_scale": 0.5, "logit_softcap": 10.0,
          "layers": [_layer(_mixer(2, 16, 32, 32, 0.3, window=9), {"kind": "dense", "ff": 48}),
                     _layer(_mixer(2, 16, 32, 32, 0.3, window=20), _moe(32, 5, 2, shared=40)),
                     _layer(_mixer(4, 8, 16, 32, 0.4, window=33, kv_from=1), None),
                     _layer(_mixer(2, 16, 32, 32, 0.3, kv_from=0), _moe(16, 3, 1))]},
    # one stream with hyper-connection tensors, one head, top 1 of 2, a window of one token, a latent
    # size (40) that only the split and the general kernels take, no cap on the logits
    "Q": {"architecture": "Viperax", "vocab": 77, "width": 48, "streams": 1, "norm": {"eps": 1e-6},
          "embedding": {"scale": 1.0}, "logit_scale": 2.0,
          "layers": [_layer(_mixer(1, 24, 8, 40, 0.2, window=1), _moe(32, 2, 1)),
                     _layer(_mixer(3, 8, 24, 40, 0.35, window=5), {"kind": "dense", "ff": 20}),
                     _layer(_mixer(1, 24, 8, 40, 0.2, window=3, kv_from=1), {"kind": "dense", "ff": 36})]},
    # no hyper-connections at all (no `streams` key: the plain pre-norm residual), no masks on the
    # first two layers, a latent of 64; top 3 of 4 with a shared expert; a last layer without a
    # feed-forward whose latent (320) is beyond what the bfloat16 attention kernels take
    "R": {"architecture": "Viperax", "vocab": 203, "width": 96, "norm": {"eps": 1e-4},
          "embedding": {"scale": 3.0}, "logit_scale": 1.0, "logit_softcap": 30.0,
          "layers": [_layer(_mixer(3, 32, 16, 64, 0.18), _moe(40, 4, 3, shared=24)),
                     _layer(_mixer(2, 16, 48, 64, 0.25, kv_from=0), {"kind": "dense", "ff": 112}),
                     _layer(_mixer(1, 40, 8, 320, 0.2, window=11), None)]},
    # three streams, a latent of 24 (the general kernel only), windows longer than most prompts
    "S": {"architecture": "Viperax", "vocab": 59, "width": 40, "streams": 3, "norm": {"eps": 1e-5},
          "embedding": {"scale": 6.0}, "logit_scale": 0.25, "logit_softcap": 5.0,
          "layers": [_layer(_mixer(2, 12, 20, 24, 0.3, window=70), {"kind": "dense", "ff": 56}),
                     _layer(_mixer(2, 12, 20, 24, 0.3, window=4, kv_from=0), _moe(8, 6, 2))]},
}
SEEDS = {"P": 3, "Q": 4, "R": 5, "S": 6}
STD_SCALE = {"P": 1.5, "Q": 1.5, "R": 1.5, "S": 1.5}


def config(name: str):
    return viperax.config_from_json(RAW[name])


def write_model(path: str, name: str, edit: Optional[Callable[[Dict[str, torch.Tensor]], None]] = None) -> str:
    cfg = config(name)
    tensors = random_tensors(cfg, SEEDS[name], torch.bfloat16, STD_SCALE[name])
    # sinks large enough to matter: a kernel that leaves one out, or counts it twice, shows
    for key in tensors:
        if key.endswith(".sink"):
            tensors[key] = (tensors[key].float() * 2.0 + 1.0).to(torch.bfloat16)
    if edit is not None:
        edit(tensors)
    os.makedirs(path, exist_ok=True)
    write_config_json(path, cfg)
    save_file({k: v.contiguous() for k, v in tensors.items()}, os.path.join(path, "model.safetensors"))
    return path


def random_raw(rng) -> dict:
    """A random config.json: widths, layer counts, streams (none to 4), heads 1 to 5, query/key and
    value sizes that are no multiples of 16, latents from 16 to 160 (some layers reading an earlier
    layer's of the same size), windows from 1 to longer than the prompts or none, every kind of
    feed-forward or none."""
    width = int(rng.choice([40, 64, 72, 96, 136, 200, 256]))
    streams = rng.choice([None, 1, 2, 3, 4])
    rank_all = int(rng.choice([16, 24, 40, 48, 64, 80, 96, 128, 160]))
    layers, own = [], []
    for i in range(int(rng.integers(2, 6))):
        dim = int(rng.choice([8, 12, 16, 24, 32, 40, 64]))
        rank = rank_all if rng.random() < 0.7 else int(rng.choice([16, 32, 56]))
        mixer = _mixer(int(rng.integers(1, 6)), dim, int(rng.choice([8, 16, 20, 32, 48])), rank,
                       float(rng.choice([0.1, 0.25, dim ** -0.5])),
                       window=int(rng.choice([1, 2, 7, 16, 17, 33, 64, 100])) if rng.random() < 0.8 else None)
        sources = [j for j in own if layers[j]["mixer"]["kv_rank"] == rank]
        if sources and rng.random() < 0.5:
            mixer["kv_from"] = int(rng.choice(sources))
        else:
            own.append(i)
        kind = rng.choice(["none", "dense", "moe"])
        if kind == "none":
            mlp = None
        elif kind == "dense":
            mlp = {"kind": "dense", "ff": int(rng.choice([24, 40, 100, 128]))}
        else:
            experts = int(rng.integers(2, 10))
            mlp = _moe(int(rng.choice([8, 24, 32, 48])), experts, int(rng.integers(1, min(experts, 3) + 1)),
                       shared=int(rng.choice([16, 40, 64])) if rng.random() < 0.5 else None)
        layers.append(_layer(mixer, mlp))
    raw = {"architecture": "Viperax", "vocab": int(rng.choice([50, 131, 300, 577])), "width": width,
           "norm": {"eps": float(rng.choice([1e-6, 1e-5]))},
           "embedding": {"scale": float(rng.choice([1.0, 4.0, width ** 0.5]))},
           "logit_scale": float(rng.choice([0.25, 1.0])), "layers": layers}
    if streams is not None:
        raw["streams"] = int(streams)
    if rng.random() < 0.7:
        raw["logit_softcap"] = float(rng.choice([5.0, 15.0, 30.0]))
    return raw


def write_raw_model(path: str, raw: dict, seed: int, std_scale: float = 1.5) -> str:
    cfg = viperax.config_from_json(raw)
    tensors = random_tensors(cfg, seed, torch.bfloat16, std_scale)
    for key in tensors:
        if key.endswith(".sink"):
            tensors[key] = (tensors[key].float() * 2.0 + 1.0).to(torch.bfloat16)
    os.makedirs(path, exist_ok=True)
    write_config_json(path, cfg)
    save_file({k: v.contiguous() for k, v in tensors.items()}, os.path.join(path, "model.safetensors"))
    return path
