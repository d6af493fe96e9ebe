"""Small Bobevik configurations and model folders with random weights for the tests.

The configurations differ from each other in every size and option: the order of the layer types,
widths that are and are not multiples of 16, one head and several, grouped and ungrouped key/value
heads, query/key sizes below, at and above the value size, rotations over part of a head and over
all of it, with and without scaled positions and capped scores, no layer, one or several layers
that mix values, decays from fast to nearly one, layers without a feed-forward, a residual
multiplier of one and others."""

from __future__ import annotations

import os
from typing import Callable, Dict, Optional

import torch
from safetensors.torch import save_file

from mini_gpt_inference_amd.config.model_config import write_config_json
from mini_gpt_inference_amd.models import bobevik
from mini_gpt_inference_amd.weights.random_init import random_tensors


def _rot(dims, base, factor=None):
    rot = {"dims": dims, "base": base}
    if factor is not None:
        rot["scaling"] = {"factor": factor}
    return rot


def attention(heads, kv_heads, dim, vdim, scale, rot=None, softcap=None, v_mix=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if rot is not None:
        m["rot"] = rot
    if softcap is not None:
        m["softcap"] = softcap
    if v_mix is not None:
        m["v_mix"] = v_mix
    return m


def state(heads, dim, vdim, decay, rot=None):
    m = {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay)}
    if rot is not None:
        m["rot"] = rot
    return m


def layer(kind, mixer, ff):
    return {"type": kind, "mixer": mixer, "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


RAW: Dict[str, dict] = {
    # every layer type, two layers that mix values (the first keeps, the second mixes) with different
    # query sizes, a layer without a feed-forward, grouped heads, rotation over half a head
    "A": {"architecture": "Bobevik", "vocab": 131, "width": 64, "norm": {"eps": 1e-5}, "residual_mult": 0.5,
          "layers": [
              layer("parallel", {"left": attention(4, 2, 16, 32, 0.25, _rot(8, 1000.0, 2.0), softcap=4.0),
                                 "right": state(2, 16, 24, [0.9, 0.5])}, 48),
              layer("retention", state(2, 32, 16, [0.97, 0.999], _rot(32, 10000.0)), 80),
              layer("attention", attention(4, 1, 24, 16, 0.2, _rot(12, 500.0), v_mix=True), None),
              layer("retention", state(3, 8, 40, [0.5, 0.8, 0.99], _rot(4, 100.0)), 32),
              layer("attention", attention(2, 1, 8, 16, 0.35, _rot(8, 10000.0), v_mix=True), 56)]},
    # head sizes that the bfloat16 matrix-core attention kernels take (64 both ways), one head, as many
    # key/value heads as heads, a retention layer first, no value mixing, multiplier one, a wider state
    "B": {"architecture": "Bobevik", "vocab": 77, "width": 96, "norm": {"eps": 1e-6}, "residual_mult": 1.0,
          "layers": [
              layer("retention", state(1, 64, 64, [0.99951171875], _rot(64, 1e6)), 64),
              layer("attention", attention(2, 2, 64, 64, 0.125, _rot(64, 10000.0)), 128),
              layer("parallel", {"left": attention(1, 1, 64, 32, 0.125, _rot(32, 50000.0, 4.0), softcap=30.0),
                                 "right": state(1, 128, 128, [0.95])}, None),
              layer("attention", attention(3, 1, 32, 64, 0.2, _rot(16, 1000.0), v_mix=False), 40)]},
    # a width and head sizes that only the general kernels take, one layer that says v_mix (it keeps its
    # values for nobody), three that do, values wider than queries, a cap that bites
    "C": {"architecture": "Bobevik", "vocab": 59, "width": 40, "norm": {"eps": 1e-4}, "residual_mult": 0.7,
          "layers": [
              layer("attention", attention(2, 2, 12, 20, 0.5, _rot(6, 200.0), v_mix=True), 24),
              layer("parallel", {"left": attention(3, 1, 20, 12, 0.6, _rot(20, 300.0, 1.5), softcap=1.5),
                                 "right": state(3, 12, 20, [0.6, 0.7, 0.999])}, 72),
              layer("attention", attention(4, 2, 20, 20, 0.3, _rot(20, 50.0), v_mix=True), None),
              layer("attention", attention(2, 2, 36, 20, 0.2, _rot(2, 10.0), v_mix=True), 24)]},
    # a single value-mixing layer among plain ones
    "D": {"architecture": "Bobevik", "vocab": 33, "width": 32, "norm": {"eps": 1e-5}, "residual_mult": 0.3,
          "layers": [
              layer("attention", attention(2, 1, 16, 16, 0.25, _rot(16, 10000.0), v_mix=True), 32),
              layer("retention", state(2, 16, 16, [0.9, 0.99], _rot(8, 10000.0)), None)]},
}
SEEDS = {"A": 11, "B": 12, "C": 13, "D": 14}
STD_SCALE = 1.5


def config(name: str):
    return bobevik.config_from_json(RAW[name])


def write_raw_model(path: str, raw: dict, seed: int, std_scale: float = STD_SCALE,
                    edit: Optional[Callable[[Dict[str, torch.Tensor]], None]] = None) -> str:
    cfg = bobevik.config_from_json(raw)
    tensors = random_tensors(cfg, seed, torch.bfloat16, std_scale)
    if edit is not None:
        edit(tensors)
    os.makedirs(path, exist_ok=True)
    write_config_json(path, cfg)
    save_file({k: v.contiguous() for k, v in tensors.items()}, os.path.join(path, "model.safetensors"))
    return path


def write_model(path: str, name: str, edit: Optional[Callable[[Dict[str, torch.Tensor]], None]] = None) -> str:
    return write_raw_model(path, RAW[name], SEEDS[name], edit=edit)


def random_raw(rng) -> dict:
    """A random config.json: two to six layers of random types, widths, head counts and sizes (also no
    multiples of 8), rotations over 2 channels to the whole head, scaled or not, caps, decays, value
    mixing on some attention layers (their key/value heads and value size then agree), feed-forwards
    or none."""
    width = int(rng.choice([24, 40, 64, 72, 96, 136, 256]))
    mix_heads, mix_vdim = int(rng.integers(1, 3)), int(rng.choice([8, 12, 16, 32, 64]))

    def rot(dim):
        dims = int(rng.choice([d for d in (2, 4, 8, 12, 16, 32, 64, dim - dim % 2) if 0 < d <= dim]))
        return _rot(dims, float(rng.choice([10.0, 1000.0, 50000.0, 1e6])),
                    float(rng.choice([2.0, 4.0])) if rng.random() < 0.4 else None)

    def att(softcap, may_mix):
        dim, vdim = int(rng.choice([8, 12, 16, 24, 32, 48, 64, 128])), int(rng.choice([8, 16, 20, 32, 64]))
        kv = int(rng.integers(1, 4))
        heads = kv * int(rng.integers(1, 4))
        mix = may_mix and rng.random() < 0.6
        if mix:
            kv, vdim = mix_heads, mix_vdim
            heads = kv * int(rng.integers(1, 4))
        return attention(heads, kv, dim, vdim, float(rng.choice([0.1, 0.3, dim ** -0.5])), rot(dim),
                         softcap=float(rng.choice([2.0, 10.0, 30.0])) if softcap else None,
                         v_mix=True if mix else (False if rng.random() < 0.3 else None))

    def sta(with_rot):
        heads, dim = int(rng.integers(1, 4)), int(rng.choice([8, 12, 16, 32, 64, 128]))
        decay = [float(rng.choice([0.5, 0.6065, 0.9, 0.96875, 0.999, 0.99951171875])) for _ in range(heads)]
        return state(heads, dim, int(rng.choice([8, 16, 24, 32, 64, 128])), decay, rot(dim) if with_rot else None)

    layers = []
    for _ in range(int(rng.integers(2, 7))):
        kind = str(rng.choice(["retention", "attention", "parallel"]))
        if kind == "retention":
            mixer = sta(True)
        elif kind == "attention":
            mixer = att(False, True)
        else:
            mixer = {"left": att(True, False), "right": sta(False)}
        layers.append(layer(kind, mixer, int(rng.choice([24, 40, 100, 128])) if rng.random() < 0.8 else None))
    return {"architecture": "Bobevik", "vocab": int(rng.choice([50, 131, 300, 577])), "width": width,
            "norm": {"eps": float(rng.choice([1e-6, 1e-5]))}, "residual_mult": float(rng.choice([0.25, 0.7, 1.0])),
            "layers": layers}
