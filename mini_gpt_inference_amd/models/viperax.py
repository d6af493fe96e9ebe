"""Viperax: a decoder whose layers are listed one by one in config.json, as data.

What the design fixes, and is therefore set here and handed to the parts as parameters:
- pre-norm layers whose norms are LayerNorms with a gain and no bias, one eps for all of them
  (config `norm.eps`), which is also the eps of the latent's RMS norm;
- the token embedding times `embedding.scale`, no position signal anywhere;
- `streams` residual streams joined by hyper-connections (per sublayer a read vector, a mixing
  matrix indexed [from, to] and a write vector); without the key, one plain residual;
- the mixer `latent_attention`: heads with query/key size `dim` and value size `vdim`, a latent of
  `kv_rank` that is all the cache keeps, a sliding window `mask.size` (a query sees itself and the
  mask.size - 1 positions before it; no mask: all earlier positions), a sink per head in the
  softmax's denominator, a sigmoid output gate; with `kv_from: j` the layer has no latent of its
  own and reads layer j's;
- feed-forwards: none (`mlp: null`), `dense` (a gated unit with silu) or `moe` (experts chosen by
  an integer table row per token id, each weighted 1 / top, plus an optional shared expert);
- the head: final LayerNorm, logits times `logit_scale`, then `logit_softcap` * tanh(. / cap).

Tensor names: `embed`, `l<i>.norm1|norm2`, `l<i>.mix.{q,dkv,dkv.norm,uk,uv,sink,g,o}`,
`l<i>.mlp.{gate,up,down}` or `l<i>.mlp.{table, e<k>.gate|up|down, shared.gate|up|down}`,
`l<i>.hc1|hc2.{in,out,mix}`, `final.norm`, `head`; linear weights are stored [out, in].
"""

from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Any, Dict, List, Mapping, Optional, Tuple

from ..config.model_config import ConfigError
from ..config.registry import Architecture, register_architecture
from ..parts.base import PartSpec
from ..parts.model import LayerRun, LayerSpec, ModelSpec

NAME = "Viperax"


@dataclass(frozen=True)
class LatentMixerConfig:
    heads: int
    dim: int
    vdim: int
    kv_rank: int
    scale: float
    window: int                 # 0: no mask entry, every earlier position is seen
    kv_from: Optional[int]      # the layer whose latents this one reads, or None


@dataclass(frozen=True)
class FeedForwardConfig:
    kind: str                   # "dense" or "moe"
    ff: int                     # hidden size (of one expert, for "moe")
    experts: int = 0
    top: int = 0
    shared_ff: int = 0          # 0: no shared expert


@dataclass(frozen=True)
class LayerConfig:
    mixer: LatentMixerConfig
    mlp: Optional[FeedForwardConfig]


@dataclass(frozen=True)
class ViperaxConfig:
    architecture: str
    vocab: int
    width: int
    layers: Tuple[LayerConfig, ...]
    norm_eps: float
    embedding_scale: float = 1.0
    streams: Optional[int] = None       # None: one plain residual, no hyper-connection tensors
    logit_scale: float = 1.0
    logit_softcap: float = 0.0          # 0: no cap


def _positive(name: str, value: Any) -> int:
    if not isinstance(value, int) or isinstance(value, bool) or value <= 0:
        raise ConfigError(f"{name} must be a positive integer, got {value!r}")
    return value


def _mixer_from_json(i: int, layer: Mapping[str, Any], n_before: List[LayerConfig]) -> LatentMixerConfig:
    if layer.get("type") != "latent_attention":
        raise ConfigError(f"layer {i}: unknown mixer type {layer.get('type')!r}")
    m = layer.get("mixer")
    if not isinstance(m, Mapping):
        raise ConfigError(f"layer {i}: no mixer sizes")
    mask = m.get("mask")
    window = _positive(f"layer {i} mask.size", mask.get("size")) if mask else 0
    kv_from = m.get("kv_from")
    cfg = LatentMixerConfig(_positive(f"layer {i} heads", m.get("heads")), _positive(f"layer {i} dim", m.get("dim")),
                            _positive(f"layer {i} vdim", m.get("vdim")),
                            _positive(f"layer {i} kv_rank", m.get("kv_rank")), float(m["scale"]), window,
                            None if kv_from is None else int(kv_from))
    if cfg.kv_from is not None:
        if not 0 <= cfg.kv_from < i:
            raise ConfigError(f"layer {i}: kv_from must name an earlier layer, got {cfg.kv_from}")
        src = n_before[cfg.kv_from].mixer
        if src.kv_from is not None or src.kv_rank != cfg.kv_rank:
            raise ConfigError(f"layer {i}: layer {cfg.kv_from} has no latents of size {cfg.kv_rank} of its own")
    return cfg


def _mlp_from_json(i: int, mlp: Optional[Mapping[str, Any]]) -> Optional[FeedForwardConfig]:
    if mlp is None:
        return None
    kind = mlp.get("kind")
    if kind == "dense":
        return FeedForwardConfig("dense", _positive(f"layer {i} mlp.ff", mlp.get("ff")))
    if kind == "moe":
        router, shared = mlp.get("router") or {}, mlp.get("shared")
        cfg = FeedForwardConfig("moe", _positive(f"layer {i} mlp.expert.ff", (mlp.get("expert") or {}).get("ff")),
                                _positive(f"layer {i} mlp.router.experts", router.get("experts")),
                                _positive(f"layer {i} mlp.router.top", router.get("top")),
                                _positive(f"layer {i} mlp.shared.ff", shared.get("ff")) if shared else 0)
        if cfg.top > cfg.experts:
            raise ConfigError(f"layer {i}: top {cfg.top} of {cfg.experts} experts")
        return cfg
    raise ConfigError(f"layer {i}: unknown feed-forward kind {kind!r}")


def _softcap(value: Any) -> float:
    if value is None:
        return 0.0          # no cap
    if not float(value) > 0.0:
        raise ConfigError(f"logit_softcap must be positive, got {value!r}")
    return float(value)


def config_from_json(raw: Mapping[str, Any]) -> ViperaxConfig:
    layers: List[LayerConfig] = []
    if not isinstance(raw.get("layers"), list) or not raw["layers"]:
        raise ConfigError("config.json lists no layers")
    for i, layer in enumerate(raw["layers"]):
        layers.append(LayerConfig(_mixer_from_json(i, layer, layers), _mlp_from_json(i, layer.get("mlp"))))
    streams = raw.get("streams")
    return ViperaxConfig(
        architecture=NAME, vocab=_positive("vocab", raw.get("vocab")), width=_positive("width", raw.get("width")),
        layers=tuple(layers), norm_eps=float(raw["norm"]["eps"]),
        embedding_scale=float((raw.get("embedding") or {}).get("scale", 1.0)),
        streams=None if streams is None else _positive("streams", streams),
        logit_scale=float(raw.get("logit_scale", 1.0)), logit_softcap=_softcap(raw.get("logit_softcap")))


def config_to_json(cfg: ViperaxConfig) -> Dict[str, Any]:
    layers = []
    for layer in cfg.layers:
        m = layer.mixer
        mixer: Dict[str, Any] = {"heads": m.heads, "dim": m.dim, "vdim": m.vdim, "kv_rank": m.kv_rank, "scale": m.scale}
        if m.window:
            mixer["mask"] = {"size": m.window}
        if m.kv_from is not None:
            mixer["kv_from"] = m.kv_from
        f = layer.mlp
        if f is None:
            mlp = None
        elif f.kind == "dense":
            mlp = {"kind": "dense", "ff": f.ff}
        else:
            mlp = {"kind": "moe", "expert": {"ff": f.ff}, "router": {"experts": f.experts, "top": f.top}}
            if f.shared_ff:
                mlp["shared"] = {"ff": f.shared_ff}
        layers.append({"type": "latent_attention", "mixer": mixer, "mlp": mlp})
    out: Dict[str, Any] = {"architecture": NAME, "vocab": cfg.vocab, "width": cfg.width, "layers": layers,
                           "norm": {"eps": cfg.norm_eps}, "embedding": {"scale": cfg.embedding_scale},
                           "logit_scale": cfg.logit_scale}
    if cfg.logit_softcap > 0.0:
        out["logit_softcap"] = cfg.logit_softcap
    if cfg.streams is not None:
        out["streams"] = cfg.streams
    return out


def model_spec(cfg: ViperaxConfig) -> ModelSpec:
    w, eps = cfg.width, cfg.norm_eps
    streams = cfg.streams if cfg.streams is not None else 1

    def norm(name: str) -> PartSpec:
        return PartSpec("layer_norm", {"width": w, "eps": eps, "bias": False}, {"weight": name})

    layers = []
    for i, layer in enumerate(cfg.layers):
        p, m, f = f"l{i}.", layer.mixer, layer.mlp
        names = {"q_weight": p + "mix.q", "gate_weight": p + "mix.g", "uk_weight": p + "mix.uk",
                 "uv_weight": p + "mix.uv", "sink": p + "mix.sink", "out_weight": p + "mix.o"}
        if m.kv_from is None:
            names.update(dkv_weight=p + "mix.dkv", dkv_norm=p + "mix.dkv.norm")
        mixer = PartSpec("latent_attention",
                         {"width": w, "n_head": m.heads, "head_dim": m.dim, "value_dim": m.vdim, "rank": m.kv_rank,
                          "scale": m.scale, "window": m.window, "eps": eps, "makes_latent": m.kv_from is None}, names)
        feed_forward = None
        if f is not None and f.kind == "dense":
            feed_forward = PartSpec("gated_mlp", {"width": w, "hidden": f.ff},
                                    {"gate_weight": p + "mlp.gate", "up_weight": p + "mlp.up",
                                     "down_weight": p + "mlp.down"})
        elif f is not None:
            names = {"table": p + "mlp.table"}
            for e in range(f.experts):
                for part in ("gate", "up", "down"):
                    names[f"e{e}_{part}"] = f"{p}mlp.e{e}.{part}"
            if f.shared_ff:
                for part in ("gate", "up", "down"):
                    names[f"shared_{part}"] = f"{p}mlp.shared.{part}"
            feed_forward = PartSpec("table_experts", {"width": w, "hidden": f.ff, "n_experts": f.experts, "top": f.top,
                                                      "vocab_size": cfg.vocab, "shared_hidden": f.shared_ff}, names)
        if cfg.streams is None:
            arrangement = PartSpec("pre_norm" if feed_forward is not None else "pre_norm_mixer", {"width": w})
        else:
            hc = {}
            for q in ("1", "2") if feed_forward is not None else ("1",):
                hc.update({"in" + q: f"{p}hc{q}.in", "out" + q: f"{p}hc{q}.out", "mix" + q: f"{p}hc{q}.mix"})
            arrangement = PartSpec("hyper_connections",
                                   {"width": w, "streams": streams, "feed_forward": feed_forward is not None}, hc)
        layers.append(LayerSpec(arrangement, norm1=norm(p + "norm1"), mixer=mixer,
                                norm2=norm(p + "norm2") if feed_forward is not None else None,
                                feed_forward=feed_forward))
    return ModelSpec(
        width=w, vocab_size=cfg.vocab,
        embedding=PartSpec("token_embedding", {"vocab_size": cfg.vocab, "width": w, "scale": cfg.embedding_scale,
                                               "copies": streams}, {"weight": "embed"}),
        position=PartSpec("none"),
        layers=tuple(layers),
        order=tuple(LayerRun(i, reads_cache_of=layer.mixer.kv_from) for i, layer in enumerate(cfg.layers)),
        final_norm=norm("final.norm"),
        head=PartSpec("linear_head", {"vocab_size": cfg.vocab, "width": w, "tied": False,
                                      "logit_scale": cfg.logit_scale, "softcap": cfg.logit_softcap}, {"weight": "head"}),
        max_positions=None, streams=streams)


def init_plan(cfg: ViperaxConfig) -> List[Tuple[str, Tuple[int, ...], str, float]]:
    """Random-weights rule, in drawing order: matrices N(0, 1/sqrt(fan_in)), gains 1 + N(0, 0.1),
    sinks N(0, 1), hyper-connection vectors around 1/S (read) and 1 (write), mixing matrices around
    the identity, and table rows of `top` different experts."""
    w = cfg.width
    plan: List[Tuple[str, Tuple[int, ...], str, float]] = [("embed", (cfg.vocab, w), "normal", 1.0 / math.sqrt(w))]

    def lin(name: str, out: int, inn: int) -> None:
        plan.append((name, (out, inn), "normal", 1.0 / math.sqrt(inn)))

    def gated(prefix: str, hidden: int) -> None:
        lin(prefix + "gate", hidden, w)
        lin(prefix + "up", hidden, w)
        lin(prefix + "down", w, hidden)

    s = cfg.streams
    for i, layer in enumerate(cfg.layers):
        p, m, f = f"l{i}.", layer.mixer, layer.mlp
        plan.append((p + "norm1", (w,), "gain", 0.1))
        lin(p + "mix.q", m.heads * m.dim, w)
        if m.kv_from is None:
            lin(p + "mix.dkv", m.kv_rank, w)
            plan.append((p + "mix.dkv.norm", (m.kv_rank,), "gain", 0.1))
        lin(p + "mix.uk", m.heads * m.dim, m.kv_rank)
        lin(p + "mix.uv", m.heads * m.vdim, m.kv_rank)
        plan.append((p + "mix.sink", (m.heads,), "normal", 1.0))
        lin(p + "mix.g", m.heads * m.vdim, w)
        lin(p + "mix.o", w, m.heads * m.vdim)
        if f is not None:
            plan.append((p + "norm2", (w,), "gain", 0.1))
            if f.kind == "dense":
                gated(p + "mlp.", f.ff)
            else:
                for e in range(f.experts):
                    gated(f"{p}mlp.e{e}.", f.ff)
                plan.append((p + "mlp.table", (cfg.vocab, f.top), "distinct", float(f.experts)))
                if f.shared_ff:
                    gated(p + "mlp.shared.", f.shared_ff)
        if s is not None:
            for q in ("1", "2") if f is not None else ("1",):
                plan.append((f"{p}hc{q}.in", (s,), "around", 1.0 / s))
                plan.append((f"{p}hc{q}.out", (s,), "gain", 0.2))
                plan.append((f"{p}hc{q}.mix", (s, s), "identity", 0.2 / s))
    plan.append(("final.norm", (w,), "gain", 0.1))
    lin("head", cfg.vocab, w)
    return plan


register_architecture(Architecture(NAME, config_from_json, model_spec, init_plan, config_to_json))
