"""Bobevik: a decoder whose layers are listed one by one in config.json and mix three kinds of
sequence mixers, as data.

What the design fixes, and is therefore set here and handed to the parts as parameters:
- every norm is an RMS norm with one eps (config `norm.eps`); the norms of the model and around
  the sublayers store their gain as its distance from one, the others as it is;
- the embedded tokens are normed (`embed.norm`) before the first layer; no position table;
- a layer norms each sublayer on both sides and scales what it adds to the residual by
  `residual_mult` (the `sandwich_norm` arrangement); `mlp: null` leaves the feed-forward out;
- layer type `retention`: a decaying state per head (`decay`), queries and keys rotated
  (`rot.dims`, `rot.base`, pairs (i, i + dims/2)), keys times dim^-1/2, each head's output divided
  by its root mean square, a silu gate;
- layer type `attention`: grouped softmax attention with rotation, queries and keys divided by
  their root mean square per head, `scale` from the config, one sigmoid gate per head, and with
  `v_mix` the values mixed with those of the first such layer (its own values kept for the others);
- layer type `parallel`: two mixers side by side on the same input, `left` a softmax attention with
  biases, rotation with linearly scaled positions (`rot.scaling.factor`), capped scores (`softcap`)
  and the gate per head, `right` a decaying state whose queries, keys and values pass silu, whose
  concatenated heads are normed with a gain and gated by a sigmoid; the layer's mixer output is the
  mean of the two, each normed over the model width with a gain of its own;
- feed-forward `dense`: down(relu(gate h) * (up h));
- the head: the model's norm (`final.norm`), then `head`, untied.

Tensor names: `embed`, `embed.norm`, `l<i>.norm1|norm1b|norm2|norm2b`, `l<i>.mix.{q,k,v,g,o}`
(retention; attention also `vmix`), `l<i>.mix.left.{q,q.b,k,k.b,v,v.b,g,o,out}`,
`l<i>.mix.right.{q,k,v,g,o,norm,out}`, `l<i>.mlp.{gate,up,down}`, `final.norm`, `head`; linear
weights are stored [out, in].
"""

from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Any, Dict, List, Mapping, Optional, Tuple

from ..config.model_config import ConfigError
from ..config.registry import Architecture, register_architecture
from ..parts.base import PartSpec
from ..parts.model import LayerRun, LayerSpec, ModelSpec

NAME = "Bobevik"


@dataclass(frozen=True)
class Rotation:
    dims: int
    base: float
    factor: float = 1.0         # positions are divided by it (linear scaling); 1: none


@dataclass(frozen=True)
class StateMixerConfig:
    """`retention`, and the right half of `parallel`."""
    heads: int
    dim: int
    vdim: int
    decay: Tuple[float, ...]
    rot: Optional[Rotation] = None


@dataclass(frozen=True)
class AttentionConfig:
    """`attention`, and the left half of `parallel`."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot: Optional[Rotation] = None
    softcap: float = 0.0        # 0: scores are not capped
    v_mix: bool = False


@dataclass(frozen=True)
class LayerConfig:
    type: str                                   # "retention", "attention" or "parallel"
    mixer: Any                                  # StateMixerConfig, AttentionConfig, or (AttentionConfig, StateMixerConfig)
    ff: Optional[int]                           # hidden size of the dense feed-forward, None: no feed-forward


@dataclass(frozen=True)
class BobevikConfig:
    architecture: str
    vocab: int
    width: int
    layers: Tuple[LayerConfig, ...]
    norm_eps: float
    residual_mult: float = 1.0


def _positive(name: str, value: Any) -> int:
    if not isinstance(value, int) or isinstance(value, bool) or value <= 0:
        raise ConfigError(f"{name} must be a positive integer, got {value!r}")
    return value


def _rotation(where: str, rot: Optional[Mapping[str, Any]], dim: int) -> Optional[Rotation]:
    if not rot:
        return None
    dims = _positive(f"{where} rot.dims", rot.get("dims"))
    if dims % 2 or dims > dim:
        raise ConfigError(f"{where}: rot.dims must be even and at most dim, got {dims}")
    factor = float((rot.get("scaling") or {}).get("factor", 1.0))
    if not (float(rot["base"]) > 0.0 and factor > 0.0):
        raise ConfigError(f"{where}: rot.base and rot.scaling.factor must be positive")
    return Rotation(dims, float(rot["base"]), factor)


def _state_mixer(where: str, m: Mapping[str, Any]) -> StateMixerConfig:
    heads = _positive(f"{where} heads", m.get("heads"))
    dim = _positive(f"{where} dim", m.get("dim"))
    decay = m.get("decay")
    if not isinstance(decay, list) or len(decay) != heads:
        raise ConfigError(f"{where}: decay must list one number per head")
    return StateMixerConfig(heads, dim, _positive(f"{where} vdim", m.get("vdim")), tuple(float(d) for d in decay),
                            _rotation(where, m.get("rot"), dim))


def _attention(where: str, m: Mapping[str, Any]) -> AttentionConfig:
    heads = _positive(f"{where} heads", m.get("heads"))
    kv_heads = _positive(f"{where} kv_heads", m.get("kv_heads"))
    if heads % kv_heads:
        raise ConfigError(f"{where}: heads must be a multiple of kv_heads")
    dim = _positive(f"{where} dim", m.get("dim"))
    cap = m.get("softcap")
    if cap is not None and not float(cap) > 0.0:
        raise ConfigError(f"{where}: softcap must be positive, got {cap!r}")
    return AttentionConfig(heads, kv_heads, dim, _positive(f"{where} vdim", m.get("vdim")), float(m["scale"]),
                           _rotation(where, m.get("rot"), dim), 0.0 if cap is None else float(cap), bool(m.get("v_mix", False)))


def config_from_json(raw: Mapping[str, Any]) -> BobevikConfig:
    if not isinstance(raw.get("layers"), list) or not raw["layers"]:
        raise ConfigError("config.json lists no layers")
    layers: List[LayerConfig] = []
    for i, layer in enumerate(raw["layers"]):
        kind, m = layer.get("type"), layer.get("mixer")
        if not isinstance(m, Mapping):
            raise ConfigError(f"layer {i}: no mixer sizes")
        if kind == "retention":
            mixer: Any = _state_mixer(f"layer {i}", m)
        elif kind == "attention":
            mixer = _attention(f"layer {i}", m)
        elif kind == "parallel":
            if not isinstance(m.get("left"), Mapping) or not isinstance(m.get("right"), Mapping):
                raise ConfigError(f"layer {i}: a parallel mixer has a left and a right half")
            mixer = (_attention(f"layer {i} left", m["left"]), _state_mixer(f"layer {i} right", m["right"]))
        else:
            raise ConfigError(f"layer {i}: unknown mixer type {kind!r}")
        mlp = layer.get("mlp")
        if mlp is not None and mlp.get("kind") != "dense":
            raise ConfigError(f"layer {i}: unknown feed-forward kind {mlp.get('kind')!r}")
        layers.append(LayerConfig(kind, mixer, None if mlp is None else _positive(f"layer {i} mlp.ff", mlp.get("ff"))))
    mixing = [l.mixer for l in layers if l.type == "attention" and l.mixer.v_mix]
    if len({(m.kv_heads, m.vdim) for m in mixing}) > 1:
        raise ConfigError("layers that mix their values with the first such layer's need its key/value heads and sizes")
    return BobevikConfig(architecture=NAME, vocab=_positive("vocab", raw.get("vocab")),
                         width=_positive("width", raw.get("width")), layers=tuple(layers),
                         norm_eps=float(raw["norm"]["eps"]), residual_mult=float(raw.get("residual_mult", 1.0)))


def _rotation_json(rot: Optional[Rotation]) -> Optional[Dict[str, Any]]:
    if rot is None:
        return None
    out: Dict[str, Any] = {"base": rot.base, "dims": rot.dims}
    if rot.factor != 1.0:
        out["scaling"] = {"factor": rot.factor}
    return out


def _state_json(m: StateMixerConfig) -> Dict[str, Any]:
    out: Dict[str, Any] = {"decay": list(m.decay), "dim": m.dim, "heads": m.heads, "vdim": m.vdim}
    if m.rot is not None:
        out["rot"] = _rotation_json(m.rot)
    return out


def _attention_json(m: AttentionConfig) -> Dict[str, Any]:
    out: Dict[str, Any] = {"dim": m.dim, "heads": m.heads, "kv_heads": m.kv_heads, "scale": m.scale, "vdim": m.vdim}
    if m.rot is not None:
        out["rot"] = _rotation_json(m.rot)
    if m.softcap > 0.0:
        out["softcap"] = m.softcap
    if m.v_mix:
        out["v_mix"] = True
    return out


def config_to_json(cfg: BobevikConfig) -> Dict[str, Any]:
    layers = []
    for layer in cfg.layers:
        if layer.type == "retention":
            mixer = _state_json(layer.mixer)
        elif layer.type == "attention":
            mixer = _attention_json(layer.mixer)
        else:
            mixer = {"left": _attention_json(layer.mixer[0]), "right": _state_json(layer.mixer[1])}
        layers.append({"type": layer.type, "mixer": mixer,
                       "mlp": None if layer.ff is None else {"kind": "dense", "ff": layer.ff}})
    return {"architecture": NAME, "vocab": cfg.vocab, "width": cfg.width, "layers": layers,
            "norm": {"eps": cfg.norm_eps}, "residual_mult": cfg.residual_mult}


def _rotary_params(rot: Optional[Rotation]) -> Optional[Dict[str, Any]]:
    return None if rot is None else {"kind": "rotary_half", "dims": rot.dims, "base": rot.base, "factor": rot.factor}


def model_spec(cfg: BobevikConfig) -> ModelSpec:
    w, eps = cfg.width, cfg.norm_eps

    def norm(name: str, one_plus: bool = True) -> PartSpec:
        return PartSpec("rms_norm", {"width": w, "eps": eps, "one_plus": one_plus}, {"weight": name})

    def attention(m: AttentionConfig, p: str, biases: bool, qk_norm: bool, value_mix: Optional[str]) -> PartSpec:
        names = {"q_weight": p + "q", "k_weight": p + "k", "v_weight": p + "v", "gate_weight": p + "g",
                 "out_weight": p + "o"}
        if biases:
            names.update(q_bias=p + "q.b", k_bias=p + "k.b", v_bias=p + "v.b")
        if value_mix is not None:
            names["mix"] = p + "vmix"
        return PartSpec("gated_attention",
                        {"width": w, "n_head": m.heads, "n_kv_head": m.kv_heads, "head_dim": m.dim, "value_dim": m.vdim,
                         "scale": m.scale, "bias": biases, "rotary": _rotary_params(m.rot),
                         "qk_norm_eps": eps if qk_norm else None, "softcap": m.softcap, "head_gate": True,
                         "value_mix": value_mix, "share": "first_values"}, names)

    def state(m: StateMixerConfig, p: str, lightning: bool) -> PartSpec:
        names = {"q_weight": p + "q", "k_weight": p + "k", "v_weight": p + "v", "gate_weight": p + "g",
                 "out_weight": p + "o"}
        params = {"width": w, "n_head": m.heads, "head_dim": m.dim, "value_dim": m.vdim, "decay": list(m.decay),
                  "rotary": _rotary_params(m.rot)}
        if lightning:
            names["norm_weight"] = p + "norm"
            params.update(input_activation="silu", out_norm_eps=eps)
        else:
            params.update(k_scale=m.dim ** -0.5, head_norm_eps=eps)
        return PartSpec("decay_state", params, names)

    layers, seen_value_mix = [], False
    for i, layer in enumerate(cfg.layers):
        p = f"l{i}."
        parts: Dict[str, Tuple[str, PartSpec]] = {"norm1": ("norm", norm(p + "norm1")), "norm1b": ("norm", norm(p + "norm1b"))}
        branches = 1
        if layer.type == "retention":
            parts["mixer"] = ("mixer", state(layer.mixer, p + "mix.", lightning=False))
        elif layer.type == "attention":
            value_mix = None
            if layer.mixer.v_mix:
                value_mix = "mix" if seen_value_mix else "keep"
                seen_value_mix = True
            parts["mixer"] = ("mixer", attention(layer.mixer, p + "mix.", biases=False, qk_norm=True, value_mix=value_mix))
        else:
            branches = 2
            left, right = layer.mixer
            parts["mixer0"] = ("mixer", attention(left, p + "mix.left.", biases=True, qk_norm=False, value_mix=None))
            parts["mixer1"] = ("mixer", state(right, p + "mix.right.", lightning=True))
            parts["join0"] = ("norm", norm(p + "mix.left.out", one_plus=False))
            parts["join1"] = ("norm", norm(p + "mix.right.out", one_plus=False))
        if layer.ff is not None:
            parts["norm2"] = ("norm", norm(p + "norm2"))
            parts["norm2b"] = ("norm", norm(p + "norm2b"))
            parts["feed_forward"] = ("feed_forward", PartSpec(
                "gated_mlp", {"width": w, "hidden": layer.ff, "activation": "relu"},
                {"gate_weight": p + "mlp.gate", "up_weight": p + "mlp.up", "down_weight": p + "mlp.down"}))
        arrangement = PartSpec("sandwich_norm", {"width": w, "residual_mult": cfg.residual_mult,
                                                 "feed_forward": layer.ff is not None, "branches": branches})
        layers.append(LayerSpec(arrangement, parts=parts))
    return ModelSpec(
        width=w, vocab_size=cfg.vocab,
        embedding=PartSpec("token_embedding", {"vocab_size": cfg.vocab, "width": w}, {"weight": "embed"}),
        position=PartSpec("none"),
        layers=tuple(layers), order=tuple(LayerRun(i) for i in range(len(layers))),
        final_norm=norm("final.norm"),
        head=PartSpec("linear_head", {"vocab_size": cfg.vocab, "width": w, "tied": False}, {"weight": "head"}),
        max_positions=None, embedding_norm=norm("embed.norm"))


def init_plan(cfg: BobevikConfig) -> List[Tuple[str, Tuple[int, ...], str, float]]:
    """Random-weights rule, in drawing order: matrices N(0, 1/sqrt(fan_in)), biases N(0, 0.5), gains stored as
    their distance from one N(0, 0.1), plain gains 1 + N(0, 0.1), mixing weights around 0.4."""
    w = cfg.width
    plan: List[Tuple[str, Tuple[int, ...], str, float]] = [("embed", (cfg.vocab, w), "normal", 1.0),
                                                          ("embed.norm", (w,), "normal", 0.1)]

    def lin(name: str, out: int, inn: int) -> None:
        plan.append((name, (out, inn), "normal", 1.0 / math.sqrt(inn)))

    def state(p: str, m: StateMixerConfig, lightning: bool) -> None:
        for n, out in (("q", m.heads * m.dim), ("k", m.heads * m.dim), ("v", m.heads * m.vdim), ("g", m.heads * m.vdim)):
            lin(p + n, out, w)
        lin(p + "o", w, m.heads * m.vdim)
        if lightning:
            plan.append((p + "norm", (m.heads * m.vdim,), "gain", 0.1))

    def attention(p: str, m: AttentionConfig, biases: bool) -> None:
        for n, out in (("q", m.heads * m.dim), ("k", m.kv_heads * m.dim), ("v", m.kv_heads * m.vdim)):
            lin(p + n, out, w)
            if biases:
                plan.append((p + n + ".b", (out,), "normal", 0.5))
        if m.v_mix:
            plan.append((p + "vmix", (), "around", 0.4))
        lin(p + "g", m.heads, w)
        lin(p + "o", w, m.heads * m.vdim)

    for i, layer in enumerate(cfg.layers):
        p = f"l{i}."
        for n in ("norm1", "norm1b") + (("norm2", "norm2b") if layer.ff is not None else ()):
            plan.append((p + n, (w,), "normal", 0.1))
        if layer.type == "retention":
            state(p + "mix.", layer.mixer, lightning=False)
        elif layer.type == "attention":
            attention(p + "mix.", layer.mixer, biases=False)
        else:
            attention(p + "mix.left.", layer.mixer[0], biases=True)
            state(p + "mix.right.", layer.mixer[1], lightning=True)
            plan.append((p + "mix.left.out", (w,), "gain", 0.1))
            plan.append((p + "mix.right.out", (w,), "gain", 0.1))
        if layer.ff is not None:
            lin(p + "mlp.gate", layer.ff, w)
            lin(p + "mlp.up", layer.ff, w)
            lin(p + "mlp.down", w, layer.ff)
    plan.append(("final.norm", (w,), "normal", 0.1))
    lin("head", cfg.vocab, w)
    return plan


register_architecture(Architecture(NAME, config_from_json, model_spec, init_plan, config_to_json))
