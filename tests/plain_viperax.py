"""A plain, slow implementation of the Viperax decoder: one function per mechanism, whole
sequences at once, float32 on the CPU, no cache.  It shares nothing with the engine: it reads the
raw config.json dictionary and a dictionary of tensors by name.

Notation: T tokens of one sequence, W the model width, S residual streams, H heads, D the
query/key size of a head, E its value size, R the latent size.
"""

from __future__ import annotations

import json
import math
import os
from typing import Dict, List, Optional, Tuple

import torch
from safetensors import safe_open


def read_model_folder(path: str) -> Tuple[dict, Dict[str, torch.Tensor]]:
    with open(os.path.join(path, "config.json"), "r", encoding="utf-8") as fh:
        cfg = json.load(fh)
    tensors: Dict[str, torch.Tensor] = {}
    with safe_open(os.path.join(path, "model.safetensors"), framework="pt", device="cpu") as fh:
        for name in fh.keys():
            t = fh.get_tensor(name)
            tensors[name] = t.to(torch.float32) if t.is_floating_point() else t.to(torch.int64)
    return cfg, tensors


# With ROUNDING set to torch.bfloat16 every matrix product takes operands rounded to that format and
# its result is rounded to it too, as a kernel that computes "in bfloat16 with 32-bit accumulation"
# does.  The difference between the two modes is the size of what rounding alone does to the
# logits: the tests' bound for the engine's bfloat16 path is a multiple of it.
ROUNDING = None


def _r(x: torch.Tensor) -> torch.Tensor:
    return x if ROUNDING is None else x.to(ROUNDING).to(torch.float32)


def lin(h: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """w h for every row of h, w stored [out, in]."""
    return _r(_r(h) @ _r(w).T)


# ---------------------------------------------------------------- norms
def layer_norm(x: torch.Tensor, gain: torch.Tensor, eps: float) -> torch.Tensor:
    """(x - mean) / sqrt(var + eps) * gain; var is the mean squared deviation; no bias."""
    mean = x.mean(dim=-1, keepdim=True)
    dev = x - mean
    var = (dev * dev).mean(dim=-1, keepdim=True)
    return dev / torch.sqrt(var + eps) * gain


def rms_norm(x: torch.Tensor, gain: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) * gain."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps) * gain


# ---------------------------------------------------------------- feed-forwards
def silu(z: torch.Tensor) -> torch.Tensor:
    return z / (1.0 + torch.exp(-z))


def gated_mlp(h: torch.Tensor, gate: torch.Tensor, up: torch.Tensor, down: torch.Tensor) -> torch.Tensor:
    """down (silu(gate h) * (up h)), matrices stored [out, in]."""
    return lin(silu(lin(h, gate)) * lin(h, up), down)


def table_moe(h: torch.Tensor, token_ids: List[int], table: torch.Tensor, experts: List[Tuple[torch.Tensor, ...]],
              shared: Optional[Tuple[torch.Tensor, ...]]) -> torch.Tensor:
    """Token t goes through the experts that row token_ids[t] of the table names, each weighted
    1/top, one token at a time; a shared expert takes every token."""
    out = torch.zeros(h.shape[0], experts[0][2].shape[0])
    top = table.shape[1]
    for t, tok in enumerate(token_ids):
        for e in table[tok].tolist():
            out[t] += gated_mlp(h[t:t + 1], *experts[e])[0] / top
    if shared is not None:
        out += gated_mlp(h, *shared)
    return out


# ---------------------------------------------------------------- latent attention
def latents(h: torch.Tensor, w_dkv: torch.Tensor, gain: torch.Tensor, eps: float) -> torch.Tensor:
    """What a layer remembers of every token: the RMS-normed down-projection, [T, R]."""
    return rms_norm(lin(h, w_dkv), gain, eps)


def sink_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, sink: Optional[torch.Tensor], scale: float,
                   window: int) -> torch.Tensor:
    """q [T, H, D], k [T, H, D], v [T, H, E] of one sequence -> [T, H, E].  Query i sees key j when
    0 <= i - j < window (window 0: every j <= i).  The softmax's denominator has one more term per
    head, exp(sink), with no value (sink None: the ordinary softmax)."""
    T, heads = q.shape[0], q.shape[1]
    out = torch.zeros(T, heads, v.shape[-1], dtype=q.dtype)
    for i in range(T):
        lo = 0 if window <= 0 else max(0, i - window + 1)
        for a in range(heads):
            s = (k[lo:i + 1, a] @ q[i, a]) * scale                 # [keys]
            top = float(s.max()) if sink is None else max(float(s.max()), float(sink[a]))
            e = torch.exp(s - top)
            denom = e.sum() + (0.0 if sink is None else math.exp(float(sink[a]) - top))
            out[i, a] = (e / denom) @ v[lo:i + 1, a]
    return out


def latent_attention(h: torch.Tensor, c: torch.Tensor, w_q: torch.Tensor, w_uk: torch.Tensor, w_uv: torch.Tensor,
                     sink: torch.Tensor, w_g: torch.Tensor, w_o: torch.Tensor, heads: int, scale: float,
                     window: int) -> torch.Tensor:
    """Queries from h, keys and values from the latents c (this layer's or another's), no position
    signal; sink_attention; the heads' outputs are gated by sigmoid(w_g h) before w_o."""
    T = h.shape[0]
    q = lin(h, w_q).view(T, heads, -1)
    k = lin(c, w_uk).view(T, heads, -1)
    v = lin(c, w_uv).view(T, heads, -1)
    out = _r(sink_attention(q, k, v, sink, scale, window))
    gate = 1.0 / (1.0 + torch.exp(-lin(h, w_g)))
    return lin(out.reshape(T, -1) * gate, w_o)


# ---------------------------------------------------------------- hyper-connections
def hyper_read(streams: torch.Tensor, w_in: torch.Tensor) -> torch.Tensor:
    """streams [S, T, W] -> sum_s w_in[s] streams[s]."""
    return torch.einsum("s,stw->tw", w_in, streams)


def hyper_write(streams: torch.Tensor, w_mix: torch.Tensor, w_out: torch.Tensor, y: torch.Tensor) -> torch.Tensor:
    """new[t] = sum_s w_mix[s, t] old[s] + w_out[t] y, all new streams from the old ones."""
    return torch.einsum("st,snw->tnw", w_mix, streams) + w_out[:, None, None] * y[None]


# ---------------------------------------------------------------- the model
def _mixer(cfg: dict, w: Dict[str, torch.Tensor], i: int, h: torch.Tensor, kept: Dict[int, torch.Tensor]
           ) -> torch.Tensor:
    layer = cfg["layers"][i]
    if layer["type"] != "latent_attention":
        raise ValueError(f"unknown mixer {layer['type']!r}")
    m, p, eps = layer["mixer"], f"l{i}.mix.", float(cfg["norm"]["eps"])
    if "kv_from" in m and m["kv_from"] is not None:
        c = kept[int(m["kv_from"])]
    else:
        c = kept[i] = latents(h, w[p + "dkv"], w[p + "dkv.norm"], eps)
    window = int(m["mask"]["size"]) if m.get("mask") else 0
    return latent_attention(h, c, w[p + "q"], w[p + "uk"], w[p + "uv"], w[p + "sink"], w[p + "g"], w[p + "o"],
                            int(m["heads"]), float(m["scale"]), window)


def _ffn(w: Dict[str, torch.Tensor], prefix: str) -> Tuple[torch.Tensor, ...]:
    return w[prefix + "gate"], w[prefix + "up"], w[prefix + "down"]


def _feed_forward(cfg: dict, w: Dict[str, torch.Tensor], i: int, h: torch.Tensor, tokens: List[int]) -> torch.Tensor:
    mlp, p = cfg["layers"][i]["mlp"], f"l{i}.mlp."
    if mlp["kind"] == "dense":
        return gated_mlp(h, *_ffn(w, p))
    if mlp["kind"] != "moe":
        raise ValueError(f"unknown feed-forward {mlp['kind']!r}")
    experts = [_ffn(w, f"{p}e{e}.") for e in range(int(mlp["router"]["experts"]))]
    shared = _ffn(w, p + "shared.") if mlp.get("shared") else None
    return table_moe(h, tokens, w[p + "table"], experts, shared)


def forward(cfg: dict, w: Dict[str, torch.Tensor], tokens: List[int]) -> Tuple[torch.Tensor, torch.Tensor]:
    """Logits [T, vocab] of one sequence, and the residual stream (the streams' sum) after every
    layer, [layers, T, W]."""
    eps = float(cfg["norm"]["eps"])
    x0 = w["embed"][torch.tensor(tokens)] * float(cfg.get("embedding", {}).get("scale", 1.0))
    hyper = "streams" in cfg
    streams = x0[None].repeat(int(cfg["streams"]), 1, 1) if hyper else x0[None].clone()
    kept: Dict[int, torch.Tensor] = {}
    after = []
    for i, layer in enumerate(cfg["layers"]):
        subs = [(1, lambda h, i=i: _mixer(cfg, w, i, h, kept))]
        if layer.get("mlp"):
            subs.append((2, lambda h, i=i: _feed_forward(cfg, w, i, h, tokens)))
        for q, fn in subs:
            if hyper:
                u = hyper_read(streams, w[f"l{i}.hc{q}.in"])
                y = fn(layer_norm(u, w[f"l{i}.norm{q}"], eps))
                streams = hyper_write(streams, w[f"l{i}.hc{q}.mix"], w[f"l{i}.hc{q}.out"], y)
            else:
                streams = streams + fn(layer_norm(streams[0], w[f"l{i}.norm{q}"], eps))[None]
        after.append(streams.sum(dim=0))
    x = streams.sum(dim=0)
    logits = _r(_r(layer_norm(x, w["final.norm"], eps)) @ _r(w["head"]).T).to(torch.float32) \
        * float(cfg.get("logit_scale", 1.0))
    if "logit_softcap" in cfg:
        cap = float(cfg["logit_softcap"])
        logits = cap * torch.tanh(logits / cap)
    return logits, torch.stack(after)


def greedy(cfg: dict, w: Dict[str, torch.Tensor], prompt: List[int], n_new: int) -> List[int]:
    ids, out = list(prompt), []
    for _ in range(n_new):
        tok = int(forward(cfg, w, ids)[0][-1].argmax())
        out.append(tok)
        ids.append(tok)
    return out
