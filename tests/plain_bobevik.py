"""A plain, slow implementation of the Bobevik decoder: one function per mechanism, whole sequences
at once on the CPU, no cache and no state carried between calls.  It shares nothing with the engine:
it reads the raw config.json dictionary and a dictionary of tensors by name.

Notation: T tokens of one sequence at positions 0 .. T-1, W the model width, H query heads, G
key/value heads, D the query/key size of a head, E its value size.
"""

from __future__ import annotations

import json
import math
import os
from typing import Dict, List, Optional, Tuple

import torch
from safetensors import safe_open

DTYPE = torch.float64       # what the functions compute in


def read_model_folder(path: str) -> Tuple[dict, Dict[str, torch.Tensor]]:
    with open(os.path.join(path, "config.json"), "r", encoding="utf-8") as fh:
        cfg = json.load(fh)
    tensors: Dict[str, torch.Tensor] = {}
    with safe_open(os.path.join(path, "model.safetensors"), framework="pt", device="cpu") as fh:
        for name in fh.keys():
            t = fh.get_tensor(name)
            tensors[name] = t.to(DTYPE) if t.is_floating_point() else t.to(torch.int64)
    return cfg, tensors


# With ROUNDING set to torch.bfloat16 every matrix product takes operands rounded to that format and
# its result is rounded to it too, as a kernel that computes "in bfloat16 with 32-bit accumulation"
# does.  The difference between the two modes is the size of what rounding alone does to the
# logits: the tests' bound for the engine's bfloat16 path is a multiple of it.
ROUNDING = None


def _r(x: torch.Tensor) -> torch.Tensor:
    return x if ROUNDING is None else x.to(ROUNDING).to(DTYPE)


def lin(h: torch.Tensor, w: torch.Tensor, b: Optional[torch.Tensor] = None) -> torch.Tensor:
    """w h (+ b) for every row of h, w stored [out, in]."""
    y = _r(h) @ _r(w).T
    return _r(y if b is None else y + b)


# ---------------------------------------------------------------- norms and activations
def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last dimension."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def rms_norm(x: torch.Tensor, gain: torch.Tensor, eps: float, one_plus: bool) -> torch.Tensor:
    """The unit-RMS rows times the gain, which is stored either as it is or as its distance from one."""
    return unit_rms(x, eps) * ((1.0 + gain) if one_plus else gain)


def silu(z: torch.Tensor) -> torch.Tensor:
    return z / (1.0 + torch.exp(-z))


def sigmoid(z: torch.Tensor) -> torch.Tensor:
    return 1.0 / (1.0 + torch.exp(-z))


def relu_gated_mlp(h: torch.Tensor, gate: torch.Tensor, up: torch.Tensor, down: torch.Tensor) -> torch.Tensor:
    """down (max(gate h, 0) * (up h))."""
    return lin(_r(torch.clamp(lin(h, gate), min=0.0) * lin(h, up)), down)


# ---------------------------------------------------------------- rotation
def rotate_half(x: torch.Tensor, dims: int, base: float, factor: float = 1.0) -> torch.Tensor:
    """x [T, heads, D]: the first `dims` channels of every head are rotated in pairs (i, i + dims/2)
    by the angle t * base^(-2i/dims) / factor at position t; the other channels pass."""
    T, half = x.shape[0], dims // 2
    freq = torch.tensor([base ** (-2.0 * i / dims) / factor for i in range(half)], dtype=DTYPE)
    angle = torch.arange(T, dtype=DTYPE)[:, None] * freq[None, :]
    c, s = torch.cos(angle)[:, None, :], torch.sin(angle)[:, None, :]
    a, b = x[..., :half], x[..., half:dims]
    return torch.cat([a * c - b * s, b * c + a * s, x[..., dims:]], dim=-1)


# ---------------------------------------------------------------- sequence mixing cores
def causal_softmax_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float,
                             softcap: Optional[float] = None) -> torch.Tensor:
    """q [T, H, D], k [T, G, D], v [T, G, E] -> [T, H, E].  Query head a reads key/value head
    a // (H / G); token t sees tokens 0 .. t; the scores may be capped by cap * tanh(s / cap)."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[2], dtype=DTYPE)
    for a in range(H):
        g = a // (H // G)
        s = (q[:, a] @ k[:, g].T) * scale
        if softcap is not None:
            s = softcap * torch.tanh(s / softcap)
        s = s.masked_fill(torch.ones(T, T, dtype=torch.bool).triu(1), -math.inf)
        out[:, a] = torch.softmax(s, dim=-1) @ v[:, g]
    return out


def decaying_state(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, decay: List[float]) -> torch.Tensor:
    """q, k [T, H, D], v [T, H, E] -> [T, H, E]: per head a matrix S [D, E] that starts at zero,
    S <- decay_a S + k_t v_t^T, and the output S^T q_t, one token after the other."""
    T, H, D = q.shape
    out = torch.zeros(T, H, v.shape[2], dtype=DTYPE)
    for a in range(H):
        S = torch.zeros(D, v.shape[2], dtype=DTYPE)
        for t in range(T):
            S = decay[a] * S + torch.outer(k[t, a], v[t, a])
            out[t, a] = S.T @ q[t, a]
    return out


# ---------------------------------------------------------------- mixers
def _rot(x: torch.Tensor, rot: Optional[dict]) -> torch.Tensor:
    if not rot:
        return x
    return rotate_half(x, int(rot["dims"]), float(rot["base"]), float((rot.get("scaling") or {}).get("factor", 1.0)))


def retention_mixer(h: torch.Tensor, m: dict, w: Dict[str, torch.Tensor], p: str, eps: float) -> torch.Tensor:
    T, H, D, E = h.shape[0], m["heads"], m["dim"], m["vdim"]
    q = _rot(lin(h, w[p + "q"]).view(T, H, D), m.get("rot"))
    k = _rot(lin(h, w[p + "k"]).view(T, H, D), m.get("rot")) * D ** -0.5
    v = lin(h, w[p + "v"]).view(T, H, E)
    o = unit_rms(decaying_state(q, k, v, m["decay"]), eps).reshape(T, H * E)
    return lin(_r(o * silu(lin(h, w[p + "g"]))), w[p + "o"])


def lightning_mixer(h: torch.Tensor, m: dict, w: Dict[str, torch.Tensor], p: str, eps: float) -> torch.Tensor:
    T, H, D, E = h.shape[0], m["heads"], m["dim"], m["vdim"]
    q = _r(silu(lin(h, w[p + "q"]))).view(T, H, D)
    k = _r(silu(lin(h, w[p + "k"]))).view(T, H, D)
    v = _r(silu(lin(h, w[p + "v"]))).view(T, H, E)
    o = rms_norm(decaying_state(q, k, v, m["decay"]).reshape(T, H * E), w[p + "norm"], eps, one_plus=False)
    return lin(_r(o * sigmoid(lin(h, w[p + "g"]))), w[p + "o"])


def attention_mixer(h: torch.Tensor, m: dict, w: Dict[str, torch.Tensor], p: str, eps: float, biases: bool,
                    qk_norm: bool, shared: dict) -> torch.Tensor:
    """shared: what the attention layers of one pass hand to each other (the first value-mixing
    layer's values)."""
    T, H, G, D, E = h.shape[0], m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    bias = (lambda n: w[p + n + ".b"]) if biases else (lambda n: None)
    q = _rot(lin(h, w[p + "q"], bias("q")).view(T, H, D), m.get("rot"))
    k = _rot(lin(h, w[p + "k"], bias("k")).view(T, G, D), m.get("rot"))
    v = lin(h, w[p + "v"], bias("v")).view(T, G, E)
    if qk_norm:
        q, k = unit_rms(q, eps), unit_rms(k, eps)
    if m.get("v_mix"):
        if "v_first" not in shared:
            shared["v_first"] = v
        else:
            lam = w[p + "vmix"]
            v = (1.0 - lam) * v + lam * shared["v_first"]
    o = causal_softmax_attention(_r(q), _r(k), _r(v), float(m["scale"]), m.get("softcap"))
    gate = sigmoid(lin(h, w[p + "g"]))                       # [T, H]
    return lin(_r((o * gate[:, :, None]).reshape(T, H * E)), w[p + "o"])


def parallel_mixer(h: torch.Tensor, m: dict, w: Dict[str, torch.Tensor], p: str, eps: float, shared: dict) -> torch.Tensor:
    left = attention_mixer(h, m["left"], w, p + "left.", eps, biases=True, qk_norm=False, shared=shared)
    right = lightning_mixer(h, m["right"], w, p + "right.", eps)
    return 0.5 * (rms_norm(left, w[p + "left.out"], eps, one_plus=False)
                  + rms_norm(right, w[p + "right.out"], eps, one_plus=False))


# ---------------------------------------------------------------- the model
def forward(cfg: dict, w: Dict[str, torch.Tensor], token_ids: List[int], layer_outputs: Optional[list] = None) -> torch.Tensor:
    """Logits [T, vocab] of one sequence; with layer_outputs a list, the residual stream after
    every layer is appended to it."""
    eps, mult = float(cfg["norm"]["eps"]), float(cfg["residual_mult"])
    x = rms_norm(w["embed"][torch.tensor(token_ids)], w["embed.norm"], eps, one_plus=True)
    shared: dict = {}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        h = _r(rms_norm(x, w[p + "norm1"], eps, one_plus=True))
        if layer["type"] == "retention":
            y = retention_mixer(h, m, w, p + "mix.", eps)
        elif layer["type"] == "attention":
            y = attention_mixer(h, m, w, p + "mix.", eps, biases=False, qk_norm=True, shared=shared)
        elif layer["type"] == "parallel":
            y = parallel_mixer(h, m, w, p + "mix.", eps, shared)
        else:
            raise ValueError(layer["type"])
        x = x + mult * rms_norm(y, w[p + "norm1b"], eps, one_plus=True)
        if layer.get("mlp") is not None:
            h = _r(rms_norm(x, w[p + "norm2"], eps, one_plus=True))
            y = relu_gated_mlp(h, w[p + "mlp.gate"], w[p + "mlp.up"], w[p + "mlp.down"])
            x = x + mult * rms_norm(y, w[p + "norm2b"], eps, one_plus=True)
        if layer_outputs is not None:
            layer_outputs.append(x.clone())
    return lin(rms_norm(x, w["final.norm"], eps, one_plus=True), w["head"])


def greedy(cfg: dict, w: Dict[str, torch.Tensor], prompt: List[int], n_new: int) -> List[int]:
    ids, out = list(prompt), []
    for _ in range(n_new):
        nxt = int(torch.argmax(forward(cfg, w, ids)[-1]))
        out.append(nxt)
        ids.append(nxt)
    return out
