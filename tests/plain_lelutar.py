"""A plain, slow Lelutar forward: whole sequences, no cache, no batching, one function per mechanism,
on the CPU in float32 or float64, sharing no code with ``velox_amd``.

Lelutar is a pre-norm decoder whose norms are Dynamic Tanh (``tanh(alpha x) w + b``, no statistics), whose
embedding adds a row of a hashed table of (previous token, token) pairs, whose layers are listed one by one in
the configuration (a layer may run another layer's weights again) and come in three kinds of mixer: grouped-query
softmax attention with biases, two head sizes and a stretched interleaved rotation; attention over a low-rank latent
without positions; and the same with one rotated key part that all heads share.  Both latent kinds send the queries
through a normed low-rank latent too, add a learned sink to the softmax's denominator and gate every head's output
with a sigmoid.  The feed-forward is ``W_down relu(W_up h)^2``, dense or as a mixture of experts with sigmoid scores,
a correction for the choice, a choice restricted to the best groups of experts, and renormalised weights.
"""
from __future__ import annotations

import json
import math
import os
from typing import Dict, List, Optional

import torch
from safetensors.torch import load_file


def read_folder(model_dir: str, dtype: torch.dtype = torch.float32):
    with open(os.path.join(model_dir, "config.json"), "r", encoding="utf-8") as handle:
        config = json.load(handle)
    weights = {name: (t.to(dtype) if t.is_floating_point() else t) for name, t in load_file(os.path.join(model_dir, "model.safetensors")).items()}
    return config, weights


def dynamic_tanh(x: torch.Tensor, w: Dict[str, torch.Tensor], name: str) -> torch.Tensor:
    """tanh(alpha x) * weight + bias, alpha a single number."""
    return torch.tanh(w[name + ".alpha"] * x) * w[name] + w[name + ".b"]


def rms_unit(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def embed(config: dict, w: Dict[str, torch.Tensor], tokens: List[int]) -> torch.Tensor:
    """x_t = E[token_t] * scale + B[(prev * mul_prev + token * mul_cur) mod buckets]; the first token reads the last row."""
    spec = config.get("embedding") or {}
    ids = torch.tensor(tokens, dtype=torch.long)
    x = w["embed"][ids] * float(spec.get("scale", 1.0))
    bigram = spec.get("bigram")
    if bigram:
        buckets = int(bigram["buckets"])
        rows = [buckets] + [(tokens[t - 1] * int(bigram["mul_prev"]) + tokens[t] * int(bigram["mul_cur"])) % buckets for t in range(1, len(tokens))]
        x = x + w["bigram"][torch.tensor(rows, dtype=torch.long)]
    return x


def stretched_frequencies(dims: int, base: float, scaling: Optional[dict]):
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = base ** (-2.0 * i / dims)
    if not scaling:
        return f, 1.0
    factor, original = float(scaling["factor"]), float(scaling["original"])

    def turn_dim(turns: float) -> float:
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(turn_dim(float(scaling["fast"]))), 0)
    hi = min(math.ceil(turn_dim(float(scaling["slow"]))), dims - 1)
    ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate_pairs(x: torch.Tensor, rot: dict) -> torch.Tensor:
    """``x`` [T, heads, d]: entries (2i, 2i + 1), i < dims / 2, of the token at position p turn by the angle p f_i (and
    grow by the stretch's magnitude); entries from ``dims`` on pass."""
    dims = int(rot["dims"])
    freqs, magnitude = stretched_frequencies(dims, float(rot["base"]), rot.get("scaling"))
    positions = torch.arange(x.shape[0], dtype=torch.float64)
    angles = (positions[:, None] * freqs[None, :]).to(torch.float32 if x.dtype == torch.float32 else x.dtype)
    cos, sin = (angles.cos() * magnitude)[:, None, :], (angles.sin() * magnitude)[:, None, :]
    out = x.clone()
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * cos - v * sin
    out[..., 1:dims:2] = v * cos + u * sin
    return out


def causal_softmax(scores: torch.Tensor, sink: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``scores`` [heads, T, T]; position i sees j <= i.  ``sink`` [heads]: exp(sink) joins every row's denominator."""
    t = scores.shape[-1]
    mask = torch.ones(t, t, dtype=torch.bool).tril()
    scores = scores.masked_fill(~mask, float("-inf"))
    if sink is None:
        return torch.softmax(scores, dim=-1)
    widened = torch.cat([scores, sink[:, None, None].expand(-1, t, 1)], dim=-1)
    return torch.softmax(widened, dim=-1)[..., :t]


def attention(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: dict) -> torch.Tensor:
    heads, groups, dim, vdim = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    t = h.shape[0]
    q = (h @ w[p + "q"].T + w[p + "q.b"]).view(t, heads, dim)
    k = (h @ w[p + "k"].T + w[p + "k.b"]).view(t, groups, dim)
    v = (h @ w[p + "v"].T + w[p + "v.b"]).view(t, groups, vdim)
    if m.get("rot"):
        q, k = rotate_pairs(q, m["rot"]), rotate_pairs(k, m["rot"])
    k = k.repeat_interleave(heads // groups, dim=1)
    v = v.repeat_interleave(heads // groups, dim=1)
    scores = torch.einsum("ihd,jhd->hij", q, k) * float(m["scale"])
    out = torch.einsum("hij,jhd->ihd", causal_softmax(scores), v)
    return out.reshape(t, heads * vdim) @ w[p + "o"].T


def latent_attention(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: dict, eps: float) -> torch.Tensor:
    """Both latent kinds: ``rot_dim`` = 0 (absent) is the one without positions."""
    heads, dim, vdim, rank = int(m["heads"]), int(m["dim"]), int(m["vdim"]), int(m["kv_rank"])
    rot_dim = int(m.get("rot_dim", 0))
    t = h.shape[0]
    c_q = rms_unit(h @ w[p + "dq"].T, eps) * w[p + "dq.norm"]
    q = (c_q @ w[p + "uq"].T).view(t, heads, dim + rot_dim)
    down = h @ w[p + "dkv"].T
    c = rms_unit(down[:, :rank], eps) * w[p + "dkv.norm"]
    k = (c @ w[p + "uk"].T).view(t, heads, dim)
    v = (c @ w[p + "uv"].T).view(t, heads, vdim)
    scores = torch.einsum("ihd,jhd->hij", q[..., :dim], k)
    if rot_dim:
        shared = rotate_pairs(down[:, None, rank:rank + rot_dim], m["rot"])[:, 0]
        turned = rotate_pairs(q[..., dim:], m["rot"])
        scores = scores + torch.einsum("ihd,jd->hij", turned, shared)
    weights = causal_softmax(scores * float(m["scale"]), w[p + "sink"])
    out = torch.einsum("hij,jhd->ihd", weights, v)
    out = out * torch.sigmoid(h @ w[p + "g"].T)[:, :, None]
    return out.reshape(t, heads * vdim) @ w[p + "o"].T


def unit(h: torch.Tensor, up: torch.Tensor, down: torch.Tensor) -> torch.Tensor:
    return torch.relu(h @ up.T).square() @ down.T


def choose_experts(z: torch.Tensor, correction: torch.Tensor, router: dict):
    """``z`` [T, E] router logits -> (indices [T, top], weights [T, top])."""
    experts, top = int(router["experts"]), int(router["top"])
    s = torch.sigmoid(z)
    choice = s + correction
    groups = router.get("groups")
    if groups:
        count, keep = int(groups["count"]), int(groups["keep"])
        per = experts // count
        grouped = choice.view(-1, count, per)
        group_score = grouped.topk(min(2, per), dim=-1).values.sum(-1)
        best = group_score.topk(keep, dim=-1).indices
        allowed = torch.zeros_like(group_score, dtype=torch.bool).scatter_(1, best, True)
        choice = grouped.masked_fill(~allowed[:, :, None], float("-inf")).reshape(-1, experts)
    index = choice.topk(top, dim=-1).indices
    picked = s.gather(1, index)
    return index, picked / (picked.sum(-1, keepdim=True) + 1e-20)


def feed_forward(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, mlp: dict) -> torch.Tensor:
    if mlp["kind"] == "dense":
        return unit(h, w[p + "up"], w[p + "down"])
    router = mlp["router"]
    index, weights = choose_experts(h.float() @ w[p + "router"].float().T if h.dtype != torch.float64 else h @ w[p + "router"].T, w[p + "correction"], router)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for k in range(index.shape[1]):
            e = int(index[t, k])
            out[t] += weights[t, k].to(h.dtype) * unit(h[t:t + 1], w[f"{p}e{e}.up"], w[f"{p}e{e}.down"])[0]
    return out


def forward(config: dict, w: Dict[str, torch.Tensor], tokens: List[int], layer_outputs: Optional[list] = None) -> torch.Tensor:
    """Logits [T, vocab] of one whole sequence."""
    eps = float(config["norm"]["eps"])
    x = embed(config, w, tokens)
    for index, layer in enumerate(config["layers"]):
        p = f"l{layer.get('weights_of', index)}."
        h = dynamic_tanh(x, w, p + "norm1")
        if layer["type"] == "attention":
            x = x + attention(h, w, p + "mix.", layer["mixer"])
        elif layer["type"] in ("latent_attention", "latent_attention_2"):
            x = x + latent_attention(h, w, p + "mix.", layer["mixer"], eps)
        else:
            raise ValueError(f"unknown layer type {layer['type']!r}")
        if layer.get("mlp") is not None:
            x = x + feed_forward(dynamic_tanh(x, w, p + "norm2"), w, p + "mlp.", layer["mlp"])
        if layer_outputs is not None:
            layer_outputs.append(x.clone())
    return (dynamic_tanh(x, w, "final.norm") @ w["head"].T) * float(config.get("logit_scale", 1.0))
