"""Gosulorn, written out plainly: whole sequences, no cache, token-by-token loops, one function per mechanism.

This is the yardstick of the tests.  It shares no code with ``velox_amd``: it takes the configuration as the dictionary
that ``config.json`` holds and the tensors by their checkpoint names, and runs in whatever float type the tensors have
(the tests hand it float64 or float32 copies).

Notation: ``n`` tokens, width ``W``; ``h`` is a sub-layer's input ``[n, W]``.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch


# ----------------------------------------------------------------------------------------------------------------------
# small pieces
# ----------------------------------------------------------------------------------------------------------------------
def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def layer_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    mean = x.mean(-1, keepdim=True)
    var = ((x - mean) ** 2).mean(-1, keepdim=True)
    return (x - mean) / torch.sqrt(var + eps) * weight


def rms_norm(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x ** 2).mean(-1, keepdim=True) + eps)


def unit_vector(x: torch.Tensor) -> torch.Tensor:
    return x / torch.sqrt((x ** 2).sum(-1, keepdim=True) + 1e-6)


def short_conv(u: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """``u`` [n, C], ``w`` [C, taps]: ``y_t = sum_j w[:, j] u_(t - taps + 1 + j)`` with zeros before the start."""
    n, taps = u.shape[0], w.shape[1]
    y = torch.zeros_like(u)
    for t in range(n):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                y[t] += w[:, j] * u[s]
    return y


def rotate_halves(x: torch.Tensor, dims: int, base: float, factor: float, first_position: int = 0) -> torch.Tensor:
    """``x`` [n, heads, d]: the first ``dims`` channels of each head are rotated, channel ``i`` paired with ``i + dims/2``."""
    if dims == 0:
        return x
    n = x.shape[0]
    half = dims // 2
    freq = torch.tensor([base ** (-2.0 * i / dims) / factor for i in range(half)], dtype=torch.float64)
    angle = torch.arange(first_position, first_position + n, dtype=torch.float64)[:, None] * freq[None, :]
    cos, sin = angle.cos().to(x.dtype)[:, None, :], angle.sin().to(x.dtype)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * cos - v * sin, v * cos + u * sin, x[..., dims:]], dim=-1)


# ----------------------------------------------------------------------------------------------------------------------
# mixers
# ----------------------------------------------------------------------------------------------------------------------
def window_attention(h: torch.Tensor, t: Dict[str, torch.Tensor], p: str, c: dict) -> torch.Tensor:
    """Softmax attention over a sliding window, with biases, a short convolution on q, k and v, and a partial rotation."""
    n = h.shape[0]
    heads, kv_heads, dim, vdim = c["heads"], c["kv_heads"], c["dim"], c["vdim"]

    def projected(name):
        y = h @ t[p + name].T
        if p + name + ".b" in t:
            y = y + t[p + name + ".b"]
        if c.get("conv"):
            y = short_conv(y, t[p + name + ".conv"])
        return y

    q = projected("q").reshape(n, heads, dim)
    k = projected("k").reshape(n, kv_heads, dim)
    v = projected("v").reshape(n, kv_heads, vdim)
    rot = c.get("rot")
    if rot:
        factor = (rot.get("scaling") or {}).get("factor", 1.0)
        q = rotate_halves(q, rot["dims"], rot["base"], factor)
        k = rotate_halves(k, rot["dims"], rot["base"], factor)
    window = (c.get("mask") or {}).get("size")
    group = heads // kv_heads
    out = torch.zeros(n, heads, vdim, dtype=h.dtype)
    for i in range(n):
        lo = 0 if window is None else max(0, i - window + 1)
        for a in range(heads):
            g = a // group
            scores = (k[lo:i + 1, g] @ q[i, a]) * c["scale"]
            weights = torch.softmax(scores, dim=0)
            out[i, a] = weights @ v[lo:i + 1, g]
    y = out.reshape(n, heads * vdim) @ t[p + "o"].T
    if p + "o.b" in t:
        y = y + t[p + "o.b"]
    return y


def delta_rule_scan(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, decay: torch.Tensor, beta: torch.Tensor) -> torch.Tensor:
    """Per head: ``S <- decay * S`` (row-wise), ``u = beta (v - S^T k)``, ``S <- S + k u^T``, ``o = S^T q``.
    ``q``, ``k`` [n, heads, d]; ``v`` [n, heads, e]; ``decay`` [n, heads, d]; ``beta`` [n, heads]."""
    n, heads, d = q.shape
    e = v.shape[-1]
    state = torch.zeros(heads, d, e, dtype=q.dtype)
    out = torch.zeros(n, heads, e, dtype=q.dtype)
    for i in range(n):
        for a in range(heads):
            s = decay[i, a][:, None] * state[a]
            u = beta[i, a] * (v[i, a] - s.T @ k[i, a])
            s = s + torch.outer(k[i, a], u)
            out[i, a] = s.T @ q[i, a]
            state[a] = s
    return out


def _delta_inputs(h, t, p, c):
    n = h.shape[0]
    heads, kv_heads, dim, vdim = c["heads"], c["kv_heads"], c["dim"], c["vdim"]

    def projected(name):
        y = h @ t[p + name].T
        if c.get("conv"):
            y = short_conv(y, t[p + name + ".conv"])
        return silu(y)

    q = unit_vector(projected("q").reshape(n, kv_heads, dim)) * dim ** -0.5
    k = unit_vector(projected("k").reshape(n, kv_heads, dim))
    v = projected("v").reshape(n, heads, vdim)
    repeat = heads // kv_heads
    q = q.repeat_interleave(repeat, dim=1)
    k = k.repeat_interleave(repeat, dim=1)
    beta = torch.sigmoid(h @ t[p + "b"].T)
    return q, k, v, beta


def delta_mixer(h: torch.Tensor, t: Dict[str, torch.Tensor], p: str, c: dict, eps: float) -> torch.Tensor:
    """Gated delta rule with one decay per head and a SiLU gate on the normed read-out."""
    n = h.shape[0]
    heads, dim, vdim = c["heads"], c["dim"], c["vdim"]
    q, k, v, beta = _delta_inputs(h, t, p, c)
    step = torch.nn.functional.softplus(h @ t[p + "a"].T + t[p + "dt_bias"])
    decay = torch.exp(-torch.exp(t[p + "A_log"]) * step)  # [n, heads]
    o = delta_rule_scan(q, k, v, decay[:, :, None].expand(n, heads, dim), beta)
    o = rms_norm(o, eps) * t[p + "norm"] * silu(h @ t[p + "g"].T).reshape(n, heads, vdim)
    return o.reshape(n, heads * vdim) @ t[p + "o"].T


def channel_delta_mixer(h: torch.Tensor, t: Dict[str, torch.Tensor], p: str, c: dict, eps: float) -> torch.Tensor:
    """Gated delta rule with one decay per head and key channel (a low-rank map) and a sigmoid gate (a low-rank map)."""
    n = h.shape[0]
    heads, dim, vdim = c["heads"], c["dim"], c["vdim"]
    q, k, v, beta = _delta_inputs(h, t, p, c)
    step = torch.nn.functional.softplus((h @ t[p + "a1"].T) @ t[p + "a2"].T + t[p + "dt_bias"]).reshape(n, heads, dim)
    decay = torch.exp(-torch.exp(t[p + "A_log"])[None, :, None] * step)
    o = delta_rule_scan(q, k, v, decay, beta)
    gate = torch.sigmoid((h @ t[p + "g1"].T) @ t[p + "g2"].T).reshape(n, heads, vdim)
    o = rms_norm(o, eps) * t[p + "norm"] * gate
    return o.reshape(n, heads * vdim) @ t[p + "o"].T


def gla_mixer(h: torch.Tensor, t: Dict[str, torch.Tensor], p: str, c: dict, eps: float) -> torch.Tensor:
    """Gated linear attention: ``S_t = diag(alpha_t) S_(t-1) + k_t v_t^T``, ``o_t = S_t^T q_t``."""
    n = h.shape[0]
    heads, dim, vdim = c["heads"], c["dim"], c["vdim"]
    q = (h @ t[p + "q"].T).reshape(n, heads, dim) * dim ** -0.5
    k = (h @ t[p + "k"].T).reshape(n, heads, dim)
    v = (h @ t[p + "v"].T).reshape(n, heads, vdim)
    z = (h @ t[p + "a1"].T) @ t[p + "a2"].T + t[p + "a2.b"]
    alpha = (torch.sigmoid(z) ** (1.0 / c["tau"])).reshape(n, heads, dim)
    state = torch.zeros(heads, dim, vdim, dtype=h.dtype)
    out = torch.zeros(n, heads, vdim, dtype=h.dtype)
    for i in range(n):
        for a in range(heads):
            state[a] = alpha[i, a][:, None] * state[a] + torch.outer(k[i, a], v[i, a])
            out[i, a] = state[a].T @ q[i, a]
    o = (rms_norm(out, eps) * t[p + "norm"]).reshape(n, heads * vdim) * silu(h @ t[p + "g"].T)
    return o @ t[p + "o"].T


def parallel_mixer(h, t, p, c, eps):
    left = window_attention(h, t, p + "left.", c["left"])
    right = channel_delta_mixer(h, t, p + "right.", c["right"], eps)
    return c["left_scale"] * left + c["right_scale"] * right


def mixer(kind: str, h, t, p, c, eps):
    if kind == "parallel":
        return parallel_mixer(h, t, p, c, eps)
    if kind == "gla":
        return gla_mixer(h, t, p, c, eps)
    if kind == "delta":
        return delta_mixer(h, t, p, c, eps)
    raise ValueError(kind)


def dense_feed_forward(h, t, p):
    return (gelu_tanh(h @ t[p + "gate"].T) * (h @ t[p + "up"].T)) @ t[p + "down"].T


# ----------------------------------------------------------------------------------------------------------------------
# the model
# ----------------------------------------------------------------------------------------------------------------------
def forward(config: dict, tensors: Dict[str, torch.Tensor], tokens: List[int], layer_outputs: Optional[list] = None) -> torch.Tensor:
    """Logits ``[n, vocab]`` of a whole sequence.  ``layer_outputs``: a list that gets the residual stream (the sum of
    the streams, where there are several) after every layer run."""
    eps = config["norm"]["eps"]
    streams = config.get("streams")
    x = tensors["embed"][torch.tensor(tokens, dtype=torch.long)]
    xs = [x.clone() for _ in range(streams)] if streams else None
    for index, layer in enumerate(config["layers"]):
        owner = layer.get("weights_of", index)
        p = f"l{owner}."
        sublayers = [(1, lambda h, layer=layer, p=p: mixer(layer["type"], h, tensors, p + "mix.", layer["mixer"], eps))]
        if layer.get("mlp") is not None:
            sublayers.append((2, lambda h, p=p: dense_feed_forward(h, tensors, p + "mlp.")))
        for number, sublayer in sublayers:
            weight = tensors[f"{p}norm{number}"]
            if xs is None:
                x = x + sublayer(layer_norm(x, weight, eps))
                continue
            w_in, w_out, w_mix = tensors[f"{p}hc{number}.in"], tensors[f"{p}hc{number}.out"], tensors[f"{p}hc{number}.mix"]
            u = sum(w_in[s] * xs[s] for s in range(streams))
            y = sublayer(layer_norm(u, weight, eps))
            xs = [sum(w_mix[s, to] * xs[s] for s in range(streams)) + w_out[to] * y for to in range(streams)]
        if layer_outputs is not None:
            layer_outputs.append(sum(xs) if xs is not None else x.clone())
    if xs is not None:
        x = sum(xs)
    return layer_norm(x, tensors["final.norm"], eps) @ tensors["embed"].T
