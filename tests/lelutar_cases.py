"""Small Lelutar configurations and weights for the tests, written here from the design's tensor names and shapes
(not from the framework's tables, so that a wrong name or shape there shows), with weights large enough that
attention is peaked and routers decide clearly: a key that is lost, a sink or a correction that is left out, a group
that is not masked or a pair hashed to another row then changes the logits by far more than any tolerance."""
from __future__ import annotations

import json
import os
from typing import Dict, List, Optional

import torch
from safetensors.torch import save_file


def rot(dims, base=10000.0, scaling=None) -> dict:
    out = {"dims": dims, "base": base}
    if scaling is not None:
        out["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    return out


def attention(heads, kv_heads, dim, vdim, scale, rotation=None, mlp=None, weights_of=None) -> dict:
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if rotation is not None:
        mixer["rot"] = rotation
    return _layer("attention", mixer, mlp, weights_of)


def latent(heads, dim, vdim, kv_rank, q_rank, scale, mlp=None, weights_of=None) -> dict:
    return _layer("latent_attention", {"heads": heads, "dim": dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank, "scale": scale}, mlp, weights_of)


def latent_2(heads, dim, rot_dim, vdim, kv_rank, q_rank, scale, base=10000.0, scaling=None, mlp=None, weights_of=None) -> dict:
    mixer = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank, "scale": scale,
             "rot": rot(rot_dim, base, scaling)}
    return _layer("latent_attention_2", mixer, mlp, weights_of)


def _layer(kind, mixer, mlp, weights_of) -> dict:
    out = {"type": kind, "mixer": mixer, "mlp": mlp}
    if weights_of is not None:
        out["weights_of"] = weights_of
    return out


def dense(ff) -> dict:
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, groups=None) -> dict:
    router = {"experts": experts, "top": top}
    if groups is not None:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    return {"kind": "moe", "router": router, "expert": {"ff": ff}}


# Every kind of layer, sizes that differ wherever two could be told apart: grouped heads with two head sizes and a
# rotation over part of a head, a stretch whose ramp lies inside the rotation and an original length below the tests'
# prompts, latents of other ranks for queries and keys, layers that run another's weights (one of each kind, one of them
# twice), a layer without a feed-forward, experts in three groups of which two are kept.
_STRETCH = (4.0, 24, 8.0, 1.0)
_A_ATTENTION = dict(heads=4, kv_heads=2, dim=16, vdim=24, scale=0.3, rotation=rot(8, 300.0, _STRETCH), mlp=dense(80))
_A_LATENT_2 = dict(heads=2, dim=16, rot_dim=8, vdim=8, kv_rank=24, q_rank=20, scale=0.25, base=500.0, scaling=(3.0, 16, 4.0, 0.5), mlp=None)
CONFIG_A = {
    "architecture": "Lelutar", "vocab": 97, "width": 64, "norm": {"eps": 1e-5}, "logit_scale": 1.5,
    "embedding": {"scale": 1.75, "bigram": {"buckets": 31, "mul_prev": 7, "mul_cur": 3}},
    "layers": [
        attention(**_A_ATTENTION),
        latent(3, 8, 12, 20, 12, 0.35, mlp=moe(6, 2, 24, groups=(3, 2))),
        latent_2(**_A_LATENT_2),
        attention(**_A_ATTENTION, weights_of=0),
        latent_2(**_A_LATENT_2, weights_of=2),
        attention(**_A_ATTENTION, weights_of=0),
    ],
}
# Everything that can be 1 or equal is: one head that is its own group, equal sizes of keys and values, a rotation over
# the whole head without a stretch, groups of one expert, one group kept, no bigram table, no scales.
CONFIG_B = {
    "architecture": "Lelutar", "vocab": 131, "width": 88, "norm": {"eps": 3e-6},
    "layers": [
        latent(1, 12, 12, 12, 12, 0.3, mlp=moe(2, 1, 20, groups=(2, 1))),
        attention(1, 1, 12, 12, 0.3, rotation=rot(12, 100.0), mlp=dense(72)),
        latent_2(1, 12, 12, 12, 12, 12, 0.2, base=100.0, mlp=moe(3, 3, 16)),
        attention(1, 1, 8, 8, 0.4, rotation=None, mlp=None),
    ],
}
# Sizes the kernels for decode-sized bfloat16 batches take (widths that are multiples of 64), experts without groups in
# one layer and four groups in another, a multiplier so large that the hash needs 64 bits.
CONFIG_C = {
    "architecture": "Lelutar", "vocab": 160, "width": 128, "norm": {"eps": 1e-5}, "logit_scale": 0.5,
    "embedding": {"scale": 3.0, "bigram": {"buckets": 257, "mul_prev": 2000000011, "mul_cur": 1999999973}},
    "layers": [
        attention(8, 2, 32, 48, 0.18, rotation=rot(32, 10000.0, (2.0, 32, 16.0, 1.0)), mlp=moe(8, 3, 64, groups=(4, 2))),
        latent(4, 32, 16, 64, 64, 0.15, mlp=dense(192)),
        latent_2(4, 32, 16, 32, 48, 64, 0.15, scaling=(8.0, 20, 16.0, 1.0), mlp=moe(8, 2, 64)),
        latent(4, 32, 16, 64, 64, 0.15, mlp=dense(192), weights_of=1),
    ],
}
# Nothing a multiple of 4, 8 or 16: rows of 200 bytes, as many key heads as query heads, cached vectors of 18 and 24
# channels, nine experts in three groups of which one is kept.
CONFIG_D = {
    "architecture": "Lelutar", "vocab": 77, "width": 100, "norm": {"eps": 1e-5}, "logit_scale": 3.0,
    "embedding": {"scale": 0.5, "bigram": {"buckets": 13, "mul_prev": 5, "mul_cur": 11}},
    "layers": [
        latent_2(3, 10, 6, 14, 18, 10, 0.3, base=50.0, scaling=(3.0, 16, 4.0, 0.5), mlp=moe(9, 2, 12, groups=(3, 1))),
        attention(3, 3, 10, 14, 0.3, rotation=rot(6, 50.0), mlp=dense(36)),
        latent(5, 6, 2, 18, 14, 0.4, mlp=moe(9, 2, 12, groups=(3, 1)), weights_of=None),
    ],
}
CONFIGS = {"A": CONFIG_A, "B": CONFIG_B, "C": CONFIG_C, "D": CONFIG_D}
PAGE_SIZE = {"A": 4, "B": 8, "C": 16, "D": 16}


def tensor_shapes(config: dict) -> Dict[str, tuple]:
    width = config["width"]
    shapes = {"embed": (config["vocab"], width), "head": (config["vocab"], width)}
    bigram = config.get("embedding", {}).get("bigram")
    if bigram:
        shapes["bigram"] = (bigram["buckets"] + 1, width)

    def norm(name):
        shapes[name], shapes[name + ".b"], shapes[name + ".alpha"] = (width,), (width,), ()

    norm("final.norm")
    for i, entry in enumerate(config["layers"]):
        if entry.get("weights_of") is not None:
            continue
        m, p = entry["mixer"], f"l{i}."
        norm(p + "norm1")
        if entry["type"] == "attention":
            for name, rows in (("q", m["heads"] * m["dim"]), ("k", m["kv_heads"] * m["dim"]), ("v", m["kv_heads"] * m["vdim"])):
                shapes[p + "mix." + name], shapes[p + "mix." + name + ".b"] = (rows, width), (rows,)
            shapes[p + "mix.o"] = (width, m["heads"] * m["vdim"])
        else:
            rot_dim = m.get("rot_dim", 0)
            shapes[p + "mix.dq"], shapes[p + "mix.dq.norm"] = (m["q_rank"], width), (m["q_rank"],)
            shapes[p + "mix.uq"] = (m["heads"] * (m["dim"] + rot_dim), m["q_rank"])
            shapes[p + "mix.dkv"], shapes[p + "mix.dkv.norm"] = (m["kv_rank"] + rot_dim, width), (m["kv_rank"],)
            shapes[p + "mix.uk"] = (m["heads"] * m["dim"], m["kv_rank"])
            shapes[p + "mix.uv"] = (m["heads"] * m["vdim"], m["kv_rank"])
            shapes[p + "mix.sink"], shapes[p + "mix.g"] = (m["heads"],), (m["heads"], width)
            shapes[p + "mix.o"] = (width, m["heads"] * m["vdim"])
        mlp = entry["mlp"]
        if mlp is None:
            continue
        norm(p + "norm2")
        if mlp["kind"] == "dense":
            shapes[p + "mlp.up"], shapes[p + "mlp.down"] = (mlp["ff"], width), (width, mlp["ff"])
        else:
            experts = mlp["router"]["experts"]
            shapes[p + "mlp.router"], shapes[p + "mlp.correction"] = (experts, width), (experts,)
            for e in range(experts):
                shapes[f"{p}mlp.e{e}.up"], shapes[f"{p}mlp.e{e}.down"] = (mlp["expert"]["ff"], width), (width, mlp["expert"]["ff"])
    return shapes


def random_weights(config: dict, seed: int, sharp: float = 3.0) -> Dict[str, torch.Tensor]:
    """float32 tensors: matrices N(0, 1 / fan-in), queries, keys, latents, routers and the head ``sharp`` times larger; norm weights
    1 + N(0, 0.1), their biases N(0, 0.1), their alphas between 0.4 and 0.8; sinks N(0, 1.5); corrections around -0.2, so
    that choice scores of both signs occur; the embedding N(0, 1) over the configuration's scale, the pair table N(0, 0.5)."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    scale = float(config.get("embedding", {}).get("scale", 1.0))
    for name, shape in tensor_shapes(config).items():
        if name.endswith(".alpha"):
            out[name] = 0.4 + 0.4 * torch.rand(shape, generator=g)
        elif name.endswith(".sink"):
            out[name] = 1.5 * torch.randn(shape, generator=g)
        elif name.endswith(".correction"):
            out[name] = -0.2 + 0.4 * torch.randn(shape, generator=g)
        elif name.endswith(".b"):
            out[name] = 0.1 * torch.randn(shape, generator=g)
        elif len(shape) == 1:
            out[name] = 1.0 + 0.1 * torch.randn(shape, generator=g)
        elif name == "embed":
            out[name] = torch.randn(shape, generator=g) / scale
        elif name == "bigram":
            out[name] = 0.5 * torch.randn(shape, generator=g)
        else:
            gain = sharp if name == "head" or name.endswith((".q", ".k", ".dq", ".uq", ".dkv", ".router", ".g")) else 1.0
            out[name] = torch.randn(shape, generator=g) * (gain / shape[1] ** 0.5)
    return out


def write_folder(path, config: dict, seed: int, dtype: str = "float32", weights: Optional[Dict[str, torch.Tensor]] = None) -> str:
    path = str(path)
    os.makedirs(path, exist_ok=True)
    weights = weights if weights is not None else random_weights(config, seed)
    storage = torch.float32 if dtype == "float32" else torch.bfloat16
    save_file({name: t.to(storage).contiguous() for name, t in weights.items()}, os.path.join(path, "model.safetensors"))
    with open(os.path.join(path, "config.json"), "w", encoding="utf-8") as handle:
        json.dump(config, handle)
    return path


def prompts(vocab: int, lengths, seed: int) -> Dict[str, List[int]]:
    g = torch.Generator().manual_seed(seed)
    return {f"r{i}": torch.randint(0, vocab, (n,), generator=g).tolist() for i, n in enumerate(lengths)}
