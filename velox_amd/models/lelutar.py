"""Lelutar as a ``ModelSpec``.

A pre-norm decoder (``x += mixer(norm1(x)); x += ff(norm2(x))``) whose norms take no statistics (``tanh(alpha x) w + b``,
``parts.norms.DynamicTanhNorm``), whose embedding is scaled and adds a row of a hashed table of (previous token, token)
pairs (``parts.model.BigramEmbedding``), and whose logits are scaled.  ``config.json`` lists the layers one by one, each with
its type and sizes, so layers may differ in everything; a layer that says ``weights_of: j`` is layer ``j``'s block run again
with a cache of its own.  Three types of layer:

``attention``
    grouped-query softmax attention with biases on q, k and v, separate sizes of key and value heads, a rotation of the
    first ``rot.dims`` channels of every head in pairs ``(2i, 2i + 1)`` with stretched frequencies, and the score scale of
    the configuration (``parts.conv_attention`` without its convolution).
``latent_attention``
    attention over a cached low-rank latent without positions (``parts.latent_attention`` with ``rot_dim`` = 0): queries
    through a normed latent of their own, a learned sink in the softmax's denominator, a sigmoid gate per head.
``latent_attention_2``
    the same with one rotated key part that all heads share beside the latent.

The feed-forward is ``W_down relu(W_up h)^2``, dense or as a mixture of experts with sigmoid scores, a correction that is
added for the choice only, a choice among the experts of the best groups, and chosen scores divided by their sum
(+ 1e-20), or absent.

Tensor names: ``embed``, ``bigram``, ``head``, ``final.norm{,.b,.alpha}``, and per layer ``l<i>.norm{1,2}{,.b,.alpha}``,
``l<i>.mix.{q,k,v}{,.b}``, ``l<i>.mix.o`` or ``l<i>.mix.{dq,dq.norm,uq,dkv,dkv.norm,uk,uv,sink,g,o}``, ``l<i>.mlp.{up,down}``
or ``l<i>.mlp.{router,correction,e<k>.up,e<k>.down}``.  What the design fixes is fixed here: the squared rectifier, sigmoid
scores with renormalisation, the sum's floor, softmax over all keys at or before the query, the pairs' layout.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

from ..config.model_config import ConfigError, ModelConfig, require
from ..config.registry import architecture_name, register_architecture
from ..parts import LayerSpec, ModelSpec, PartSpec, ScheduleEntry

# positions an engine is given when its caller names no limit (the configuration has none)
DEFAULT_MAX_POSITION = 1 << 17
RENORMALIZE_FLOOR = 1e-20  # added to the sum of the chosen scores before they are divided by it

_LATENT_NAMES = (("q_down", "dq"), ("q_norm", "dq.norm"), ("q_up", "uq"), ("down", "dkv"), ("down_norm", "dkv.norm"), ("up_k", "uk"), ("up_v", "uv"),
                 ("gate", "g"), ("out", "o"), ("sink", "sink"))
_TYPES = ("attention", "latent_attention", "latent_attention_2")


def _section(raw: Dict[str, Any], key: str, where: str) -> Dict[str, Any]:
    value = raw.get(key)
    if not isinstance(value, dict):
        raise ConfigError(f"config.json: {where}{key!r} must be an object")
    return value


def _rotation(mixer: Dict[str, Any], where: str, limit: int) -> Optional[tuple]:
    """``(dims, base, stretch or None)`` of a mixer's ``rot`` entry, or None when it has none."""
    rot = mixer.get("rot")
    if rot is None:
        return None
    if not isinstance(rot, dict):
        raise ConfigError(f"{where}rot must be an object")
    dims, base = require(rot, "dims", int), require(rot, "base", float)
    if dims <= 0 or dims % 2 or dims > limit or base <= 0:
        raise ConfigError(f"{where}rot: dims={dims} must be even, positive and at most {limit}; base must be positive")
    stretch = None
    if rot.get("scaling") is not None:
        stretch = tuple(require(rot["scaling"], key, float) for key in ("factor", "original", "fast", "slow"))
        if min(stretch) <= 0:
            raise ConfigError(f"{where}rot.scaling: factor, original, fast and slow must be positive")
    return dims, base, stretch


def _feed_forward(mlp: Optional[Dict[str, Any]], where: str) -> Optional[Dict[str, Any]]:
    if mlp is None:
        return None
    kind = mlp.get("kind")
    if kind == "dense":
        out = {"kind": "dense", "ff": require(mlp, "ff", int)}
    elif kind == "moe":
        router = _section(mlp, "router", where + "mlp.")
        out = {"kind": "moe", "ff": require(_section(mlp, "expert", where + "mlp."), "ff", int), "experts": require(router, "experts", int),
               "top": require(router, "top", int), "groups": None}
        if not 1 <= out["top"] <= out["experts"]:
            raise ConfigError(f"{where}mlp.router: top={out['top']} must lie between 1 and experts={out['experts']}")
        if router.get("groups") is not None:
            count, keep = require(router["groups"], "count", int), require(router["groups"], "keep", int)
            if count < 1 or out["experts"] % count or not 1 <= keep <= count or keep * (out["experts"] // count) < out["top"]:
                raise ConfigError(f"{where}mlp.router.groups: {out['experts']} experts must form {count} equal groups, of which the {keep} kept must "
                                  f"hold at least top={out['top']} experts")
            out["groups"] = (count, keep)
    else:
        raise ConfigError(f"{where}mlp.kind={kind!r} is not a feed-forward of this design ('dense' or 'moe')")
    if out["ff"] <= 0:
        raise ConfigError(f"{where}mlp: ff must be positive")
    return out


@dataclass
class LelutarConfig(ModelConfig):
    width: int = 0
    vocab: int = 0
    norm_eps: float = 0.0
    embedding_scale: float = 1.0
    bigram: Optional[tuple] = None  # (buckets, mul_prev, mul_cur)
    logit_scale: float = 1.0
    layers: List[Dict[str, Any]] = field(default_factory=list)  # validated copies of the entries; "owner" = whose tensors a layer runs

    @staticmethod
    def from_dict(raw: Dict[str, Any]) -> "LelutarConfig":
        width, vocab = require(raw, "width", int), require(raw, "vocab", int)
        eps = require(_section(raw, "norm", ""), "eps", float)
        if width <= 0 or vocab <= 0 or eps <= 0:
            raise ConfigError("width, vocab and norm.eps must be positive")
        embedding = raw.get("embedding") or {}
        scale = float(embedding.get("scale", 1.0))
        bigram = None
        if embedding.get("bigram") is not None:
            bigram = tuple(require(embedding["bigram"], key, int) for key in ("buckets", "mul_prev", "mul_cur"))
            if not 1 <= bigram[0] < 2 ** 31:
                raise ConfigError("embedding.bigram: buckets must be positive (and below 2^31)")
        listed = raw.get("layers")
        if not isinstance(listed, list) or not listed:
            raise ConfigError("config.json: 'layers' must list at least one layer")
        layers: List[Optional[Dict[str, Any]]] = [None] * len(listed)
        # whose tensors a layer runs: itself, or the layer its ``weights_of`` names (followed to a layer that owns tensors)
        owners: List[int] = []
        for index, entry in enumerate(listed):
            if not isinstance(entry, dict) or entry.get("type") not in _TYPES:
                raise ConfigError(f"layers[{index}].type={entry.get('type') if isinstance(entry, dict) else entry!r} is not a layer of this design ({', '.join(_TYPES)})")
            owner, seen = index, set()
            while listed[owner].get("weights_of") is not None:
                seen.add(owner)
                owner = int(listed[owner]["weights_of"])
                if not 0 <= owner < len(listed) or owner in seen or not isinstance(listed[owner], dict):
                    raise ConfigError(f"layers[{index}].weights_of must lead to a layer that owns its tensors")
            if listed[owner].get("type") != entry["type"]:
                raise ConfigError(f"layers[{index}].a layer that runs layer {owner}'s weights is of its type")
            owners.append(owner)
        for index, entry in enumerate(listed):
            where = f"layers[{index}]."
            kind = entry["type"]
            if owners[index] != index:
                continue
            mixer = _section(entry, "mixer", where)
            keys = ("heads", "kv_heads", "dim", "vdim") if kind == "attention" else ("heads", "dim", "vdim", "kv_rank", "q_rank")
            sizes = {key: require(mixer, key, int) for key in keys}
            if kind == "latent_attention_2":
                sizes["rot_dim"] = require(mixer, "rot_dim", int)
            if min(sizes.values()) <= 0:
                raise ConfigError(f"{where}mixer: {', '.join(sizes)} must be positive")
            if kind == "attention" and sizes["heads"] % sizes["kv_heads"]:
                raise ConfigError(f"{where}mixer: heads={sizes['heads']} must be a multiple of kv_heads={sizes['kv_heads']}")
            rotation = None
            if kind != "latent_attention":
                rotation = _rotation(mixer, where + "mixer.", sizes["dim"] if kind == "attention" else sizes["rot_dim"])
            if kind == "latent_attention_2" and rotation is None:
                raise ConfigError(f"{where}mixer: a layer with a rotated key part states its rotation ('rot')")
            parsed = {"type": kind, "owner": index, "sizes": sizes, "scale": require(mixer, "scale", float), "rotation": rotation,
                      "mlp": _feed_forward(entry.get("mlp"), where)}
            if not parsed["scale"] > 0:
                raise ConfigError(f"{where}mixer.scale must be positive")
            layers[index] = parsed
        for index, owner in enumerate(owners):
            if owner != index:
                layers[index] = dict(layers[owner], owner=owner)
        return LelutarConfig(architecture=architecture_name(raw), raw=dict(raw), width=width, vocab=vocab, norm_eps=eps, embedding_scale=scale,
                             bigram=bigram, logit_scale=float(raw.get("logit_scale", 1.0)), layers=layers)

    def to_json_dict(self) -> Dict[str, Any]:
        return dict(self.raw)


def lelutar_spec(config: LelutarConfig, max_position: Optional[int] = None) -> ModelSpec:
    max_position = int(max_position or DEFAULT_MAX_POSITION)
    width = config.width
    norm = PartSpec.of("dynamic_tanh", hidden_size=width, weight_name="", bias_name=".b", alpha_name=".alpha")
    positions: Dict[str, PartSpec] = {}
    key_of: Dict[tuple, str] = {}
    layers: List[LayerSpec] = []
    schedule: List[ScheduleEntry] = []
    owning = [index for index, layer in enumerate(config.layers) if layer["owner"] == index]
    place: Dict[int, int] = {index: at for at, index in enumerate(owning)}  # configuration index of a weight-owning layer -> its place in ``layers``
    for index, layer in enumerate(config.layers):
        schedule.append(ScheduleEntry(place[layer["owner"]]))
    for index in owning:
        layer = config.layers[index]
        position = None
        if layer["rotation"] is not None:
            if layer["rotation"] not in key_of:  # layers with the same rotation share its tables
                key_of[layer["rotation"]] = f"rotation{len(key_of)}"
                dims, base, stretch = layer["rotation"]
                positions[key_of[layer["rotation"]]] = PartSpec.of("rotary", rotary_dim=dims, theta=base, max_position=max_position, layout="interleaved",
                                                                   stretch=stretch)
            position = key_of[layer["rotation"]]
        sizes = layer["sizes"]
        if layer["type"] == "attention":
            mixer = PartSpec.of("conv_attention", hidden_size=width, num_heads=sizes["heads"], num_kv_heads=sizes["kv_heads"], dim=sizes["dim"],
                                vdim=sizes["vdim"], scale=layer["scale"], window=None, conv_taps=0, qkv_bias=True, out_bias=False)
        else:
            mixer = PartSpec.of("latent_attention", hidden_size=width, num_heads=sizes["heads"], dim=sizes["dim"], rot_dim=sizes.get("rot_dim", 0),
                                vdim=sizes["vdim"], kv_rank=sizes["kv_rank"], q_rank=sizes["q_rank"], scale=layer["scale"], norm_eps=config.norm_eps,
                                gate="head", sink=True, own_latent=True, names=_LATENT_NAMES)
        mlp = layer["mlp"]
        if mlp is None:
            feed_forward = PartSpec.of("none")
        elif mlp["kind"] == "dense":
            feed_forward = PartSpec.of("plain_mlp", hidden_size=width, intermediate_size=mlp["ff"], activation="relu2", names=("up", "down"))
        else:
            feed_forward = PartSpec.of("routed_experts", hidden_size=width, intermediate_size=mlp["ff"], num_experts=mlp["experts"], top=mlp["top"],
                                       score="sigmoid", renormalize=True, renormalize_floor=RENORMALIZE_FLOOR, scale_input=False, ungated="relu2",
                                       groups=mlp["groups"], expert_names=("e{e}.up", "e{e}.down"), router_name="router", correction_name="correction")
        layers.append(LayerSpec(prefix=f"l{index}.", mixer=mixer, feed_forward=feed_forward, mixer_norm=norm, ff_norm=norm, position=position,
                                arrangement="pre_norm", mixer_prefix="mix.", feed_forward_prefix="mlp.", mixer_norm_prefix="norm1", ff_norm_prefix="norm2"))
    if config.bigram is not None:
        embedding = PartSpec.of("bigram_table", scale=config.embedding_scale, buckets=config.bigram[0], mul_prev=config.bigram[1], mul_cur=config.bigram[2],
                                bigram_name="bigram")
    else:
        embedding = PartSpec.of("table", scale=config.embedding_scale)
    return ModelSpec(vocab_size=config.vocab, hidden_size=width, max_position=max_position, layers=layers, schedule=schedule, final_norm=norm,
                     positions=positions, tie_head=False, embed_name="embed", head_name="head", final_norm_prefix="final.norm", eos_token_ids=(),
                     embedding=embedding, head=PartSpec.of("linear", scale=config.logit_scale))


register_architecture("Lelutar", LelutarConfig.from_dict, lelutar_spec)
