"""Gosulorn as a ``ModelSpec``.

A decoder of pre-norm layers (layer norm with a weight and no bias), optionally over several residual streams
(hyper-connections, ``parts.block.HyperConnectionBlock``), whose mixers keep a state of fixed size.  ``config.json``
lists the layers one by one; a layer is one of

``parallel``  two mixers side by side on the same input (``parts.parallel_mixer``): on the left softmax attention over a
              sliding window with biases, a short convolution on q, k and v, a rotation of part of each head with
              linearly scaled positions (``parts.conv_attention``); on the right a gated delta rule with a decay per
              head and key channel and a low-rank sigmoid gate; the result is ``left_scale * left + right_scale * right``;
``gla``       gated linear attention: ``S <- diag(alpha) S + k v^T`` with ``alpha = sigmoid(z)^(1 / tau)`` per key channel;
``delta``     a gated delta rule with one decay per head and a SiLU gate

(the last three are ``parts.linear_recurrence`` with other options), each followed by a dense feed-forward with the
tanh form of GELU on its gate branch, or by none.  A layer that says ``weights_of: j`` owns no tensors: it is layer
``j``'s block run again, with a cache and state of its own (the schedule names the layer twice).  The output head is
the embedding table.  There is no position limit in the configuration, so ``max_position`` is the caller's.

Tensor names: ``embed``, ``final.norm``, per layer ``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.hc{1,2}.{in,out,mix}``,
``l<i>.mlp.{gate,up,down}`` and ``l<i>.mix.*`` as the mixers' parts name them (``left.`` / ``right.`` below a parallel
layer's).  What the design fixes is fixed in the parts' options chosen here: SiLU behind the convolutions of the
recurrent mixers and none behind the attention's, unit q and k for the delta rules, q times ``dim ** -0.5``.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

from ..config.model_config import ConfigError, ModelConfig, require
from ..config.registry import architecture_name, register_architecture
from ..parts import LayerSpec, ModelSpec, PartSpec, ScheduleEntry

# positions an engine is given when its caller names no limit (the configuration has none)
DEFAULT_MAX_POSITION = 1 << 17
_LAYER_KINDS = ("parallel", "gla", "delta")


def _section(raw: Dict[str, Any], key: str, where: str) -> Dict[str, Any]:
    value = raw.get(key)
    if not isinstance(value, dict):
        raise ConfigError(f"config.json: {where}{key!r} must be an object")
    return value


def _sizes(mixer: Dict[str, Any], where: str, kv_heads_default_to_heads: bool = False) -> Dict[str, int]:
    sizes = {key: require(mixer, key, int) for key in ("heads", "dim", "vdim")}
    sizes["kv_heads"] = int(mixer["kv_heads"]) if "kv_heads" in mixer or not kv_heads_default_to_heads else sizes["heads"]
    if min(sizes.values()) <= 0 or sizes["heads"] % sizes["kv_heads"]:
        raise ConfigError(f"{where}: heads, kv_heads, dim and vdim must be positive and heads a multiple of kv_heads")
    return sizes


def _attention(mixer: Dict[str, Any], where: str) -> Dict[str, Any]:
    out: Dict[str, Any] = dict(_sizes(mixer, where))
    out["scale"] = require(mixer, "scale", float)
    if not out["scale"] > 0:
        raise ConfigError(f"{where}.scale must be positive")
    out["conv"] = int(mixer.get("conv") or 0)
    mask = mixer.get("mask")
    out["window"] = None
    if mask is not None:
        out["window"] = require(_section(mixer, "mask", where + "."), "size", int)
        if out["window"] < 1:
            raise ConfigError(f"{where}.mask.size must be at least 1")
    out["rot"] = None
    if mixer.get("rot") is not None:
        rot = _section(mixer, "rot", where + ".")
        dims, base = require(rot, "dims", int), require(rot, "base", float)
        factor = 1.0
        if rot.get("scaling") is not None:
            factor = require(_section(rot, "scaling", where + ".rot."), "factor", float)
        if dims < 0 or dims % 2 or dims > out["dim"] or not base > 0 or not factor > 0:
            raise ConfigError(f"{where}.rot: dims must be even and at most dim, base and scaling.factor positive")
        if dims:
            out["rot"] = (dims, base, factor)
    return out


def _recurrent(mixer: Dict[str, Any], where: str, kind: str) -> Dict[str, Any]:
    out: Dict[str, Any] = dict(_sizes(mixer, where, kv_heads_default_to_heads=True))
    out["conv"] = int(mixer.get("conv") or 0)
    if kind == "gla":
        out["tau"] = require(mixer, "tau", float)
        if not out["tau"] > 0:
            raise ConfigError(f"{where}.tau must be positive")
        if out["kv_heads"] != out["heads"]:
            raise ConfigError(f"{where}: gated linear attention has as many q/k heads as value heads")
    return out


@dataclass
class GosulornConfig(ModelConfig):
    width: int = 0
    vocab: int = 0
    norm_eps: float = 0.0
    streams: int = 1
    layers: List[Dict[str, Any]] = field(default_factory=list)  # validated copies of the configuration's entries

    @staticmethod
    def from_dict(raw: Dict[str, Any]) -> "GosulornConfig":
        width, vocab = require(raw, "width", int), require(raw, "vocab", int)
        eps = require(_section(raw, "norm", ""), "eps", float)
        streams = int(raw.get("streams") or 1)  # (no such key: one residual, no weights on it)
        if width <= 0 or vocab <= 0 or eps <= 0 or streams < 1:
            raise ConfigError("width, vocab, norm.eps and streams must be positive")
        listed = raw.get("layers")
        if not isinstance(listed, list) or not listed:
            raise ConfigError("config.json: 'layers' must list at least one layer")
        shapes = raw.get("tensor_shapes") or {}
        layers: List[Dict[str, Any]] = []
        for index, entry in enumerate(listed):
            where = f"layers[{index}]"
            kind = entry.get("type")
            if kind not in _LAYER_KINDS:
                raise ConfigError(f"{where}.type={kind!r} is not a layer of this design ({', '.join(_LAYER_KINDS)})")
            mixer = _section(entry, "mixer", where + ".")
            owner = entry.get("weights_of")
            if owner is not None:
                owner = int(owner)
                if not 0 <= owner < index or layers[owner]["owner"] != owner:
                    raise ConfigError(f"{where}.weights_of must name an earlier layer that owns its tensors")
                if layers[owner]["kind"] != kind:
                    raise ConfigError(f"{where}: a layer that runs layer {owner}'s weights is of its type")
                layers.append(dict(layers[owner], owner=owner))
                continue
            prefix = f"l{index}.mix."
            parsed: Dict[str, Any] = {"kind": kind, "owner": index}
            if kind == "parallel":
                parsed["left"] = _attention(_section(mixer, "left", where + ".mixer."), where + ".mixer.left")
                parsed["right"] = _recurrent(_section(mixer, "right", where + ".mixer."), where + ".mixer.right", "parallel")
                parsed["right"]["ranks"] = _ranks(shapes, mixer["right"], prefix + "right.", ("a1", "g1"), where + ".mixer.right")
                parsed["left_scale"], parsed["right_scale"] = float(mixer.get("left_scale", 1.0)), float(mixer.get("right_scale", 1.0))
            else:
                parsed["mixer"] = _recurrent(mixer, where + ".mixer", kind)
                if kind == "gla":
                    parsed["mixer"]["ranks"] = _ranks(shapes, mixer, prefix, ("a1",), where + ".mixer")
            mlp = entry.get("mlp")
            parsed["ff"] = None
            if mlp is not None:
                if mlp.get("kind") != "dense":
                    raise ConfigError(f"{where}.mlp.kind={mlp.get('kind')!r} is not a feed-forward of this design (only 'dense')")
                parsed["ff"] = require(mlp, "ff", int)
                if parsed["ff"] <= 0:
                    raise ConfigError(f"{where}.mlp.ff must be positive")
            layers.append(parsed)
        return GosulornConfig(architecture=architecture_name(raw), raw=dict(raw), width=width, vocab=vocab, norm_eps=eps, streams=streams, layers=layers)

    def to_json_dict(self) -> Dict[str, Any]:
        return {key: value for key, value in self.raw.items() if key != "tensor_shapes"}


def _ranks(shapes: Dict[str, Any], mixer: Dict[str, Any], prefix: str, maps, where: str) -> Dict[str, int]:
    """The inner sizes of a mixer's low-rank maps: sizes that only the tensors' shapes give (rows of ``a1`` / ``g1``).  A
    folder's reader notes the shapes under ``tensor_shapes``; a configuration without a folder states ``<map>_rank``."""
    out = {}
    for name in maps:
        if prefix + name in shapes:
            out[name] = int(shapes[prefix + name][0])
        elif mixer.get(name + "_rank") is not None:
            out[name] = int(mixer[name + "_rank"])
        else:
            raise ConfigError(f"{where}: the inner size of the low-rank map is the first size of tensor {prefix + name!r}; "
                              f"read the configuration from a model folder or state '{name}_rank'")
        if out[name] < 1:
            raise ConfigError(f"{where}: the low-rank map {name!r} needs a positive inner size")
    return out


def _recurrence_spec(config: GosulornConfig, sizes: Dict[str, Any], kind: str) -> PartSpec:
    common = dict(hidden_size=config.width, num_heads=sizes["heads"], num_kv_heads=sizes["kv_heads"], dim=sizes["dim"], vdim=sizes["vdim"],
                  norm_eps=config.norm_eps, conv_taps=sizes["conv"])
    if kind == "gla":
        return PartSpec.of("linear_recurrence", rule="additive", decay="sigmoid_channel", gate="silu", unit_qk=False, tau=sizes["tau"],
                           decay_rank=sizes["ranks"]["a1"], **common)
    if kind == "delta":
        return PartSpec.of("linear_recurrence", rule="delta", decay="head", gate="silu", unit_qk=True, qkv_silu=True, **common)
    return PartSpec.of("linear_recurrence", rule="delta", decay="channel", gate="sigmoid_low_rank", unit_qk=True, qkv_silu=True,
                       decay_rank=sizes["ranks"]["a1"], gate_rank=sizes["ranks"]["g1"], **common)


def gosulorn_spec(config: GosulornConfig, max_position: Optional[int] = None) -> ModelSpec:
    max_position = int(max_position or DEFAULT_MAX_POSITION)
    width, streams = config.width, config.streams
    norm = PartSpec.of("stream_norm", hidden_size=width, eps=config.norm_eps, weight_name="", streams=streams, center=True)
    layers: List[LayerSpec] = []
    schedule: List[ScheduleEntry] = []
    positions: Dict[str, PartSpec] = {}
    place: Dict[int, int] = {}  # configuration index of a weight-owning layer -> its place in ``layers``
    for index, layer in enumerate(config.layers):
        if layer["owner"] != index:
            schedule.append(ScheduleEntry(place[layer["owner"]]))
            continue
        position = None
        if layer["kind"] == "parallel":
            left = layer["left"]
            if left["rot"] is not None:
                dims, base, factor = left["rot"]
                position = f"rot_{dims}_{base!r}_{factor!r}"
                positions.setdefault(position, PartSpec.of("rotary", rotary_dim=dims, theta=base, max_position=max_position, scaling_factor=factor,
                                                           exact_angles=True))
            attention = PartSpec.of("conv_attention", hidden_size=width, num_heads=left["heads"], num_kv_heads=left["kv_heads"], dim=left["dim"],
                                    vdim=left["vdim"], scale=left["scale"], window=left["window"], conv_taps=left["conv"], qkv_bias=True, out_bias=True)
            mixer = PartSpec.of("parallel_mixers", left=attention, right=_recurrence_spec(config, layer["right"], "parallel"),
                                left_scale=layer["left_scale"], right_scale=layer["right_scale"])
        else:
            mixer = _recurrence_spec(config, layer["mixer"], layer["kind"])
        if layer["ff"] is None:
            feed_forward = PartSpec.of("none")
        else:
            feed_forward = PartSpec.of("gated_mlp", hidden_size=width, intermediate_size=layer["ff"], activation="gelu_tanh", names=("gate", "up", "down"))
        place[index] = len(layers)
        layers.append(LayerSpec(prefix=f"l{index}.", mixer=mixer, feed_forward=feed_forward, mixer_norm=norm, ff_norm=norm, position=position,
                                arrangement="hyper_connection", arrangement_args=(("learned", config.raw.get("streams") is not None), ("streams", streams)),
                                mixer_prefix="mix.", feed_forward_prefix="mlp.", mixer_norm_prefix="norm1", ff_norm_prefix="norm2"))
        schedule.append(ScheduleEntry(place[index]))
    return ModelSpec(vocab_size=config.vocab, hidden_size=width, max_position=max_position, layers=layers, schedule=schedule, final_norm=norm,
                     positions=positions, tie_head=True, embed_name="embed", head_name="head", final_norm_prefix="final.norm", eos_token_ids=(),
                     residual_streams=streams)


register_architecture("Gosulorn", GosulornConfig.from_dict, gosulorn_spec, reads_tensor_shapes=True)
