"""Small Gosulorn configurations and weights for the tests, written here from the design's tensor names and shapes
(not from the framework's tables, so that a wrong name or shape there shows).  The weights are sharp: attention is
peaked, decays lie between "forgets within a few tokens" and "keeps for hundreds", gates and step sizes are spread, the
streams' matrices are far from the identity.  A key that is lost, a window that is one off, a state that is not carried
or a stream that is mixed the wrong way round then changes the logits by far more than any tolerance."""
from __future__ import annotations

import json
import os
from typing import Dict, List, Optional

import torch
from safetensors.torch import save_file


def attention(heads, kv_heads, dim, vdim, scale, window=None, conv=None, rot=None) -> dict:
    """``rot``: (dims, base, factor or None)."""
    out = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if window is not None:
        out["mask"] = {"size": window}
    if conv is not None:
        out["conv"] = conv
    if rot is not None:
        out["rot"] = {"dims": rot[0], "base": rot[1]}
        if rot[2] is not None:
            out["rot"]["scaling"] = {"factor": rot[2]}
    return out


def delta(heads, kv_heads, dim, vdim, conv=None, rank=None, gate_rank=None) -> dict:
    """``rank`` / ``gate_rank``: inner sizes of the low-rank maps of the mixer on the right of a parallel layer (they are
    sizes that only tensors give; ``a1_rank`` / ``g1_rank`` stand for them where no folder is at hand)."""
    out = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim}
    if conv is not None:
        out["conv"] = conv
    if rank is not None:
        out["a1_rank"], out["g1_rank"] = rank, gate_rank
    return out


def gla(heads, dim, vdim, tau, rank) -> dict:
    return {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau, "a1_rank": rank}


def layer(kind: str, mixer: dict, ff: Optional[int], weights_of: Optional[int] = None) -> dict:
    out = {"type": kind, "mixer": mixer, "mlp": None if ff is None else {"kind": "dense", "ff": ff}}
    if weights_of is not None:
        out["weights_of"] = weights_of
    return out


def parallel(left: dict, right: dict, left_scale: float, right_scale: float) -> dict:
    return {"left": left, "right": right, "left_scale": left_scale, "right_scale": right_scale}


# Sizes that differ wherever two could be told apart: three streams, query/key heads wider and narrower than value heads,
# heads that are no multiple of 16, a window of 6 (smaller than a page of 8, larger than a page of 4), a rotation of part of a
# head with scaled positions, convolutions of 2, 3 and 4 taps, a layer without a feed-forward, two layers that run an
# earlier layer's weights again.
_A0 = parallel(attention(4, 2, 16, 8, 0.5, window=6, conv=3, rot=(8, 100.0, 2.0)), delta(4, 2, 8, 12, conv=2, rank=5, gate_rank=3), 0.7, 1.3)
_A1 = gla(2, 12, 20, 4.0, 6)
CONFIG_A = {
    "architecture": "Gosulorn", "vocab": 97, "width": 64, "norm": {"eps": 1e-5}, "streams": 3,
    "layers": [
        layer("parallel", _A0, 48),
        layer("gla", _A1, None),
        layer("delta", delta(4, 2, 16, 8, conv=4), 40),
        layer("parallel", _A0, 48, weights_of=0),
        layer("gla", _A1, None, weights_of=1),
    ],
}
# Nothing a multiple of 4, 8 or 16 where it need not be; no streams at all (the plain residual sum); attention without a
# window, without a convolution and with every channel rotated at unscaled positions; a recurrence without convolutions.
CONFIG_B = {
    "architecture": "Gosulorn", "vocab": 131, "width": 86, "norm": {"eps": 3e-6},
    "layers": [
        layer("delta", delta(3, 3, 10, 6), 22),
        layer("parallel", parallel(attention(3, 3, 10, 6, 0.6, rot=(10, 50.0, None)), delta(2, 1, 6, 10, conv=4, rank=3, gate_rank=7), 1.5, 0.6), 30),
        layer("gla", gla(3, 6, 14, 2.5, 4), 18),
    ],
}
# Sizes the kernels for decode-sized bfloat16 batches and the matrix cores take (multiples of 64 and 8), key heads of 128
# channels (a column of the state then spreads over sixteen lanes), two streams.
_C0 = parallel(attention(4, 2, 64, 32, 0.2, window=24, conv=4, rot=(32, 10000.0, 4.0)), delta(4, 4, 32, 64, conv=3, rank=16, gate_rank=8), 0.9, 1.2)
CONFIG_C = {
    "architecture": "Gosulorn", "vocab": 160, "width": 128, "norm": {"eps": 1e-5}, "streams": 2,
    "layers": [
        layer("gla", gla(2, 64, 64, 8.0, 16), 192),
        layer("parallel", _C0, 128),
        layer("delta", delta(4, 2, 128, 32, conv=4), 128),
        layer("parallel", _C0, 128, weights_of=1),
    ],
}
# What other configurations make differ is equal or 1 here: one stream (with its learned weights), one head everywhere, a
# window of one token, convolutions of one tap, both scales 1, tau 1, a rotation scaled by 1, inner sizes of 1.
CONFIG_D = {
    "architecture": "Gosulorn", "vocab": 64, "width": 48, "norm": {"eps": 1e-6}, "streams": 1,
    "layers": [
        layer("parallel", parallel(attention(1, 1, 16, 16, 0.4, window=1, conv=1, rot=(16, 10.0, 1.0)), delta(1, 1, 16, 16, conv=1, rank=1, gate_rank=1), 1.0, 1.0), 48),
        layer("gla", gla(1, 16, 16, 1.0, 1), 16),
        layer("delta", delta(1, 1, 48, 48, conv=1), None),
    ],
}
# No layer keeps pages: every mixer's memory is a state of fixed size.
CONFIG_E = {
    "architecture": "Gosulorn", "vocab": 80, "width": 32, "norm": {"eps": 1e-5}, "streams": 2,
    "layers": [
        layer("gla", gla(2, 8, 8, 3.0, 4), 24),
        layer("delta", delta(2, 1, 8, 12, conv=3), 24),
        layer("gla", gla(2, 8, 8, 3.0, 4), 24, weights_of=0),
    ],
}
CONFIGS = {"A": CONFIG_A, "B": CONFIG_B, "C": CONFIG_C, "D": CONFIG_D, "E": CONFIG_E}
PAGE_SIZE = {"A": 4, "B": 8, "C": 16, "D": 16, "E": 4}


def _recurrence_shapes(shapes: dict, p: str, m: dict, width: int, kind: str) -> None:
    heads, dim, vdim = m["heads"], m["dim"], m["vdim"]
    kv_heads = m.get("kv_heads", heads)
    shapes[p + "q"], shapes[p + "k"], shapes[p + "v"] = (kv_heads * dim, width), (kv_heads * dim, width), (heads * vdim, width)
    shapes[p + "o"], shapes[p + "norm"] = (width, heads * vdim), (vdim,)
    if m.get("conv"):
        for name, rows in (("q", kv_heads * dim), ("k", kv_heads * dim), ("v", heads * vdim)):
            shapes[p + name + ".conv"] = (rows, m["conv"])
    if kind == "gla":
        shapes[p + "g"] = (heads * vdim, width)
        shapes[p + "a1"], shapes[p + "a2"], shapes[p + "a2.b"] = (m["a1_rank"], width), (heads * dim, m["a1_rank"]), (heads * dim,)
        return
    shapes[p + "b"], shapes[p + "A_log"] = (heads, width), (heads,)
    if kind == "delta":
        shapes[p + "a"], shapes[p + "dt_bias"], shapes[p + "g"] = (heads, width), (heads,), (heads * vdim, width)
    else:
        shapes[p + "a1"], shapes[p + "a2"], shapes[p + "dt_bias"] = (m["a1_rank"], width), (heads * dim, m["a1_rank"]), (heads * dim,)
        shapes[p + "g1"], shapes[p + "g2"] = (m["g1_rank"], width), (heads * vdim, m["g1_rank"])


def tensor_shapes(config: dict) -> Dict[str, tuple]:
    width, streams = config["width"], config.get("streams")
    shapes = {"embed": (config["vocab"], width), "final.norm": (width,)}
    for i, entry in enumerate(config["layers"]):
        if entry.get("weights_of") is not None:
            continue
        m, p = entry["mixer"], f"l{i}."
        shapes[p + "norm1"] = (width,)
        if entry["type"] == "parallel":
            left, q = m["left"], p + "mix.left."
            for name, rows in (("q", left["heads"] * left["dim"]), ("k", left["kv_heads"] * left["dim"]), ("v", left["kv_heads"] * left["vdim"])):
                shapes[q + name], shapes[q + name + ".b"] = (rows, width), (rows,)
                if left.get("conv"):
                    shapes[q + name + ".conv"] = (rows, left["conv"])
            shapes[q + "o"], shapes[q + "o.b"] = (width, left["heads"] * left["vdim"]), (width,)
            _recurrence_shapes(shapes, p + "mix.right.", m["right"], width, "parallel")
        else:
            _recurrence_shapes(shapes, p + "mix.", m, width, entry["type"])
        numbers = [1]
        if entry["mlp"] is not None:
            ff = entry["mlp"]["ff"]
            shapes[p + "norm2"] = (width,)
            shapes[p + "mlp.gate"], shapes[p + "mlp.up"], shapes[p + "mlp.down"] = (ff, width), (ff, width), (width, ff)
            numbers.append(2)
        if streams:
            for n in numbers:
                shapes[f"{p}hc{n}.in"], shapes[f"{p}hc{n}.out"], shapes[f"{p}hc{n}.mix"] = (streams,), (streams,), (streams, streams)
    return shapes


def random_weights(config: dict, seed: int) -> Dict[str, torch.Tensor]:
    """float32 tensors.  Matrices N(0, gain / fan-in) with larger gains where a decision is taken (q and k of the attention:
    peaked weights; gates, decays, beta: spread over their range); convolution taps around +-0.6; ``A_log`` so that rates
    lie between 0.05 and 2; biases of the decays spread; the streams' weights far from identity and average; norm weights
    1 + N(0, 0.1); the embedding N(0, 1)."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(config).items():
        last = name.rsplit(".", 1)[-1]
        if name.endswith(".conv"):
            out[name] = 0.6 * torch.randn(shape, generator=g)
        elif last == "A_log":
            out[name] = torch.log(0.05 + 1.95 * torch.rand(shape, generator=g))
        elif last == "dt_bias" or name.endswith(".a2.b"):
            out[name] = 1.5 * torch.randn(shape, generator=g)
        elif last == "in" and ".hc" in name:
            out[name] = 1.0 / shape[0] + 0.4 * torch.randn(shape, generator=g)
        elif last == "out" and ".hc" in name:
            out[name] = 1.0 + 0.4 * torch.randn(shape, generator=g)
        elif last == "mix" and ".hc" in name:
            out[name] = 0.8 * torch.eye(shape[0]) + 0.3 * torch.randn(shape, generator=g)
        elif name.endswith(".b") and len(shape) == 1:
            out[name] = 0.3 * torch.randn(shape, generator=g)
        elif len(shape) == 1:
            out[name] = 1.0 + 0.1 * torch.randn(shape, generator=g)
        elif name == "embed":
            out[name] = torch.randn(shape, generator=g)
        else:
            gain = 1.0
            if ".left." in name and last in ("q", "k"):
                gain = 3.0
            elif last in ("b", "a", "a2", "g", "g2", "gate", "up"):
                gain = 2.5
            out[name] = torch.randn(shape, generator=g) * (gain / shape[1] ** 0.5)
    return out


def write_folder(path, config: dict, seed: int, dtype: str = "float32", weights: Optional[Dict[str, torch.Tensor]] = None, strip: bool = True) -> str:
    """``strip``: the written configuration does not state the inner sizes of the low-rank maps, as a folder from
    elsewhere would not: the reader has to take them from the tensors' shapes."""
    path = str(path)
    os.makedirs(path, exist_ok=True)
    weights = weights if weights is not None else random_weights(config, seed)
    storage = torch.float32 if dtype == "float32" else torch.bfloat16
    save_file({name: t.to(storage).contiguous() for name, t in weights.items()}, os.path.join(path, "model.safetensors"))
    written = json.loads(json.dumps(config))
    if strip:
        for entry in written["layers"]:
            for mixer in (entry["mixer"], entry["mixer"].get("right", {})):
                mixer.pop("a1_rank", None)
                mixer.pop("g1_rank", None)
    with open(os.path.join(path, "config.json"), "w", encoding="utf-8") as handle:
        json.dump(written, handle)
    return path


def read_folder(path):
    """-> (configuration, float64 tensors) for the plain model."""
    from safetensors.torch import load_file

    with open(os.path.join(path, "config.json"), "r", encoding="utf-8") as handle:
        config = json.load(handle)
    return config, {name: t.double() for name, t in load_file(os.path.join(path, "model.safetensors")).items()}


def prompts(vocab: int, lengths, seed: int) -> Dict[str, List[int]]:
    g = torch.Generator().manual_seed(seed)
    return {f"r{i}": torch.randint(0, vocab, (n,), generator=g).tolist() for i, n in enumerate(lengths)}
