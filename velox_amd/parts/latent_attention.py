"""Attention over a cached low-rank latent.

Per token one vector of ``kv_rank`` numbers (the latent ``c``, RMS-normed) and one rotated key part of
``rot_dim`` numbers that all heads share are kept in the cache; nothing per head is.  With
``q_h = [a_h ; b_h]`` (``dim`` plain and ``rot_dim`` rotated channels), keys ``[U_h c ; r]`` and values
``V_h c``::

    score_h(t, j) = (a_h(t) . U_h c_j + b_h(t) . r_j) * scale
                  = ([U_h^T a_h(t) ; b_h(t)] . [c_j ; r_j]) * scale
    out_h(t)      = V_h (sum_j p_h(t, j) c_j)

so every head attends over the SAME cached vectors ``[c_j ; r_j]``: the step's queries are taken through ``U_h^T``
once (a product per head over the step's tokens only), the paged attention kernels run with one key/value head
whose "values" are the cached vectors themselves, and the result is taken through ``V_h``.  The cache is read as it
stands, whatever the number of heads; keys and values per head are never formed.

The cached vector is padded with zeros to a multiple of 16 channels (the attention kernels' tile; beyond 256 channels a
plain kernel of any size takes their place), and is held
twice, as keys ``[page, 1, offset, D]`` and transposed as values ``[page, 1, D, offset]``, the layout those
kernels read (``parts.attention.kv_pages``).

Options of the part: a sigmoid gate on the concatenated heads (``gate``: one number per channel, or ``"head"``: one per
head), and ``own_latent`` = False for a layer
that makes no latent of its own and reads another schedule entry's cache (``ScheduleEntry.cache_from``) with its
own ``U``, ``V``, queries and output product.  The rotation (which channels pair up, the frequencies, a factor on
cos and sin) is the position encoding's; it is applied to the first ``2 * table width`` channels of the rotated part;
``rot_dim`` = 0 is attention without positions.  ``q_rank``: the queries pass a latent of their own,
``q = W_uq rmsnorm(W_dq x)``, the norm in float32 inside the kernel that writes the cache.  ``sink``: a learned number per
head whose exponential joins the softmax's denominator (it has no key and no value and is not scaled).
"""
from __future__ import annotations

from typing import Dict, Optional, Tuple

import torch

from .attention import SHORT_CONTEXT_KEYS, kv_pages
from .base import Mixer, Param, PositionEncoding, fused_rows, register_part, single

_NAMES = {"q": "q.weight", "down": "down.weight", "down_norm": "down_norm.weight", "up_k": "up_k.weight", "up_v": "up_v.weight",
          "gate": "gate.weight", "out": "out.weight", "q_down": "q_down.weight", "q_norm": "q_norm.weight", "q_up": "q_up.weight", "sink": "sink"}


class LatentAttentionMixer(Mixer):
    def __init__(self, prefix: str, hidden_size: int, num_heads: int, dim: int, rot_dim: int, vdim: int, kv_rank: int, scale: float,
                 norm_eps: float, position: Optional[PositionEncoding] = None, gate=True, own_latent: bool = True,
                 names: Tuple[Tuple[str, str], ...] = (), q_rank: Optional[int] = None, sink: bool = False) -> None:
        """``names``: pairs (role, tensor name below the prefix) that replace the defaults for the roles ``q``, ``down``,
        ``down_norm``, ``up_k``, ``up_v``, ``gate``, ``out``, ``q_down``, ``q_norm``, ``q_up``, ``sink``.  ``gate``: False,
        True (a number per channel of the concatenated heads) or ``"head"`` (a number per head)."""
        super().__init__(prefix)
        for label, value in (("hidden_size", hidden_size), ("num_heads", num_heads), ("dim", dim), ("vdim", vdim), ("kv_rank", kv_rank)):
            if int(value) < 1:
                raise ValueError(f"{label}={value} must be positive")
        if int(rot_dim) < 0 or not float(scale) > 0:
            raise ValueError(f"rot_dim={rot_dim} must not be negative and scale={scale} must be positive")
        self.hidden_size, self.num_heads = int(hidden_size), int(num_heads)
        self.dim, self.rot_dim, self.vdim, self.kv_rank = int(dim), int(rot_dim), int(vdim), int(kv_rank)
        self.scale, self.norm_eps = float(scale), float(norm_eps)
        self.position = position
        if gate not in (True, False, "head", "channel"):
            raise ValueError(f"gate={gate!r} must be False, True, 'channel' or 'head'")
        self.gate, self.own_latent = bool(gate), bool(own_latent)
        self.gate_per_head = gate == "head"
        self.q_rank = int(q_rank) if q_rank else 0
        self.sink = bool(sink)
        self.names = dict(_NAMES)
        self.names.update(dict(names))
        self.cached_dim = (self.kv_rank + self.rot_dim + 15) // 16 * 16
        if self.cached_dim > 1024:
            raise ValueError(f"kv_rank + rot_dim = {self.kv_rank + self.rot_dim}: the attention kernels take at most 1,024 cached channels per token")
        self.q_size = self.num_heads * (self.dim + self.rot_dim)
        self.gate_size = (self.num_heads if self.gate_per_head else self.num_heads * self.vdim) if self.gate else 0
        self.first_size = self.q_rank or self.q_size  # what stands first in the rows of the input product: the queries or their latent
        self.down_size = self.kv_rank + self.rot_dim if self.own_latent else 0
        self.in_weight: Optional[torch.Tensor] = None  # rows [W_q (or W_dq) ; W_gate ; W_down]
        self.q_norm_weight: Optional[torch.Tensor] = None
        self.q_up_weight: Optional[torch.Tensor] = None  # [heads * (dim + rot_dim), q_rank]
        self.sink_logits: Optional[torch.Tensor] = None  # float32 [heads]
        self.down_norm_weight: Optional[torch.Tensor] = None
        self.up_k_weight: Optional[torch.Tensor] = None  # [heads * dim, kv_rank]
        self.up_v_weight: Optional[torch.Tensor] = None  # [heads * vdim, kv_rank]
        self.out_weight: Optional[torch.Tensor] = None
        self.query_maps: Optional[torch.Tensor] = None  # [heads, kv_rank, dim]: U_h^T
        self.value_maps: Optional[torch.Tensor] = None  # [heads, vdim, kv_rank]: V_h

    def params(self) -> Dict[str, Param]:
        h, n = self.hidden_size, self.names
        sources, shapes = ([n["q_down"]], [(self.q_rank, h)]) if self.q_rank else ([n["q"]], [(self.q_size, h)])
        if self.gate:
            sources.append(n["gate"])
            shapes.append((self.gate_size, h))
        if self.own_latent:
            sources.append(n["down"])
            shapes.append((self.down_size, h))
        out = {
            "in_weight": fused_rows(tuple(sources), tuple(shapes)),
            "up_k_weight": single(n["up_k"], (self.num_heads * self.dim, self.kv_rank)),
            "up_v_weight": single(n["up_v"], (self.num_heads * self.vdim, self.kv_rank)),
            "out_weight": single(n["out"], (h, self.num_heads * self.vdim)),
        }
        if self.own_latent:
            out["down_norm_weight"] = single(n["down_norm"], (self.kv_rank,), role="vector", init="one_plus_normal")
        if self.q_rank:
            out["q_norm_weight"] = single(n["q_norm"], (self.q_rank,), role="vector", init="one_plus_normal")
            out["q_up_weight"] = single(n["q_up"], (self.q_size, self.q_rank))
        if self.sink:
            out["sink_logits"] = single(n["sink"], (self.num_heads,), role="vector")
        return out

    def cache_need(self):
        return kv_pages(1, self.cached_dim)

    def finalize(self, device, dtype) -> None:
        self.query_maps = self.up_k_weight.view(self.num_heads, self.dim, self.kv_rank).transpose(1, 2).contiguous()
        self.value_maps = self.up_v_weight.view(self.num_heads, self.vdim, self.kv_rank)

    def _rotary(self):
        tables = self.position.rotary_tables() if self.position is not None else None
        if tables is None:
            return None, None, False
        return tables[0], tables[1], getattr(self.position, "layout", "halves") == "interleaved"

    def prepare_kernels(self, ops) -> None:
        load = getattr(ops, "attention_library", None)
        if load is not None and self.cached_dim <= getattr(ops, "MAX_TILED_HEAD_DIM", self.cached_dim):
            load(self.cached_dim)  # (larger cached vectors go to the plain attention kernel of the core library)
        cos, _, _ = self._rotary()
        if cos is not None and 2 * cos.shape[1] > self.rot_dim:
            raise ValueError(f"the rotation spans {2 * cos.shape[1]} channels but the rotated part has {self.rot_dim}")
        self.prepare_weight(ops, "in_weight")
        self.prepare_weight(ops, "out_weight")
        if self.q_rank:
            self.prepare_weight(ops, "q_up_weight")

    def capture_key_bounds(self, ops, batch: int, max_model_len: int):
        choose = getattr(ops, "choose_splits", None)
        if choose is None or max_model_len <= SHORT_CONTEXT_KEYS or self.cached_dim > getattr(ops, "MAX_TILED_HEAD_DIM", self.cached_dim):
            return ()
        differs = choose(batch, 1, 1, max_model_len, True) != choose(batch, 1, 1, SHORT_CONTEXT_KEYS, True)
        return (SHORT_CONTEXT_KEYS,) if differs else ()

    def workspace_needs(self, ops, limits):
        sizes = getattr(ops, "attention_scratch_elems", None)
        if sizes is None:
            return {}
        partial_out, partial_lse = sizes(self.num_heads, 1, self.cached_dim, limits.max_num_tokens, limits.max_num_seqs, limits.max_model_len)
        return {"attention_partial_out": partial_out, "attention_partial_lse": partial_lse}

    def forward(self, x, ctx, cache, owns_cache: bool = True, sink=None):
        ops = ctx.ops
        if owns_cache != self.own_latent:
            raise ValueError("a latent-attention layer writes the cache exactly when it has a down-projection of its own")
        cos, sin, interleaved = self._rotary()
        meta = cache.batch
        projected = ops.linear(x, self.operand("in_weight"), None, ctx.dtype)  # [T, q (or its latent) | gate | down]
        down_offset = self.first_size + self.gate_size if self.own_latent else -1
        if self.q_rank:
            # norm of the latent, rotation of the shared key part and their write into the cache; the queries' own latent
            # is normed by the same kernel and goes through W_uq; then the rotation of the queries' rotated parts
            q_latent = ops.latent_write(
                projected, self.rot_dim, self.kv_rank, self.cached_dim, down_offset, ctx.positions, cos, sin, interleaved, self.down_norm_weight, self.norm_eps,
                meta.slot_mapping, cache.tensors["k"], cache.tensors["v"], cache.block_size, q_latent=(0, self.q_rank, self.q_norm_weight))
            q_source = ops.linear(q_latent, self.operand("q_up_weight"), None, ctx.dtype)
            queries = ops.latent_rotate_write(
                q_source, self.num_heads, self.dim, self.rot_dim, self.kv_rank, self.cached_dim, -1, ctx.positions, cos, sin, interleaved,
                None, self.norm_eps, None, None, None, cache.block_size)
        else:
            # rotation of the queries' rotated parts; norm of the latent, rotation of the shared key part and their write
            # into the cache; the rotated query parts land behind the room for U_h^T a_h in the queries the kernels read
            q_source = projected
            queries = ops.latent_rotate_write(
                projected, self.num_heads, self.dim, self.rot_dim, self.kv_rank, self.cached_dim, down_offset,
                ctx.positions, cos, sin, interleaved, self.down_norm_weight, self.norm_eps,
                meta.slot_mapping, cache.tensors["k"], cache.tensors["v"], cache.block_size)
        # queries[t, h, :kv_rank] = U_h^T a_h(t)
        ops.head_linear(q_source, self.dim + self.rot_dim, 0, self.query_maps, queries, self.cached_dim, 0)
        attended = ops.paged_attention(
            queries, self.num_heads, 1, self.cached_dim,
            cache.tensors["k"], cache.tensors["v"], cache.block_size,
            meta.block_tables, ctx.cu_q, meta.kv_lens,
            ctx.max_q_len, meta.max_kv_len, self.scale, None,
            ctx.all_decode, ctx.workspace,
            decode_prefix=getattr(ctx, "decode_prefix", 0), portions_max_kv_len=getattr(meta, "max_kv_len_of_portions", 0) or None,
            **({"sinks": self.sink_logits} if self.sink else {}),
        )
        # heads[t, h] = V_h attended[t, h, :kv_rank], times sigmoid(gate) when the layer has a gate
        heads = torch.empty((x.shape[0], self.num_heads * self.vdim), dtype=ctx.dtype, device=x.device)
        ops.head_linear(attended, self.cached_dim, 0, self.value_maps, heads, self.vdim, 0,
                        gate=projected if self.gate else None, gate_offset=self.first_size, **({"gate_per_head": True} if self.gate_per_head else {}))
        return ops.linear(heads, self.operand("out_weight"), None, ctx.dtype, partials_ok=True)


register_part("mixer", "latent_attention", LatentAttentionMixer)
