"""Grouped-query softmax attention whose queries, keys and values pass a short causal convolution over time.

Beside ``parts.attention`` and ``parts.normed_attention`` this mixer has

* biases on the q, k, v and output projections (each optional);
* a short causal convolution per channel of q, k and v, directly behind the projection and before the rotation:
  ``y_t = sum_j w[:, j] u_(t - taps + 1 + j)``, zeros before the sequence's start (the last column of ``w`` meets the
  current token).  The last ``taps - 1`` projected rows of a sequence are kept in its state slot, in the run dtype, as
  the projection left them, so a portion's first tokens see exactly what they would have seen in a whole prompt;
* a rotation of the first ``rotary_dim`` channels of each query and key head only (the rest passes), in either layout of
  the position encoding: channel ``i`` with ``i + rotary_dim / 2`` or channel ``2i`` with ``2i + 1``;
* its own sizes for query/key heads (``dim``) and value heads (``vdim``), a scale from the configuration, a sliding
  window (``window``: a query at ``i`` sees ``j`` with ``0 <= i - j < window``; pages behind it are given back).

How it meets the kernels: as for ``NormedAttentionMixer`` the paged cache holds heads of ``D = ceil16(max(dim, vdim))``
channels with zeros in the padding, the queries are written at that size by the kernel that rotates them and writes the
cache, and the output product reads a copy of its weight with zero columns at the padding's places.
"""
from __future__ import annotations

from typing import Dict, Optional, Tuple

import torch

from .attention import SHORT_CONTEXT_KEYS, kv_pages
from .base import CompositeNeed, Mixer, Param, PositionEncoding, StateNeed, fused_rows, register_part, single


class ConvAttentionMixer(Mixer):
    def __init__(self, prefix: str, hidden_size: int, num_heads: int, num_kv_heads: int, dim: int, vdim: int, scale: float,
                 window: Optional[int] = None, conv_taps: int = 0, qkv_bias: bool = True, out_bias: bool = True,
                 position: Optional[PositionEncoding] = None, names: Tuple[Tuple[str, str], ...] = ()) -> None:
        """``conv_taps``: columns of the convolution's weights (0 or 1 column less than 2: 0 = no convolution);
        ``names``: pairs (tensor, name below the prefix) that replace the default names ``q``, ``k``, ``v``, ``o``; a
        bias is the tensor's name with ``.b`` added, a convolution's weights with ``.conv``."""
        super().__init__(prefix)
        if num_heads % num_kv_heads != 0:
            raise ValueError(f"num_heads={num_heads} must be a multiple of num_kv_heads={num_kv_heads}")
        if min(int(dim), int(vdim)) < 1 or not float(scale) > 0:
            raise ValueError("dim and vdim must be positive, and so must the scale")
        if window is not None and window < 1:
            raise ValueError(f"window={window} must be at least 1")
        if conv_taps < 0:
            raise ValueError("conv_taps must not be negative")
        self.interleaved = getattr(position, "layout", "halves") == "interleaved"
        self.hidden_size = int(hidden_size)
        self.num_heads = int(num_heads)
        self.num_kv_heads = int(num_kv_heads)
        self.dim = int(dim)
        self.vdim = int(vdim)
        self.cached_dim = (max(self.dim, self.vdim) + 15) // 16 * 16  # one head in the cache and in the kernels
        self.scale = float(scale)
        self.window = window
        self.conv_taps = int(conv_taps)
        self.qkv_bias = bool(qkv_bias)
        self.out_bias = bool(out_bias)
        self.position = position
        if position is not None and getattr(position, "rotary_dim", 0) > self.dim:
            raise ValueError(f"the rotation spans {position.rotary_dim} channels but a query head has {self.dim}")
        self.names = {"q": "q", "k": "k", "v": "v", "o": "o"}
        self.names.update(dict(names))
        self.q_size = self.num_heads * self.dim
        self.k_size = self.num_kv_heads * self.dim
        self.v_size = self.num_kv_heads * self.vdim
        self.channels = self.q_size + self.k_size + self.v_size
        self.qkv_weight: Optional[torch.Tensor] = None
        self.qkv_bias_vec: Optional[torch.Tensor] = None
        self.conv_weight: Optional[torch.Tensor] = None
        self.o_weight: Optional[torch.Tensor] = None
        self.o_bias_vec: Optional[torch.Tensor] = None
        self.o_padded: Optional[torch.Tensor] = None

    def params(self) -> Dict[str, Param]:
        h, n = self.hidden_size, self.names
        sizes = (self.q_size, self.k_size, self.v_size)
        out = {"qkv_weight": fused_rows((n["q"], n["k"], n["v"]), tuple((s, h) for s in sizes))}
        if self.qkv_bias:
            out["qkv_bias_vec"] = fused_rows((n["q"] + ".b", n["k"] + ".b", n["v"] + ".b"), tuple((s,) for s in sizes), role="vector")
        if self.conv_taps:
            out["conv_weight"] = fused_rows((n["q"] + ".conv", n["k"] + ".conv", n["v"] + ".conv"), tuple((s, self.conv_taps) for s in sizes), role="vector")
        out["o_weight"] = single(n["o"], (h, self.num_heads * self.vdim))
        if self.out_bias:
            out["o_bias_vec"] = single(n["o"] + ".b", (h,), role="vector")
        return out

    def cache_need(self):
        pages = kv_pages(self.num_kv_heads, self.cached_dim, self.window)
        if self.conv_taps < 2:
            return pages
        return CompositeNeed((pages, StateNeed((("conv_tail", (self.conv_taps - 1, self.channels), None),))))

    def finalize(self, device, dtype) -> None:
        self.refresh_derived()

    def refresh_derived(self) -> None:
        """The output weight at the kernels' head size; to be called again after a tensor was bound anew."""
        self.o_padded = None
        if self.o_weight is not None and self.cached_dim != self.vdim:
            wide = torch.zeros((self.hidden_size, self.num_heads, self.cached_dim), dtype=self.o_weight.dtype, device=self.o_weight.device)
            wide[:, :, : self.vdim] = self.o_weight.view(self.hidden_size, self.num_heads, self.vdim)
            self.o_padded = wide.view(self.hidden_size, self.num_heads * self.cached_dim)
        self._prepared.pop("o_padded", None)

    def prepare_kernels(self, ops) -> None:
        load = getattr(ops, "attention_library", None)
        if load is not None and self.cached_dim <= getattr(ops, "MAX_TILED_HEAD_DIM", self.cached_dim):
            load(self.cached_dim)
        self.prepare_weight(ops, "qkv_weight")
        self.prepare_weight(ops, "o_padded" if self.o_padded is not None else "o_weight")

    def capture_key_bounds(self, ops, batch: int, max_model_len: int):
        choose = getattr(ops, "choose_splits", None)
        if choose is None or max_model_len <= SHORT_CONTEXT_KEYS:
            return ()
        differs = choose(batch, self.num_kv_heads, 1, max_model_len, True) != choose(batch, self.num_kv_heads, 1, SHORT_CONTEXT_KEYS, True)
        return (SHORT_CONTEXT_KEYS,) if differs else ()

    def workspace_needs(self, ops, limits):
        sizes = getattr(ops, "attention_scratch_elems", None)
        if sizes is None:
            return {}
        partial_out, partial_lse = sizes(self.num_heads, self.num_kv_heads, self.cached_dim, limits.max_num_tokens, limits.max_num_seqs, limits.max_model_len)
        return {"attention_partial_out": partial_out, "attention_partial_lse": partial_lse}

    def forward(self, x, ctx, cache, owns_cache: bool = True):
        ops = ctx.ops
        if self.conv_taps >= 2:
            pages, state = cache.views
        else:
            pages, state = cache, None
        meta = pages.batch
        qkv = ops.linear(x, self.operand("qkv_weight"), self.qkv_bias_vec if self.qkv_bias else None, ctx.dtype)
        if self.conv_taps >= 1:
            qkv = ops.short_conv(qkv, self.channels, self.conv_weight, state.tensors["conv_tail"] if state is not None else None,
                                 ctx.slots, ctx.cu_q, ctx.max_q_len, activation="none", update_state=owns_cache)
        cos, sin = (self.position.rotary_tables() if self.position is not None else None) or (None, None)
        q = ops.rotate_pad_write(
            qkv, self.num_heads, self.num_kv_heads, self.dim, self.vdim, self.cached_dim, ctx.positions, cos, sin,
            meta.slot_mapping, pages.tensors["k"], pages.tensors["v"], pages.block_size, write_kv=owns_cache,
            **({"interleaved": True} if self.interleaved else {}),
        )
        attn = ops.paged_attention(
            q, self.num_heads, self.num_kv_heads, self.cached_dim,
            pages.tensors["k"], pages.tensors["v"], pages.block_size,
            meta.block_tables, ctx.cu_q, meta.kv_lens,
            ctx.max_q_len, meta.max_kv_len, self.scale, self.window,
            ctx.all_decode, ctx.workspace,
            decode_prefix=getattr(ctx, "decode_prefix", 0), portions_max_kv_len=getattr(meta, "max_kv_len_of_portions", 0) or None,
        )
        return ops.linear(attn, self.operand("o_padded" if self.o_padded is not None else "o_weight"), self.o_bias_vec if self.out_bias else None, ctx.dtype)


register_part("mixer", "conv_attention", ConvAttentionMixer)
