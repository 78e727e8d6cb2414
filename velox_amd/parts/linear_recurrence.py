"""Mixers whose memory is a matrix per head that is carried from token to token (linear attention with decay).

Per head, with a state ``S`` of ``dim x vdim`` float32 numbers (rows belong to key channels), a decay ``g_t`` (one number
per head, or one per head and key channel: it multiplies rows), a key ``k_t``, a value ``v_t`` and a query ``q_t``:

``rule="additive"``   ``S <- diag(g_t) S + k_t v_t^T``;                                           ``o_t = S^T q_t``
``rule="delta"``      ``S <- diag(g_t) S``; ``u = beta_t (v_t - S^T k_t)``; ``S <- S + k_t u^T``;  ``o_t = S^T q_t``

(the read-out sees the current token's write).  Around that, all options of the part:

* q and k have ``kv_heads`` heads of ``dim`` channels, v has ``heads`` heads of ``vdim``; head ``h`` reads q/k head
  ``h // (heads / kv_heads)``.  q is multiplied by ``dim ** -0.5``.
* ``conv_taps``: q, k and v pass a short causal convolution per channel (``y_t = sum_j w[:, j] u_(t - taps + 1 + j)``, zeros
  before the start) and then SiLU; the last ``taps - 1`` projected rows of a sequence are part of its state.  With
  ``qkv_silu`` and no convolution the SiLU alone remains (a convolution of one tap whose weights are ones).
* ``unit_qk``: q and k become unit vectors per head, ``x / sqrt(sum(x^2) + 1e-6)`` (before q's factor).
* ``decay``:
  ``"head"``             ``g = exp(-exp(A_log_h) softplus(W_a x + dt_bias_h))``, one per head;
  ``"channel"``          ``g = exp(-exp(A_log_h) softplus(W_a2 (W_a1 x) + dt_bias))``, per head and key channel (a low-rank map);
  ``"sigmoid_channel"``  ``g = sigmoid(W_a2 (W_a1 x) + b)^(1 / tau)``, per head and key channel, computed as
                         ``exp(-softplus(-z) / tau)``.
* ``beta = sigmoid(W_b x)`` per head (``rule="delta"`` only).
* the read-out of each head is divided by its root mean square over ``vdim`` (``eps`` inside the root), multiplied with a
  weight of ``vdim`` entries that all heads share and with a gate: ``gate="silu"``: ``silu(W_g x)``; ``"sigmoid_low_rank"``:
  ``sigmoid(W_g2 (W_g1 x))``.  Then the output product.

Decays, step sizes, ``beta``, the unit vectors, the state and the read-out's norm are float32 in both run dtypes; the
projections, the convolution and its SiLU are the run dtype's.  The state lives in the request's state slot,
``[heads, dim, vdim]`` float32, beside the convolution's last inputs ``[taps - 1, channels]`` in the run dtype.

Kernels of a step: one product for everything that reads ``x`` directly (``[q; k; v; b; a; g]``), one for the first
halves of the low-rank maps and one for their second halves (a block-diagonal weight built at load time, so that decay and gate
cost one product together), the convolution, ``recurrence_prepare`` (unit vectors, decay, beta), ``linear_scan`` (the
recurrence itself, token by token, a sequence's portion in order from its slot's state), ``gated_head_norm``, the output
product.
"""
from __future__ import annotations

from typing import Dict, Optional, Tuple

import torch

from .base import Mixer, Param, StateNeed, fused_rows, register_part, single

_DEFAULT_NAMES = {"q": "q", "k": "k", "v": "v", "o": "o", "beta": "b", "A_log": "A_log", "dt_bias": "dt_bias", "norm": "norm",
                  "a": "a", "a1": "a1", "a2": "a2", "a2_bias": "a2.b", "g": "g", "g1": "g1", "g2": "g2"}


class LinearRecurrenceMixer(Mixer):
    def __init__(self, prefix: str, hidden_size: int, num_heads: int, num_kv_heads: int, dim: int, vdim: int, norm_eps: float,
                 rule: str = "delta", decay: str = "head", gate: str = "silu", conv_taps: int = 0, unit_qk: bool = False, qkv_silu: bool = False,
                 decay_rank: Optional[int] = None, gate_rank: Optional[int] = None, tau: float = 1.0,
                 names: Tuple[Tuple[str, str], ...] = ()) -> None:
        """``decay_rank`` / ``gate_rank``: the inner sizes of the low-rank maps (rows of ``a1`` / ``g1``)."""
        super().__init__(prefix)
        if rule not in ("delta", "additive"):
            raise ValueError(f"rule must be 'delta' or 'additive', got {rule!r}")
        if decay not in ("head", "channel", "sigmoid_channel"):
            raise ValueError(f"decay must be 'head', 'channel' or 'sigmoid_channel', got {decay!r}")
        if gate not in ("silu", "sigmoid_low_rank"):
            raise ValueError(f"gate must be 'silu' or 'sigmoid_low_rank', got {gate!r}")
        if num_heads % num_kv_heads != 0 or min(num_heads, num_kv_heads, dim, vdim) < 1:
            raise ValueError("heads must be a positive multiple of kv_heads, dim and vdim positive")
        if decay != "head" and not decay_rank:
            raise ValueError("a decay per channel needs decay_rank, the inner size of its low-rank map")
        if gate == "sigmoid_low_rank" and not gate_rank:
            raise ValueError("a low-rank gate needs gate_rank")
        if decay == "sigmoid_channel" and not tau > 0:
            raise ValueError("tau must be positive")
        self.hidden_size = int(hidden_size)
        self.num_heads = int(num_heads)
        self.num_kv_heads = int(num_kv_heads)
        self.dim = int(dim)
        self.vdim = int(vdim)
        self.norm_eps = float(norm_eps)
        self.rule, self.decay, self.gate = rule, decay, gate
        self.conv_taps = int(conv_taps)
        self.unit_qk = bool(unit_qk)
        self.qkv_silu = bool(qkv_silu)
        self.decay_rank = int(decay_rank or 0) if decay != "head" else 0
        self.gate_rank = int(gate_rank or 0) if gate == "sigmoid_low_rank" else 0
        self.tau = float(tau)
        self.names = dict(_DEFAULT_NAMES)
        self.names.update(dict(names))
        self.q_size = self.k_size = self.num_kv_heads * self.dim
        self.v_size = self.num_heads * self.vdim
        self.conv_channels = self.q_size + self.k_size + self.v_size
        # columns of the first product, in order: q, k, v, then beta, the decay per head and the full gate where there are such
        at = self.conv_channels
        self.beta_at = self.a_at = self.g_at = None
        if rule == "delta":
            self.beta_at, at = at, at + self.num_heads
        if decay == "head":
            self.a_at, at = at, at + self.num_heads
        if gate == "silu":
            self.g_at, at = at, at + self.v_size
        self.main_columns = at
        self.decay_columns = self.num_heads if decay == "head" else self.num_heads * self.dim
        self.main_weight = self.conv_weight = self.o_weight = self.norm_weight = None
        self.low_in_weight = self.a2_weight = self.g2_weight = self.a2_bias = None
        self.A_log = self.dt_bias = None
        self.low_out_weight = self.low_out_bias = self.decay_rate = self.decay_bias = None

    # -- tensors --------------------------------------------------------------------------------
    def params(self) -> Dict[str, Param]:
        h, n = self.hidden_size, self.names
        rows = [(n["q"], self.q_size), (n["k"], self.k_size), (n["v"], self.v_size)]
        if self.rule == "delta":
            rows.append((n["beta"], self.num_heads))
        if self.decay == "head":
            rows.append((n["a"], self.num_heads))
        if self.gate == "silu":
            rows.append((n["g"], self.v_size))
        out = {"main_weight": fused_rows(tuple(r[0] for r in rows), tuple((r[1], h) for r in rows))}
        if self.conv_taps:
            out["conv_weight"] = fused_rows((n["q"] + ".conv", n["k"] + ".conv", n["v"] + ".conv"),
                                            tuple((s, self.conv_taps) for s in (self.q_size, self.k_size, self.v_size)), role="vector")
        low = []
        if self.decay_rank:
            low.append((n["a1"], self.decay_rank))
            out["a2_weight"] = single(n["a2"], (self.num_heads * self.dim, self.decay_rank))
        if self.gate_rank:
            low.append((n["g1"], self.gate_rank))
            out["g2_weight"] = single(n["g2"], (self.v_size, self.gate_rank))
        if low:
            out["low_in_weight"] = fused_rows(tuple(r[0] for r in low), tuple((r[1], h) for r in low))
        if self.decay == "sigmoid_channel":
            out["a2_bias"] = single(n["a2_bias"], (self.num_heads * self.dim,), role="vector")
        else:
            out["A_log"] = single(n["A_log"], (self.num_heads,), role="vector")
            out["dt_bias"] = single(n["dt_bias"], (self.decay_columns,), role="vector")
        out["norm_weight"] = single(n["norm"], (self.vdim,), role="vector", init="one_plus_normal")
        out["o_weight"] = single(n["o"], (h, self.v_size))
        return out

    def finalize(self, device, dtype) -> None:
        self.refresh_derived()

    def refresh_derived(self) -> None:
        """What is derived from the bound tensors: the block-diagonal second half of the low-rank maps, and the decay's
        rate per head and bias per column.  To be called again after a tensor was bound anew."""
        inner = self.decay_rank + self.gate_rank
        self.low_out_weight = None
        if inner and (self.a2_weight is not None or self.g2_weight is not None):
            source = self.a2_weight if self.a2_weight is not None else self.g2_weight
            rows = (self.num_heads * self.dim if self.decay_rank else 0) + (self.v_size if self.gate_rank else 0)
            wide = torch.zeros((rows, inner), dtype=source.dtype, device=source.device)
            at = 0
            if self.decay_rank:
                wide[: self.num_heads * self.dim, : self.decay_rank] = self.a2_weight
                at = self.num_heads * self.dim
            if self.gate_rank:
                wide[at:, self.decay_rank:] = self.g2_weight
            self.low_out_weight = wide
        self._prepared.pop("low_out_weight", None)
        if self.conv_taps == 0 and self.qkv_silu and self.main_weight is not None:
            self.conv_weight = torch.ones((self.conv_channels, 1), dtype=torch.float32, device=self.main_weight.device)
        if self.decay == "sigmoid_channel":
            if self.a2_bias is not None:
                self.decay_rate = torch.full((self.num_heads,), 1.0 / self.tau, dtype=torch.float32, device=self.a2_bias.device)
                self.decay_bias = self.a2_bias
        elif self.A_log is not None:
            self.decay_rate = torch.exp(self.A_log.float())
            self.decay_bias = self.dt_bias

    def cache_need(self):
        tensors = [("state", (self.num_heads, self.dim, self.vdim), torch.float32)]
        if self.conv_taps >= 2:
            tensors.append(("conv_tail", (self.conv_taps - 1, self.conv_channels), None))
        return StateNeed(tuple(tensors))

    def prepare_kernels(self, ops) -> None:
        self.prepare_weight(ops, "main_weight")
        self.prepare_weight(ops, "o_weight")
        check = getattr(ops, "linear_scan_supports", None)
        if check is not None:
            check(self.dim, self.vdim)

    # -- arithmetic -----------------------------------------------------------------------------
    def forward(self, x, ctx, cache, owns_cache: bool = True):
        if not owns_cache:
            raise RuntimeError("a recurrent mixer cannot read another entry's state: every run of it advances a state of its own")
        ops = ctx.ops
        heads, kv_heads, dim, vdim = self.num_heads, self.num_kv_heads, self.dim, self.vdim
        main = ops.linear(x, self.operand("main_weight"), None, ctx.dtype)
        qkv, q_at, k_at, v_at = main, 0, self.q_size, self.q_size + self.k_size
        if self.conv_taps >= 1 or self.qkv_silu:
            tail = cache.tensors["conv_tail"] if self.conv_taps >= 2 else None
            qkv = ops.short_conv(main, self.conv_channels, self.conv_weight, tail, ctx.slots, ctx.cu_q, ctx.max_q_len, activation="silu")
        low = None
        if self.low_out_weight is not None:
            inner = ops.linear(x, self.low_in_weight, None, ctx.dtype)
            low = ops.linear(inner, self.low_out_weight, None, torch.float32)
        if self.decay == "head":
            decay_source, decay_at = main, self.a_at
        else:
            decay_source, decay_at = low, 0
        sign = -1.0 if self.decay == "sigmoid_channel" else 1.0
        qk, decay, beta = ops.recurrence_prepare(
            qkv, q_at, k_at, kv_heads, dim, self.unit_qk, float(dim) ** -0.5,
            decay_source, decay_at, heads, self.decay_columns, self.decay_rate, self.decay_bias, sign,
            main if self.rule == "delta" else None, self.beta_at or 0,
        )
        read = ops.linear_scan(qk, qkv, v_at, decay, beta, cache.tensors["state"], ctx.slots, ctx.cu_q, ctx.max_q_len,
                               heads, kv_heads, dim, vdim, self.rule == "delta")
        if self.gate == "silu":
            gate_source, gate_at, gate_kind = main, self.g_at, "silu"
        else:
            gate_source, gate_at, gate_kind = low, (heads * dim if self.decay_rank else 0), "sigmoid"
        y = ops.gated_head_norm(read, self.norm_weight, self.norm_eps, gate_source, gate_at, gate_kind, heads, vdim, ctx.dtype)
        return ops.linear(y, self.operand("o_weight"), None, ctx.dtype)


register_part("mixer", "linear_recurrence", LinearRecurrenceMixer)
