"""Norms that own the residual update: RMSNorm, a norm over several residual streams (``StreamNorm``) and a norm without
statistics (``DynamicTanhNorm``).

Formula (reference ``src/rmsnorm.py:20-28``): in float32, ``y = x * rsqrt(mean(x^2) + eps) * w``,
one rounding at the store.  The reference adds the residual in the model dtype
before the norm (``src/decoder_layer.py:49,54``); here the residual stream is a
float32 tensor and the add is fused into the norm kernel, so the sum is exact
in 32-bit in both run dtypes.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .base import DeferredNorm, Norm, Param, ResidualCopy, ScaledSum, StreamUpdate, register_part, single


class RMSNorm(Norm):
    def __init__(self, prefix: str, hidden_size: int, eps: float, weight_name: str = "weight") -> None:
        """``weight_name``: the tensor's name below the prefix (an architecture whose checkpoint names the norm's
        weight by the prefix alone passes "")."""
        super().__init__(prefix)
        self.hidden_size = int(hidden_size)
        self.eps = float(eps)
        self.weight_name = weight_name
        self.weight: Optional[torch.Tensor] = None

    def params(self) -> Dict[str, Param]:
        return {"weight": single(self.weight_name, (self.hidden_size,), role="vector", init="one_plus_normal")}

    def deferred_form(self):
        return self.weight, self.eps

    def forward(self, residual, delta, ctx, rows=None):
        if isinstance(delta, DeferredNorm):
            # the product before this norm has added itself to the residual and applied the weight; the rest of the
            # norm is a row scale in whatever multiplies next
            if delta.norm is not self or rows is not None:
                raise ValueError("a DeferredNorm can only go to the norm it was made for, on all rows")
            return delta
        if isinstance(delta, ResidualCopy):
            delta = None  # (the block before has added everything itself)
        if rows is None:
            return ctx.ops.add_rmsnorm(residual, delta, self.weight, self.eps, ctx.dtype)
        return ctx.ops.add_rmsnorm_rows(residual, delta, rows, self.weight, self.eps, ctx.dtype)

    def add_normed(self, residual, delta, mult, ctx):
        return ctx.ops.norm_add(residual, delta, self.weight, self.eps, float(mult), ctx.dtype)


register_part("norm", "rmsnorm", RMSNorm)


class StreamNorm(Norm):
    """A norm with a weight and no bias over ``streams`` copies of the residual: the residual is float32 ``[T, streams * H]``
    (one stream after the other within a token's row), the norm reads ``u = sum_s in[s] x_s`` (``in`` None: the plain sum)
    and gives ``(u - mean(u)) / sqrt(var(u) + eps) * w`` (``center``, a layer norm without bias) or ``u / sqrt(mean(u^2) +
    eps) * w``.  What the sub-layer before it produced reaches it as a ``StreamUpdate`` and is worked into the streams
    by the same kernel, before they are read.  With one stream and no weights on the streams this is the plain
    ``residual += delta; normalise(residual)``."""

    def __init__(self, prefix: str, hidden_size: int, eps: float, weight_name: str = "weight", streams: int = 1, center: bool = True) -> None:
        super().__init__(prefix)
        if int(streams) < 1:
            raise ValueError(f"streams={streams} must be at least 1")
        self.hidden_size = int(hidden_size)
        self.eps = float(eps)
        self.weight_name = weight_name
        self.streams = int(streams)
        self.center = bool(center)
        self.weight: Optional[torch.Tensor] = None

    def params(self) -> Dict[str, Param]:
        return {"weight": single(self.weight_name, (self.hidden_size,), role="vector", init="one_plus_normal")}

    def forward_streams(self, residual, update, in_weights, ctx, rows=None):
        """``update``: a ``StreamUpdate``, a plain delta (tensor or ``ScaledSum``: every stream takes it as it is) or None."""
        if isinstance(update, ResidualCopy):
            update = None
        if update is not None and not isinstance(update, StreamUpdate):
            update = StreamUpdate(update)
        terms, scales = (), ()
        if update is not None:
            y = update.y
            if isinstance(y, ScaledSum):
                terms, scales = tuple(y.terms), tuple(float(s) for s in y.scales)
            else:
                if y.dim() == 3:
                    y = y.sum(0)  # (float32 partial sums of a product)
                terms, scales = (y,), (1.0,)
        return ctx.ops.stream_norm(residual, terms, scales, update.mix if update is not None else None, update.out if update is not None else None,
                                   in_weights, self.weight, self.eps, self.streams, self.center, ctx.dtype, rows=rows)

    def forward(self, residual, delta, ctx, rows=None):
        if isinstance(delta, DeferredNorm):
            raise ValueError("this norm cannot be split into a product's epilogue")
        return self.forward_streams(residual, delta, None, ctx, rows=rows)


register_part("norm", "stream_norm", StreamNorm)


class DynamicTanhNorm(Norm):
    """A norm that takes no mean and no variance: ``y = tanh(alpha * x) * w + b`` per channel, with one learned number
    ``alpha`` for the whole layer, a weight and a bias.  The residual update is the same as for every norm here
    (``residual += delta`` in float32 inside the norm's kernel); ``alpha`` stays on the device, so the norm reads nothing
    on the host.  It cannot be split into a product's epilogue and the next product's row scale (there is no row scale).

    ``weight_name``, ``bias_name`` and ``alpha_name`` are the tensors' names below the prefix."""

    def __init__(self, prefix: str, hidden_size: int, weight_name: str = "weight", bias_name: str = "bias", alpha_name: str = "alpha") -> None:
        super().__init__(prefix)
        self.hidden_size = int(hidden_size)
        self.weight_name, self.bias_name, self.alpha_name = weight_name, bias_name, alpha_name
        self.weight: Optional[torch.Tensor] = None
        self.bias: Optional[torch.Tensor] = None
        self.alpha: Optional[torch.Tensor] = None

    def params(self) -> Dict[str, Param]:
        return {
            "weight": single(self.weight_name, (self.hidden_size,), role="vector", init="one_plus_normal"),
            "bias": single(self.bias_name, (self.hidden_size,), role="vector"),
            "alpha": single(self.alpha_name, (), role="vector", init="one_plus_normal"),
        }

    def forward(self, residual, delta, ctx, rows=None):
        if isinstance(delta, DeferredNorm):
            raise ValueError("this norm cannot be split into a product's epilogue")
        if isinstance(delta, ResidualCopy):
            delta = None
        return ctx.ops.add_dynamic_tanh(residual, delta, self.weight, self.bias, self.alpha, ctx.dtype, rows=rows)


register_part("norm", "dynamic_tanh", DynamicTanhNorm)
