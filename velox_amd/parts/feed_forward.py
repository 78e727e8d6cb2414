"""Feed-forwards: the dense gated one, routed experts, and none at all.

Reference ``src/mlp.py:9-15``: one fused product with rows ``[Wgate; Wup]`` (no bias),
``act(gate) * up``, down product (no bias); ``silu(x) = x * sigmoid(x)``.  The
activation and the product ``act(gate) * up`` are computed in float32 with one
rounding at the store; for decode-sized batches they are the epilogue of the
gate/up product itself, which then never writes its ``[T, 2I]`` result.

``RoutedExperts`` (no counterpart in the reference): ``E`` small gated units of which every token uses ``top``,
chosen by a router whose logits are float32.  The score function, whether the chosen scores are renormalised and
whether a score scales the expert's input or its output are options of the part.  Nothing is decided on the host:
a plan kernel sorts the (token, choice) pairs by expert on the device, two grouped products run every expert on
its own rows, and a last kernel adds each token's results in the order of its choices, so the step can be captured
and a token's result does not depend on which other tokens share its experts.
"""
from __future__ import annotations

from typing import Dict, Optional, Tuple

import torch

from .base import FeedForward, Param, fused_rows, register_part, single


SILU_UNIT = (1.0, float("inf"), 0.0)  # (alpha, limit, shift) of ``silu(gate) * up``
UNGATED_ACTIVATIONS = ("relu2",)  # activations of a unit without a gate branch


class GatedMLP(FeedForward):
    def __init__(self, prefix: str, hidden_size: int, intermediate_size: int, activation: str = "silu",
                 names: Tuple[str, str, str] = ("gate_proj.weight", "up_proj.weight", "down_proj.weight")) -> None:
        """``names``: the gate, up and down tensors below the prefix."""
        super().__init__(prefix)
        self.names = tuple(names)
        if activation not in ("silu", "gelu_tanh"):
            raise ValueError(f"activation {activation!r} is not implemented ('silu' or 'gelu_tanh')")
        self.activation = activation
        self.hidden_size = int(hidden_size)
        self.intermediate_size = int(intermediate_size)
        self.gate_up_weight: Optional[torch.Tensor] = None
        self.down_weight: Optional[torch.Tensor] = None

    def params(self) -> Dict[str, Param]:
        h, i = self.hidden_size, self.intermediate_size
        return {
            "gate_up_weight": fused_rows(self.names[:2], ((i, h), (i, h))),
            "down_weight": single(self.names[2], (h, i)),
        }

    def prepare_kernels(self, ops) -> None:
        self.prepare_weight(ops, "gate_up_weight", stacked=2)
        self.prepare_weight(ops, "down_weight")

    accepts_sink = True  # its last product may add itself to the residual (ResidualSink)
    accepts_deferred = True  # its first product can read a DeferredNorm

    def forward(self, x, ctx, sink=None, partials_ok: bool = True):
        ops = ctx.ops
        if self.activation == "silu":
            act = ops.linear_silu_mul(x, self.operand("gate_up_weight"), ctx.dtype)
        else:
            # gelu_tanh(z) = z / 2 * (1 + tanh(sqrt(2 / pi) (z + 0.044715 z^3))), in float32 with one rounding at the store
            fused = getattr(ops, "linear_gated_act", None)  # (one kernel for decode-sized batches where the operations have it)
            if fused is not None:
                act = fused(x, self.operand("gate_up_weight"), ctx.dtype, self.activation)
            else:
                act = ops.gated_act_mul(ops.linear(x, self.operand("gate_up_weight"), None, ctx.dtype), self.activation)
        return ops.linear(act, self.operand("down_weight"), None, ctx.dtype, partials_ok=partials_ok, residual_norm=sink)


register_part("feed_forward", "gated_mlp", GatedMLP)


class PlainMLP(FeedForward):
    """``W_down act(W_up x)`` without a gate branch and without biases; ``act`` is ``relu2`` (the square of the rectified
    value).  The activation is float32 with one rounding at the store."""

    def __init__(self, prefix: str, hidden_size: int, intermediate_size: int, activation: str = "relu2",
                 names: Tuple[str, str] = ("up_proj.weight", "down_proj.weight")) -> None:
        super().__init__(prefix)
        if activation not in UNGATED_ACTIVATIONS:
            raise ValueError(f"activation {activation!r} is not implemented ({', '.join(UNGATED_ACTIVATIONS)})")
        self.activation = activation
        self.names = tuple(names)
        self.hidden_size = int(hidden_size)
        self.intermediate_size = int(intermediate_size)
        self.up_weight: Optional[torch.Tensor] = None
        self.down_weight: Optional[torch.Tensor] = None

    def params(self) -> Dict[str, Param]:
        h, i = self.hidden_size, self.intermediate_size
        return {"up_weight": single(self.names[0], (i, h)), "down_weight": single(self.names[1], (h, i))}

    def prepare_kernels(self, ops) -> None:
        self.prepare_weight(ops, "up_weight")
        self.prepare_weight(ops, "down_weight")

    def forward(self, x, ctx, sink=None):
        ops = ctx.ops
        act = ops.linear_act(x, self.operand("up_weight"), ctx.dtype, self.activation)
        return ops.linear(act, self.operand("down_weight"), None, ctx.dtype, partials_ok=True)


register_part("feed_forward", "plain_mlp", PlainMLP)


class NoFeedForward(FeedForward):
    """A layer without a feed-forward: ``forward`` gives None and the block adds nothing."""

    def __init__(self, prefix: str = "") -> None:
        super().__init__(prefix)

    def forward(self, x, ctx, sink=None):
        return None


register_part("feed_forward", "none", NoFeedForward)


class RoutedExperts(FeedForward):
    """``y = sum_k unit_{e_k}(s_k x)`` (``scale_input``) or ``sum_k s_k unit_{e_k}(x)``, plus ``shared(x)`` when there is
    a shared unit; ``unit(x) = W_down (silu(W_gate x) * (W_up x))``; ``e_1 .. e_top`` are the experts with the largest
    scores ``s = score(W_router x)`` (``sigmoid``, or ``softmax`` over all experts), kept as they are or divided by their
    sum (``renormalize``).  The router's logits and the scores are float32.

    Tensors: the experts' gate and up matrices are held as one ``[E * 2 F, H]`` tensor (expert after expert, each gate
    rows then up rows), the down matrices as ``[E * H, F]``; ``expert_names(e)`` gives the three names of expert ``e``
    below the prefix."""

    def __init__(self, prefix: str, hidden_size: int, intermediate_size: int, num_experts: int, top: int, score: str = "sigmoid",
                 renormalize: bool = False, scale_input: bool = True, shared_intermediate_size: Optional[int] = None,
                 expert_names: Tuple[str, str, str] = ("experts.{e}.gate.weight", "experts.{e}.up.weight", "experts.{e}.down.weight"),
                 router_name: str = "router.weight", shared_prefix: str = "shared.",
                 shared_names: Tuple[str, str, str] = ("gate_proj.weight", "up_proj.weight", "down_proj.weight"),
                 unit: Tuple[float, float, float] = SILU_UNIT, identity_experts: int = 0, correction_name: Optional[str] = None,
                 ungated: Optional[str] = None, groups: Optional[Tuple[int, int]] = None, renormalize_floor: float = 0.0) -> None:
        """``unit = (alpha, limit, shift)``: a unit's middle is ``g sigmoid(alpha g) (u + shift)`` with ``g = min(W_gate x,
        limit)`` and ``u = clamp(W_up x, -limit, limit)``; ``(1, inf, 0)`` is ``silu(gate) * up``.  ``identity_experts``: the
        router has that many outputs more than there are units; an identity expert's result is its input (times the
        weight, wherever the weight stands).  ``correction_name``: a float32 vector over all router outputs that is added
        to the scores for the choice only; the weights are the scores without it.  ``ungated``: the units have no gate
        branch, ``W_down act(W_up x)`` with this activation (``relu2``); ``expert_names`` then names two tensors (up, down)
        and ``unit`` is not used.  ``groups = (count, keep)``: the experts form ``count`` equal groups of neighbours, a group's
        score is the sum of its two largest choice scores, and only experts of the ``keep`` best groups can be chosen.
        ``renormalize_floor``: added to the sum that renormalised weights are divided by."""
        super().__init__(prefix)
        if ungated is not None and ungated not in UNGATED_ACTIVATIONS:
            raise ValueError(f"ungated={ungated!r} is not implemented ({', '.join(UNGATED_ACTIVATIONS)})")
        self.ungated = ungated
        if ungated is not None and (identity_experts or shared_intermediate_size):
            raise ValueError("units without a gate branch come without identity experts and without a shared unit")
        self.groups = (int(groups[0]), int(groups[1])) if groups else None
        if self.groups is not None:
            count, keep = self.groups
            total = int(num_experts) + int(identity_experts)
            if count < 1 or total % count != 0 or not 1 <= keep <= count or keep * (total // count) < int(top):
                raise ValueError(f"groups={groups}: {total} experts must form equal groups, and the kept groups must hold at least top={top} experts")
        self.renormalize_floor = float(renormalize_floor)
        self.unit = (float(unit[0]), float(unit[1]), float(unit[2]))
        if not self.unit[1] > 0:
            raise ValueError(f"unit: the limit must be positive (inf for none), got {self.unit[1]}")
        self.identity_experts = int(identity_experts)
        if self.identity_experts < 0:
            raise ValueError("identity_experts must not be negative")
        self.correction_name = correction_name
        self.correction: Optional[torch.Tensor] = None
        if score not in ("sigmoid", "softmax"):
            raise ValueError(f"score {score!r} is not implemented ('sigmoid' or 'softmax')")
        if not 1 <= int(top) <= int(num_experts) + int(identity_experts):
            raise ValueError(f"top={top} must lie between 1 and the number of experts ({int(num_experts) + int(identity_experts)})")
        self.hidden_size = int(hidden_size)
        self.intermediate_size = int(intermediate_size)
        self.num_experts = int(num_experts)
        self.top = int(top)
        self.score = score
        self.renormalize = bool(renormalize)
        self.scale_input = bool(scale_input)
        self.expert_names = tuple(expert_names)
        self.router_name = router_name
        self.shared = None
        if shared_intermediate_size:
            self.shared = GatedMLP(prefix + shared_prefix, hidden_size, int(shared_intermediate_size), names=shared_names)
        self.router_weight: Optional[torch.Tensor] = None
        self.gate_up_weight: Optional[torch.Tensor] = None
        self.down_weight: Optional[torch.Tensor] = None

    def params(self) -> Dict[str, Param]:
        h, f, e = self.hidden_size, self.intermediate_size, self.num_experts
        first, down = self.expert_names[:-1], self.expert_names[-1]  # (gate, up) or, without a gate branch, (up,)
        if len(first) != (1 if self.ungated else 2):
            raise ValueError(f"expert_names must name {'up and down' if self.ungated else 'gate, up and down'}")
        gate_up_names = tuple(name.format(e=i) for i in range(e) for name in first)
        out = {
            "router_weight": single(self.router_name, (e + self.identity_experts, h)),
            "gate_up_weight": fused_rows(gate_up_names, ((f, h),) * (len(first) * e)),
            "down_weight": fused_rows(tuple(down.format(e=i) for i in range(e)), ((h, f),) * e),
        }
        if self.correction_name is not None:
            out["correction"] = single(self.correction_name, (e + self.identity_experts,), role="vector")
        return out

    def children(self):
        return (self.shared,) if self.shared is not None else ()

    def workspace_needs(self, ops, limits):
        sizes = getattr(ops, "routed_plan_elems", None)
        if sizes is None:
            return {}
        return {"routed_plan": sizes(limits.max_num_tokens, self.top, self.num_experts)}

    accepts_output_norm = True  # its last kernel can norm the sum of the experts' results and add it to the residual

    def forward(self, x, ctx, sink=None, output_norm=None):
        ops = ctx.ops
        x = ops.materialize(x)
        logits = ops.linear(x, self.router_weight, None, torch.float32)
        options = {}
        if self.correction is not None:
            options["correction"] = self.correction
        if self.groups is not None:
            options["groups"] = self.groups
        if self.renormalize_floor:
            options["norm_floor"] = self.renormalize_floor
        choice, weight = ops.route_top(logits, self.top, self.score, self.renormalize, **options)
        if self.ungated is not None:
            return ops.routed_experts(x, choice, weight, self.gate_up_weight, self.down_weight, self.num_experts, self.scale_input, None,
                                      ctx.dtype, ctx.workspace, ungated=self.ungated, **({"output_norm": output_norm} if output_norm is not None else {}))
        shared = self.shared.forward(x, ctx, partials_ok=False) if self.shared is not None else None
        if output_norm is not None:
            return ops.routed_experts(x, choice, weight, self.gate_up_weight, self.down_weight, self.num_experts, self.scale_input, shared,
                                      ctx.dtype, ctx.workspace, unit=self.unit, identity_experts=self.identity_experts, output_norm=output_norm)
        if self.unit == SILU_UNIT and not self.identity_experts:
            return ops.routed_experts(x, choice, weight, self.gate_up_weight, self.down_weight, self.num_experts, self.scale_input, shared,
                                      ctx.dtype, ctx.workspace)
        return ops.routed_experts(x, choice, weight, self.gate_up_weight, self.down_weight, self.num_experts, self.scale_input, shared,
                                  ctx.dtype, ctx.workspace, unit=self.unit, identity_experts=self.identity_experts)


register_part("feed_forward", "routed_experts", RoutedExperts)
