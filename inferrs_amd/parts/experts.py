"""Routed experts: a router scores every expert for a token, the `top` best run, and their outputs are added up
with score * scale as weights.  An expert: g = min(W_gate h, limit), u = clamp(W_up h, -limit, limit),
W_down (g * sigmoid(alpha g) * (u + 1)).  The router's logits are 32-bit.

`forward` returns `RoutedRows`: one 32-bit output row a (token, chosen expert) and the weights; whoever adds the
feed-forward's output to the stream adds them up, a token's rows in the order of its choice, so a token's sum does
not depend on the other tokens of the step (`.materialize()` gives the plain sum for a block that knows nothing of
this).

Options of the spec: `identity` more outputs of the router behind the experts', each standing for an expert that hands
its input on (no tensors: `RoutedRows.sel` and `.real_experts` tell whoever adds the rows up which pairs these are, and
the stream's own row takes their place); `correction`, a vector added to the scores for the choice only; `shared`, a
feed-forward of the experts' form that runs for every token (`ClampedMlp`; its output rides along as `RoutedRows.extra`),
behind a sigmoid gate a token with `shared_gate` (its row stands behind the router's in one matrix, so that the gate is
formed like a router's logit: `RoutedRows.extra_scale`); `weight_on_input`, a chosen expert runs on weight * h and its
output counts as it is (`RoutedRows.weights` is None then)."""
from __future__ import annotations

from typing import Dict

import torch

from .. import ops
from ..config.spec import ClampedMlpSpec, RoutedExpertsSpec, SpecError
from ..weights.loader import TensorSpec
from .base import FeedForward, part_class, register_ffn
from .linear import Linear, to_compute


class RoutedRows:
    """rows [n, top, width] (32-bit) and weights [n, top] (32-bit): the output is sum_k weights[:, k] * rows[:, k].
    `sel` [n, top] with `real_experts`: a pair whose choice is `real_experts` or more has no row here; the
    feed-forward's own input stands for it.  `extra` [n, width]: a dense output to be added beside the rows, times
    `extra_scale` [n] (32-bit) where that is given.  `weights` None: the rows are added as they are."""
    __slots__ = ("rows", "weights", "sel", "real_experts", "extra", "extra_scale")

    def __init__(self, rows: torch.Tensor, weights, sel=None, real_experts: int = 0, extra=None, extra_scale=None):
        self.rows, self.weights, self.sel, self.real_experts, self.extra = rows, weights, sel, real_experts, extra
        self.extra_scale = extra_scale

    def materialize(self) -> torch.Tensor:
        if self.sel is not None or self.extra is not None or self.weights is None:
            raise SpecError("routed_experts: experts that hand their input on, and a shared expert, need a block "
                            "arrangement that adds the routed rows up itself")
        n, top, width = self.rows.shape
        streams = torch.zeros((n, 1, width), dtype=torch.float32, device=self.rows.device)
        one = torch.ones((1,), dtype=torch.float32, device=self.rows.device)
        ops.streams_step(streams, y=self.rows, y_weights=self.weights, mix=one, out=one)
        return streams.view(n, width)


@register_ffn("routed_experts")
class RoutedExperts(FeedForward):
    graph_safe = True

    @classmethod
    def tensors(cls, spec: RoutedExpertsSpec) -> Dict[str, TensorSpec]:
        t = {"router": TensorSpec((spec.experts + spec.identity, spec.hidden))}
        if spec.correction:
            t["correction"] = TensorSpec((spec.experts + spec.identity,))
        if spec.shared is not None:
            for local, ts in part_class("ffn", spec.shared).tensors(spec.shared).items():
                t["shared." + local] = ts
            if spec.shared_gate:
                t["shared.sg"] = TensorSpec((1, spec.hidden))
        for e in range(spec.experts):
            t[f"e{e}.gate"] = TensorSpec((spec.intermediate, spec.hidden))
            t[f"e{e}.up"] = TensorSpec((spec.intermediate, spec.hidden))
            t[f"e{e}.down"] = TensorSpec((spec.hidden, spec.intermediate))
        return t

    def __init__(self, spec: RoutedExpertsSpec, tensors: Dict[str, torch.Tensor], dtype, device):
        outputs = spec.experts + spec.identity
        if (not (1 <= spec.top <= outputs <= ops.mix.MAX_EXPERTS) or spec.top > ops.mix.MAX_TOP or spec.experts < 1
                or spec.identity < 0):
            raise SpecError(f"routed_experts: top {spec.top} of {spec.experts} experts and {spec.identity} that hand their "
                            f"input on (up to {ops.mix.MAX_TOP} of {ops.mix.MAX_EXPERTS})")
        if spec.score not in ops.mix.SCORE_FUNCTIONS:
            raise SpecError(f"routed_experts: score {spec.score!r} has no kernel (known: {sorted(ops.mix.SCORE_FUNCTIONS)})")
        self.spec = spec
        # the router's logits are 32-bit sums whatever its matrix is stored in (`ops.route`)
        self.router = to_compute(tensors["router"], dtype, device)
        if spec.shared_gate and (spec.shared is None or spec.identity):
            raise SpecError("routed_experts: a gate on the shared expert needs a shared expert, and a router whose outputs "
                            "are all experts")
        if spec.weight_on_input and spec.identity:
            raise SpecError("routed_experts: weights on the experts' inputs do not go with outputs that hand the input on")
        if spec.shared_gate:                         # (the gate's row behind the router's: one walk over h serves both)
            self.router = torch.cat([self.router, to_compute(tensors["shared.sg"], dtype, device).view(1, -1)], dim=0).contiguous()
        self.correction = (tensors["correction"].to(device=device, dtype=torch.float32).contiguous()
                           if spec.correction else None)
        self.shared = None
        if spec.shared is not None:
            self.shared = part_class("ffn", spec.shared)(
                spec.shared, {k[len("shared."):]: v for k, v in tensors.items() if k.startswith("shared.") and k != "shared.sg"},
                dtype, device)
        E = spec.experts
        gate_up = torch.stack([torch.cat([to_compute(tensors[f"e{e}.gate"], dtype, device),
                                          to_compute(tensors[f"e{e}.up"], dtype, device)], dim=0) for e in range(E)])
        down = torch.stack([to_compute(tensors[f"e{e}.down"], dtype, device) for e in range(E)])
        # bfloat16 experts whose sizes the matrix cores take keep their weights as tiles of 64 features x 64 inputs
        self.tiled = ops.mix.experts_tiled_fits(dtype, spec.hidden, spec.intermediate)
        if self.tiled:
            gate_up = ops.mix.tile_weights(gate_up.view(E, 2, spec.intermediate, spec.hidden))
            down = ops.mix.tile_weights(down)
        self.gate_up, self.down = gate_up.contiguous(), down.contiguous()

    def forward(self, ctx, h):
        s = self.spec
        if hasattr(h, "materialize"):
            h = h.materialize()
        gate = None
        if s.shared_gate:
            sel, weights, gate = ops.route(h, self.router, s.top, s.scale, s.score, s.renormalize, self.correction, gates=1)
        else:
            sel, weights = ops.route(h, self.router, s.top, s.scale, s.score, s.renormalize, self.correction)
        rows = ops.experts_forward(h, sel, self.gate_up, self.down, s.limit, s.alpha,
                                   ff=s.intermediate if self.tiled else None,
                                   in_weight=weights if s.weight_on_input else None)
        extra = self.shared.forward(ctx, h) if self.shared is not None else None
        if s.weight_on_input:
            weights = None
        if s.identity == 0 and extra is None and weights is not None:
            return RoutedRows(rows, weights)
        return RoutedRows(rows, weights, sel if s.identity else None, s.experts, extra, gate)


@register_ffn("clamped_mlp")
class ClampedMlp(FeedForward):
    """A gated feed-forward in the form of a routed expert, for every token: W_down (g' * sigmoid(alpha g') * (u' + 1)),
    g' = min(W_gate h, limit), u' = clamp(W_up h, -limit, limit).  Gate and up share one product."""
    graph_safe = True

    @classmethod
    def tensors(cls, spec: ClampedMlpSpec) -> Dict[str, TensorSpec]:
        return {"gate": TensorSpec((spec.intermediate, spec.hidden)), "up": TensorSpec((spec.intermediate, spec.hidden)),
                "down": TensorSpec((spec.hidden, spec.intermediate))}

    def __init__(self, spec: ClampedMlpSpec, tensors: Dict[str, torch.Tensor], dtype, device):
        if not spec.limit > 0:
            raise SpecError(f"clamped_mlp: limit {spec.limit} must be positive")
        self.spec = spec
        self.gate_up = Linear([tensors["gate"], tensors["up"]], dtype, device)
        self.down = Linear([tensors["down"]], dtype, device)

    def forward(self, ctx, h):
        if hasattr(h, "materialize"):
            h = h.materialize()
        act = ops.clamped_gate_mul(self.gate_up(h), self.spec.limit, self.spec.alpha)
        if getattr(ctx, "partial_sums", False):
            split = ops.linear_partials(act, self.down.weight, self.down.bias)
            if split is not None:
                return split
        return self.down(act)
