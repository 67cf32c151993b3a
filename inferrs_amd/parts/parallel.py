"""A layer whose two sub-layers read ONE normed copy of a residual stream kept in 32-bit, their outputs added together:

    h = norm(x);   x <- x + mixer(h) + ffn(h)                      (a layer may lack the feed-forward)
    x <- x + rmsnorm(W_proj (act(W_gate x) * e)) * w               (optional: what the token itself adds behind the sum;
                                                                    e is the layer's slice of a second embedding table's row)

The stream that this arrangement hands from block to block is the 32-bit array [tokens, width].  One kernel
(`ops.parallel_step`) adds a layer's outputs up (a dense output or one still split along its k, the rows of routed
experts, a shared expert's output times its gate a token), takes the token's row in through its norm, and forms the
normed rows that the NEXT layer's sub-layers read; where a token's row enters it runs twice a layer, the small products
of that row between the two runs.  A block leaves the normed rows for its successor in `ctx.normed` together with the
norm part they went through; a block that does not find its own norm there norms the stream itself (the first layer).
`enter` makes the stream from the embedding's rows and `leave` turns the wanted rows into the final norm's output, so the
model's own two ends stay as they are.
"""
from __future__ import annotations

from typing import Dict, Tuple

import torch

from .. import ops
from ..config.spec import LayerSpec, ParallelSpec, SpecError
from ..weights.loader import TensorSpec
from .base import BlockBase, part_class, register_block
from .block import sub_tensors
from .experts import RoutedRows
from .linear import Linear
from .norm import build_norm, norm_tensors


@register_block("parallel")
class ParallelBlock(BlockBase):

    @classmethod
    def tensors(cls, spec: LayerSpec) -> Dict[str, TensorSpec]:
        if len(spec.norms) != 1 or len(spec.norm_names) != 1:
            raise SpecError(f"the arrangement 'parallel' has one norm, the layer names {len(spec.norms)}")
        out: Dict[str, TensorSpec] = {}
        for local, ts in part_class("mixer", spec.mixer).tensors(spec.mixer).items():
            out[spec.mixer_prefix + local] = ts
        if spec.ffn is not None:
            for local, ts in part_class("ffn", spec.ffn).tensors(spec.ffn).items():
                out[spec.ffn_prefix + local] = ts
        out.update(norm_tensors(spec.norm_names[0], spec.norms[0]))
        side = getattr(spec.residual, "side", None)
        if side is not None:
            hidden = spec.norms[0].size
            out[side.prefix + "gate"] = TensorSpec((side.dim, hidden))
            out[side.prefix + "proj"] = TensorSpec((hidden, side.dim))
            out[side.prefix + "norm"] = TensorSpec((hidden,), "norm")
        return out

    def __init__(self, spec: LayerSpec, tensors: Dict[str, torch.Tensor], dtype, device):
        self.spec, self.dtype = spec, dtype
        residual = spec.residual if spec.residual is not None else ParallelSpec()
        if not isinstance(residual, ParallelSpec):
            raise SpecError("parallel: the layer's `residual` is a ParallelSpec")
        self.mixer = part_class("mixer", spec.mixer)(spec.mixer, sub_tensors(tensors, spec.mixer_prefix), dtype, device)
        self.ffn = None
        if spec.ffn is not None:
            self.ffn = part_class("ffn", spec.ffn)(spec.ffn, sub_tensors(tensors, spec.ffn_prefix), dtype, device)
        self.norm = build_norm(spec.norm_names[0], spec.norms[0], tensors, dtype, device)
        _norm_args(self.norm)                        # (refuses a norm this arrangement's kernel does not form)
        self.first_norm = self.norm
        self.side = residual.side
        if self.side is not None:
            if self.side.activation not in ops.ACTIVATIONS:
                raise SpecError(f"parallel: activation {self.side.activation!r} has no kernel (known: {sorted(ops.ACTIVATIONS)})")
            p = self.side.prefix
            self.side_gate = Linear([tensors[p + "gate"]], dtype, device)
            self.side_proj = Linear([tensors[p + "proj"]], dtype, device)
            self.side_norm_w = tensors[p + "norm"].to(device=device, dtype=torch.float32).contiguous()

    graph_safe = True

    def parts(self):
        return [self, self.mixer, self.ffn, self.norm, getattr(self.mixer, "position", None),
                *getattr(self.mixer, "parts", lambda: [])(), getattr(self.ffn, "shared", None)]

    # ---- the model's two ends ---------------------------------------------------------------------
    def enter(self, ctx, rows: torch.Tensor) -> torch.Tensor:
        """The embedding's rows -> the 32-bit stream."""
        ctx.normed = None
        return rows if rows.dtype == torch.float32 else ops.widen(rows)

    def leave(self, ctx, x: torch.Tensor, pending, rows: torch.Tensor, norm) -> torch.Tensor:
        """The final norm of the wanted rows (the last block has left nothing to be added)."""
        if pending is not None:
            raise SpecError("parallel: the block before leaves something that this arrangement does not take")
        if norm is None:
            raise SpecError("parallel: the model ends with a norm")
        ctx.normed = None
        return ops.parallel_step(x, rows=rows, h_dtype=self.dtype, **_norm_args(norm))[1]

    # ---- a layer ------------------------------------------------------------------------------------
    def forward(self, ctx, x: torch.Tensor, pending, cache, next_norm=None) -> Tuple[torch.Tensor, object]:
        if x.dim() != 2 or x.dtype != torch.float32:
            raise SpecError(f"parallel: the block takes a 32-bit stream [tokens, width], got {tuple(x.shape)} {x.dtype}")
        if pending is not None:
            raise SpecError("parallel: the block before leaves something that this arrangement does not take")
        ctx.stream = ctx.stream_norm = None
        # steps of few rows: a part's last product may stay split along k (gemm_mid.hip), for `ops.parallel_step` to add up
        ctx.partial_sums = self.dtype == torch.bfloat16 and ops.MID_MIN_ROWS <= x.shape[0] <= ops.MID_MAX_ROWS
        ready = getattr(ctx, "normed", None)
        if ready is not None and ready[0] is self.norm and ready[1].shape == x.shape:
            h = ready[1]
        else:
            h = ops.parallel_step(x, h_dtype=self.dtype, **_norm_args(self.norm))[1]
        ctx.normed = None
        adds = dict(y1=_dense(self.mixer.forward(ctx, h, cache)))
        if self.ffn is not None:
            out = self.ffn.forward(ctx, h)
            if isinstance(out, RoutedRows):
                if out.sel is not None:
                    raise SpecError("parallel: experts that hand their input on are not taken by this arrangement")
                adds.update(routed=out.rows, routed_weights=out.weights, y3=_dense(out.extra), y3_scale=out.extra_scale)
            else:
                adds["y2"] = _dense(out)
        ctx.partial_sums = False
        follow = _norm_args(next_norm) if next_norm is not None else {}
        h_dtype = self.dtype if next_norm is not None else None
        if self.side is None:
            _, h_next = ops.parallel_step(x, h_dtype=h_dtype, **adds, **follow)
        else:
            if getattr(ctx, "side_rows", None) is None:
                raise SpecError("parallel: the token's own input needs an embedding that hands out its second table's rows")
            xr, _ = ops.parallel_step(x, x_dtype=self.dtype, **adds)
            gated = ops.gate_rows(self.side_gate(xr), ctx.side_rows, self.side.offset, self.side.activation)
            _, h_next = ops.parallel_step(x, enter=self.side_proj(gated), enter_weight=self.side_norm_w,
                                          enter_eps=self.side.eps, h_dtype=h_dtype, **follow)
        if next_norm is not None:
            ctx.normed = (next_norm, h_next)
        return x, None


def _dense(out):
    """A sub-layer's dense output as `ops.parallel_step` takes it: rows, or a product still split along its k."""
    if out is None or isinstance(out, ops.Partials) or not hasattr(out, "materialize"):
        return out
    return out.materialize()


def _norm_args(norm) -> dict:
    """The norm at the end of `ops.parallel_step`: a layer norm with weight and bias, or a plain RMS norm."""
    if getattr(norm, "add_one", False) or not hasattr(norm, "weight") or not hasattr(norm, "eps"):
        raise SpecError("parallel: the norms are layer norms with weight and bias, or plain RMS norms")
    bias = getattr(norm, "bias", None)
    return dict(norm_weight=norm.weight, norm_bias=bias, norm_eps=norm.eps, center=getattr(norm, "kind", "") == "layernorm")
