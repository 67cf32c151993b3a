"""A layer whose stream is normed AFTER every sum, around a residual stream kept in 32-bit:

    x <- norm_a(alpha x + mixer(x));   x <- norm_b(alpha x + ffn(x))          (a layer may lack the feed-forward)

Both sub-layers read the stream as it stands.  The stream that this arrangement hands from block to block is the 32-bit
array [tokens, width]; beside it goes the same array once more in the products' precision (`ctx.post_rows`: what the
next sub-layer's products read; in a 32-bit model the stream itself).  One kernel does what stands behind a sub-layer
(`ops.postnorm_step`): it scales the stream, adds the sub-layer's output (a dense one, the weighted rows of routed
experts with the stream's own row for an expert that hands its input on, a shared expert's output beside them), norms
the sum and writes both arrays.  A block leaves nothing to be added: its last kernel has closed the layer.  `enter`
makes the stream from the embedding's rows and `leave` turns the wanted rows into the final norm's output, so the model's
own two ends stay as they are.
"""
from __future__ import annotations

from typing import Dict, Tuple

import torch

from .. import ops
from ..config.spec import LayerSpec, PostNormSpec, SpecError
from ..weights.loader import TensorSpec
from .base import BlockBase, part_class, register_block
from .block import sub_tensors
from .experts import RoutedRows


@register_block("post_norm")
class PostNormBlock(BlockBase):

    @classmethod
    def tensors(cls, spec: LayerSpec) -> Dict[str, TensorSpec]:
        n_norms = 1 if spec.ffn is None else 2
        if len(spec.norms) != n_norms or len(spec.norm_names) != n_norms:
            raise SpecError(f"the arrangement 'post_norm' has {n_norms} norms here, the layer names {len(spec.norms)}")
        out: Dict[str, TensorSpec] = {}
        for local, ts in part_class("mixer", spec.mixer).tensors(spec.mixer).items():
            out[spec.mixer_prefix + local] = ts
        if spec.ffn is not None:
            for local, ts in part_class("ffn", spec.ffn).tensors(spec.ffn).items():
                out[spec.ffn_prefix + local] = ts
        for name, nspec in zip(spec.norm_names, spec.norms):
            (ts,) = part_class("norm", nspec).tensors(nspec).values()
            out[name] = ts
        for name in cls.optional(spec):
            (ts,) = part_class("norm", spec.norms[0]).tensors(spec.norms[0]).values()
            out[name] = ts
        return out

    @classmethod
    def optional(cls, spec: LayerSpec):
        """Names that a file may leave out: the second norm of a layer that has no feed-forward."""
        name = getattr(spec.residual, "bare_norm_name", None)
        return {name} if spec.ffn is None and name else set()

    def __init__(self, spec: LayerSpec, tensors: Dict[str, torch.Tensor], dtype, device):
        self.spec, self.dtype = spec, dtype
        residual = spec.residual if spec.residual is not None else PostNormSpec()
        if not isinstance(residual, PostNormSpec):
            raise SpecError("post_norm: the layer's `residual` is a PostNormSpec (the factor on the stream in every sum)")
        self.alpha = float(residual.alpha)
        self.mixer = part_class("mixer", spec.mixer)(spec.mixer, sub_tensors(tensors, spec.mixer_prefix), dtype, device)
        self.ffn = None
        if spec.ffn is not None:
            self.ffn = part_class("ffn", spec.ffn)(spec.ffn, sub_tensors(tensors, spec.ffn_prefix), dtype, device)
        self.norms = [part_class("norm", nspec)(nspec, {"weight": tensors[name]}, dtype, device)
                      for name, nspec in zip(spec.norm_names, spec.norms)]
        if len(self.norms) != (1 if self.ffn is None else 2):
            raise SpecError("post_norm: a norm behind every sub-layer")
        for name in self.optional(spec):
            if name in tensors:                 # (the file holds a second norm for a layer without a feed-forward)
                self.norms.append(part_class("norm", spec.norms[0])(spec.norms[0], {"weight": tensors[name]}, dtype, device))
        for n in self.norms:
            if getattr(n, "add_one", False) or not hasattr(n, "weight") or not hasattr(n, "eps"):
                raise SpecError("post_norm: the norms must be plain RMS norms")
        self.first_norm = None                      # (no norm reads the stream ahead of this block's parts)

    def parts(self):
        return [self.mixer, self.ffn, *self.norms, getattr(self.mixer, "position", None),
                *getattr(self.mixer, "parts", lambda: [])(), getattr(self.ffn, "shared", None)]

    # ---- the model's two ends ---------------------------------------------------------------------
    def enter(self, ctx, rows: torch.Tensor) -> torch.Tensor:
        """The embedding's rows -> the 32-bit stream; the rows in the products' precision go beside it."""
        if rows.dtype == torch.float32:
            if self.dtype == torch.float32:
                ctx.post_rows = rows
            return rows                              # (an embedding that leaves 32-bit rows has put the others into ctx.post_rows)
        ctx.post_rows = rows
        return ops.widen(rows)

    def leave(self, ctx, x: torch.Tensor, pending, rows: torch.Tensor, norm) -> torch.Tensor:
        """The final norm of the wanted rows (the last block has left nothing to be added)."""
        if pending is not None:
            raise SpecError("post_norm: the block before leaves something that this arrangement does not take")
        if norm is None or getattr(norm, "add_one", False):
            raise SpecError("post_norm: the model ends with a plain RMS norm")
        ctx.post_rows = None
        return ops.postnorm_step(x, weight=norm.weight, eps=norm.eps, h_dtype=self.dtype, rows=rows)

    # ---- a layer ------------------------------------------------------------------------------------
    def _close(self, x: torch.Tensor, out, norm):
        """x <- norm(alpha x + out); returns what the next products read."""
        if out is None:
            extra = {}
        elif isinstance(out, RoutedRows):
            extra = dict(routed=out.rows, routed_weights=out.weights, sel=out.sel, real_experts=out.real_experts, y2=out.extra)
        else:
            # (a product still split along its k is added up by the kernel itself)
            extra = dict(y=out if isinstance(out, ops.Partials) or not hasattr(out, "materialize") else out.materialize())
        h = ops.postnorm_step(x, alpha=self.alpha, weight=norm.weight, eps=norm.eps,
                              h_dtype=None if self.dtype == torch.float32 else self.dtype, **extra)
        return x if h is None else h

    def forward(self, ctx, x: torch.Tensor, pending, cache, next_norm=None) -> Tuple[torch.Tensor, object]:
        if x.dim() != 2 or x.dtype != torch.float32:
            raise SpecError(f"post_norm: the block takes a 32-bit stream [tokens, width], got {tuple(x.shape)} {x.dtype}")
        if pending is not None:
            raise SpecError("post_norm: the block before leaves something that this arrangement does not take")
        ctx.stream = ctx.stream_norm = None
        # steps of few rows: a part's last product may stay split along k (gemm_mid.hip), for `ops.postnorm_step` to add up
        ctx.partial_sums = self.dtype == torch.bfloat16 and ops.MID_MIN_ROWS <= x.shape[0] <= ops.MID_MAX_ROWS
        h = getattr(ctx, "post_rows", None)
        if h is None or h.shape != x.shape:
            h = x if self.dtype == torch.float32 else x.to(self.dtype)
        h = self._close(x, self.mixer.forward(ctx, h, cache), self.norms[0])
        if self.ffn is not None:
            h = self._close(x, self.ffn.forward(ctx, h), self.norms[1])
        elif len(self.norms) > 1:
            h = self._close(x, None, self.norms[1])
        ctx.post_rows = h
        ctx.partial_sums = False
        return x, None
