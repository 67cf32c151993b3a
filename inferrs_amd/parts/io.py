"""The two ends of a decoder: token ids into the stream (`inferrs-models/src/models/qwen3.rs:398-405`,
a gather without scaling) and normed rows into logits (`qwen3.rs:369-372`, `attention_utils.rs:382-395`:
a product with the head's matrix, or with the embedding table when the file holds no head).  Both are
registered parts, so a model whose ends differ (a scaled embedding, capped logits) brings its own."""
from __future__ import annotations

from typing import Dict

import torch

from .. import ops
from ..weights.loader import TensorSpec
from .base import Embedding, Head, Part, register_embedding, register_head, register_pass_input
from .linear import Linear, to_compute


@register_embedding("embedding")
class TableEmbedding(Embedding):
    graph_safe = True

    @classmethod
    def tensors(cls, spec) -> Dict[str, TensorSpec]:
        t = {spec.name: TensorSpec((spec.vocab_size, spec.hidden), "matrix")}
        if getattr(spec, "side_name", None):
            t[spec.side_name] = TensorSpec((spec.vocab_size, spec.side_width), "matrix")
        return t

    def __init__(self, spec, tensors: Dict[str, torch.Tensor], dtype, device):
        self.spec = spec
        self.table = to_compute(tensors[spec.name], dtype, device)
        # a second table whose rows for the step's tokens the layers take slices of (`ctx.side_rows`)
        self.side_table = to_compute(tensors[spec.side_name], dtype, device) if getattr(spec, "side_name", None) else None

    def forward(self, ctx) -> torch.Tensor:
        if self.side_table is not None:
            ctx.side_rows = ops.embed_gather(self.side_table, ctx.token_ids)
        scale, wide = float(getattr(self.spec, "scale", 1.0)), bool(getattr(self.spec, "wide", False))
        if wide:
            # 32-bit rows for a stream that is kept so: the factor meets the table's values unrounded
            if self.table.dtype == torch.float32:
                return ops.embed_gather_scaled(self.table, ctx.token_ids, scale)
            rows, ctx.post_rows = ops.embed_gather_scaled(self.table, ctx.token_ids, scale, rounded=True)
            return rows
        rows = ops.embed_gather(self.table, ctx.token_ids)
        if scale != 1.0:
            rows = ops.embed_gather_scaled(self.table, ctx.token_ids, scale).to(rows.dtype)
        return rows


@register_head("lm_head")
class LinearHead(Head):
    graph_safe = True

    @classmethod
    def tensors(cls, spec) -> Dict[str, TensorSpec]:
        if spec.name is None:
            return {}
        return {spec.name: TensorSpec((spec.vocab_size, spec.hidden), "matrix")}

    @classmethod
    def optional(cls, spec):
        """Names that a file may leave out: the embedding table then serves, as in the reference, which
        decides by the tensor's presence alone."""
        return set() if spec.name is None else {spec.name}

    @classmethod
    def generated(cls, spec):
        """Names that a random model is written with."""
        return {spec.name} if spec.name is not None and spec.required else set()

    def __init__(self, spec, tensors: Dict[str, torch.Tensor], dtype, device, embedding=None):
        self.spec = spec
        own = tensors.get(spec.name) if spec.name is not None else None
        if own is not None:
            self.weight = Linear([own], dtype, device).weight
        else:
            table = getattr(embedding, "table", None)
            if table is None or tuple(table.shape) != (spec.vocab_size, spec.hidden):
                raise ValueError("the logits head has no matrix of its own and the embedding offers no table of "
                                 f"[{spec.vocab_size}, {spec.hidden}] to share")
            self.weight = table                      # logits share the embedding table

    def forward(self, rows: torch.Tensor) -> torch.Tensor:
        logits = ops.linear(rows, self.weight, torch.float32)
        scale = float(getattr(self.spec, "scale", 1.0))
        return logits if scale == 1.0 else ops.scale_inplace(logits, scale)


@register_head("capped_lm_head")
class CappedHead(LinearHead):
    """A product with the head's matrix, then cap * tanh(logits / cap) (`spec.cap` None: no cap)."""

    def forward(self, rows: torch.Tensor) -> torch.Tensor:
        logits = super().forward(rows)
        if self.spec.cap is not None:
            ops.softcap(logits, float(self.spec.cap))
        return logits


@register_pass_input("pass_input")
class PassInput(Part):
    """What enters the stream before pass t over a looped range of layers: row t of a [times, hidden] tensor (kept in
    32-bit) and, before every pass but the first, the embedding's rows once more.  The block that runs first in the pass
    adds them."""
    graph_safe = True

    @classmethod
    def tensors(cls, spec) -> Dict[str, TensorSpec]:
        return {spec.name: TensorSpec((spec.times, spec.hidden), "matrix")}

    def __init__(self, spec, tensors: Dict[str, torch.Tensor], dtype, device):
        self.spec = spec
        self.steps = tensors[spec.name].to(device=device, dtype=torch.float32).contiguous()

    def inputs(self, first_rows: torch.Tensor, t: int):
        if not (0 <= t < self.spec.times):
            raise ValueError(f"pass {t} of a range that runs {self.spec.times} times")
        return (first_rows if self.spec.readd_embedding and t > 0 else None), self.steps[t]
