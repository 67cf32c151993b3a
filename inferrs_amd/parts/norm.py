"""RMS norm: x / sqrt(mean(x^2) + eps) * w, statistics in 32-bit
(`candle-nn/src/ops.rs:443-504`, `inferrs-kernels/candle-kernels/src/reduce.cu:189-228`); and a layer norm with weight
and bias, (x - mean) / sqrt(var + eps) * w + b, for streams kept in 32-bit.

A norm's first tensor, "weight", is stored under the name the layer gives the norm; a norm with more tensors names a
suffix for each (`file_names`)."""
from __future__ import annotations

from typing import Dict

import torch

from .. import ops
from ..config.spec import LayerNormSpec, NormSpec, SpecError
from ..weights.loader import TensorSpec
from .base import Norm, part_class, register_norm


@register_norm("rmsnorm")
class RMSNorm(Norm):
    graph_safe = True

    @classmethod
    def tensors(cls, spec: NormSpec) -> Dict[str, TensorSpec]:
        return {"weight": TensorSpec((spec.size,), "norm")}

    def __init__(self, spec: NormSpec, tensors: Dict[str, torch.Tensor], dtype, device):
        self.spec = spec
        self.eps = float(spec.eps)
        self.add_one = bool(spec.add_one)
        # Norm weights are vectors: kept in 32-bit whatever the activations are stored in.
        self.weight = tensors["weight"].to(device=device, dtype=torch.float32).contiguous()

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return ops.rmsnorm(x, self.weight, self.eps, self.add_one)

    def add_forward(self, x: torch.Tensor, delta: torch.Tensor) -> torch.Tensor:
        return ops.add_rmsnorm(x, delta, self.weight, self.eps, self.add_one)

    def add_forward_partials(self, x: torch.Tensor, delta: "ops.Partials") -> torch.Tensor:
        """`add_forward` for a product that is still split along k."""
        return ops.add_rmsnorm_partials(x, delta, self.weight, self.eps, self.add_one)

    def rows_for_product(self, x: torch.Tensor, added: "ops.Added") -> ops.NormedRows:
        """The norm of a stream's rows left to the product that reads them: `added` holds the rows times
        this norm's weight and their sums of squares."""
        return ops.NormedRows(x, added.scaled, added.sums, self.weight, self.eps, self.add_one)


def file_names(name: str, spec) -> Dict[str, str]:
    """A norm's tensors (as its part names them) -> their names in the file, for a norm stored under `name`."""
    cls = part_class("norm", spec)
    suffixes = cls.suffixes(spec) if hasattr(cls, "suffixes") else {}
    return {local: name + suffixes.get(local, "") for local in cls.tensors(spec)}


def norm_tensors(name: str, spec) -> Dict[str, TensorSpec]:
    """The tensors of a norm stored under `name`, by their names in the file."""
    specs = part_class("norm", spec).tensors(spec)
    return {full: specs[local] for local, full in file_names(name, spec).items()}


def build_norm(name: str, spec, tensors: Dict[str, torch.Tensor], dtype, device, pop: bool = False):
    """The norm part stored under `name`, its tensors taken from `tensors` (by file name; `pop`: removed from there)."""
    take = tensors.pop if pop else tensors.__getitem__
    return part_class("norm", spec)(spec, {local: take(full) for local, full in file_names(name, spec).items()}, dtype, device)


@register_norm("layernorm")
class LayerNorm(Norm):
    """(x - mean) / sqrt(var + eps) * w + b over a 32-bit stream's rows; the rows leave in the products' precision."""
    graph_safe = True

    @classmethod
    def tensors(cls, spec: LayerNormSpec) -> Dict[str, TensorSpec]:
        return {"weight": TensorSpec((spec.size,), "norm"), "bias": TensorSpec((spec.size,), "bias")}

    @classmethod
    def suffixes(cls, spec: LayerNormSpec) -> Dict[str, str]:
        return {"bias": spec.bias_suffix}

    def __init__(self, spec: LayerNormSpec, tensors: Dict[str, torch.Tensor], dtype, device):
        self.spec = spec
        self.eps = float(spec.eps)
        self.dtype = dtype
        self.weight = tensors["weight"].to(device=device, dtype=torch.float32).contiguous()
        self.bias = tensors["bias"].to(device=device, dtype=torch.float32).contiguous()

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if x.dtype != torch.float32:
            raise SpecError("layernorm: the rows of a 32-bit stream")
        return ops.parallel_step(x, norm_weight=self.weight, norm_bias=self.bias, norm_eps=self.eps, h_dtype=self.dtype)[1]
