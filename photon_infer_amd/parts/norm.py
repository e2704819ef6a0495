"""Normalisation parts: RMS norm, and layer norm with weight and bias.

Formula (include/photon/ops/kernels/rmsnorm_kernel.hpp:55-87): mean of squares over
the row, ``rms = sqrt(mean + eps)`` with eps inside the root, ``y = w * (x / rms)``;
no mean-centring, no bias.  A model that stores its weights around zero uses ``offset + w``.  Sum, root and scaling run in float32; the result is
rounded once to the compute dtype.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from .. import ops
from ..weights.loader import TensorSpec
from .base import NORMS, Norm


class RMSNorm(Norm):
    consumes_deferred = True   # reads the stream through ops.rmsnorm, which adds a pending update
    graph_safe = True

    def __init__(self, dim: int, eps: float, offset: float = 0.0, tensor_name: str = "weight"):
        """``offset``: what is added to the stored weight (1.0 for weights stored around zero, used
        as 1 + w); the sum is made and kept in float32.  ``tensor_name``: the weight's name
        after the part's prefix (may be empty: the prefix is the name)."""
        self.dim = int(dim)
        self.eps = float(eps)
        self.offset = float(offset)
        self.tensor_name = tensor_name
        self.weight: Optional[torch.Tensor] = None

    def tensor_specs(self) -> List[TensorSpec]:
        return [TensorSpec(self.tensor_name, (self.dim,), "norm_zero" if self.offset else "norm")]

    def load(self, tensors: Dict[str, torch.Tensor], dtype, device) -> None:
        super().load(tensors, dtype, device)
        self.weight = tensors[self.tensor_name]
        if self.offset:
            self.weight = (self.weight.to(torch.float32) + self.offset).contiguous()

    def weight_f32(self) -> torch.Tensor:
        """The weight as the kernels that want float32 weights take it (made once)."""
        if getattr(self, "_w32", None) is None:
            self._w32 = self.weight.to(torch.float32).contiguous()
        return self._w32

    def forward(self, x: torch.Tensor, ctx=None, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        m = x.shape[0] if rows is None else rows.shape[0]
        out = torch.empty((m, self.dim), dtype=self.dtype, device=x.device)
        ops.rmsnorm(out, x, self.weight, self.eps, rows, ws=ctx.workspace if ctx is not None else None)
        return out


NORMS.register("rmsnorm", RMSNorm)


class LayerNorm(Norm):
    """Layer norm with weight and bias: ``(x - mean) / sqrt(variance + eps) * w + b``, the variance the mean of the
    squared deviations; mean, variance and scaling in float32, rounded once to the compute dtype.
    ``tensor_name``: the weight's name after the part's prefix (may be empty: the prefix is the name); the bias is
    that name plus ``bias_suffix``."""

    graph_safe = True

    def __init__(self, dim: int, eps: float, tensor_name: str = "weight", bias_suffix: str = ".b"):
        self.dim, self.eps = int(dim), float(eps)
        self.tensor_name, self.bias_name = tensor_name, tensor_name + bias_suffix
        self.weight: Optional[torch.Tensor] = None
        self.bias: Optional[torch.Tensor] = None

    def tensor_specs(self) -> List[TensorSpec]:
        return [TensorSpec(self.tensor_name, (self.dim,), "norm"), TensorSpec(self.bias_name, (self.dim,), "small_bias")]

    def load(self, tensors: Dict[str, torch.Tensor], dtype, device) -> None:
        super().load(tensors, dtype, device)
        self.weight = tensors[self.tensor_name].to(torch.float32).contiguous()
        self.bias = tensors[self.bias_name].to(torch.float32).contiguous()

    def weight_bias_f32(self):
        """(weight, bias) as the kernels that fold this norm into another pass take them."""
        return self.weight, self.bias

    def forward(self, x: torch.Tensor, ctx=None, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        m = x.shape[0] if rows is None else rows.shape[0]
        out = torch.empty((m, self.dim), dtype=self.dtype, device=x.device)
        ops.layer_norm(out, x, self.weight, self.bias, self.eps, rows)
        return out


NORMS.register("layernorm", LayerNorm)
