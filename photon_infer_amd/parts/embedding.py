"""Token embedding and output head.

Embedding is a row gather without scaling (src/ops/kernels/cuda/embedding_kernel.cu:31-63);
the head is ``logits = h W^T`` in float32 without bias or scaling
(src/arch/llama_model.cpp:256,601).  A tied head uses the embedding's tensor itself
(the reference copies it, src/io/checkpoint.cpp:305-313).
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from .. import ops
from ..weights.loader import TensorSpec
from .base import Part


class TokenEmbedding(Part):
    graph_safe = True

    def __init__(self, vocab_size: int, hidden_size: int, tensor_name: str = "weight", scale: float = 1.0):
        self.vocab_size = int(vocab_size)
        self.hidden_size = int(hidden_size)
        self.tensor_name = tensor_name          # after the part's prefix; may be empty
        self.scale = float(scale)               # a factor on every row as it enters the stream (the table itself stays as stored)
        self.weight: Optional[torch.Tensor] = None

    def tensor_specs(self) -> List[TensorSpec]:
        return [TensorSpec(self.tensor_name, (self.vocab_size, self.hidden_size), "table")]

    def load(self, tensors: Dict[str, torch.Tensor], dtype, device) -> None:
        super().load(tensors, dtype, device)
        self.weight = tensors[self.tensor_name]

    def forward(self, token_ids: torch.Tensor, ctx=None) -> torch.Tensor:
        """int32 [T] -> float32 residual stream [T, hidden].  ``ctx``: the step's context, for
        embeddings that look at more than the ids."""
        x = torch.empty((token_ids.shape[0], self.hidden_size), dtype=torch.float32, device=token_ids.device)
        ops.embedding(x, self.weight, token_ids, self.scale)
        return x


class PositionedEmbedding(TokenEmbedding):
    """``x = norm(table[token] * scale + positions[p])``: a scaled embedding, a learned vector per
    absolute position (not scaled; the table's rows bound the sequence length), and a norm of the
    sum, whose float32 result is the residual stream.  ``norm`` = (tensor name prefix, Norm) or None."""

    def __init__(self, vocab_size: int, hidden_size: int, max_positions: int, scale: float = 1.0, norm=None,
                 tensor_name: str = "weight", position_name: str = "positions"):
        super().__init__(vocab_size, hidden_size, tensor_name, scale)
        self.max_positions = int(max_positions)
        self.position_name = position_name
        self.norm_prefix, self.norm = norm if norm is not None else ("", None)

    def tensor_specs(self) -> List[TensorSpec]:
        specs = super().tensor_specs() + [TensorSpec(self.position_name, (self.max_positions, self.hidden_size), "table")]
        if self.norm is not None:
            specs += [s.with_prefix(self.norm_prefix) for s in self.norm.tensor_specs()]
        return specs

    def load(self, tensors: Dict[str, torch.Tensor], dtype, device) -> None:
        super().load(tensors, dtype, device)
        self.positions = tensors[self.position_name].to(self.weight.dtype)
        if self.norm is not None:
            names = [self.norm_prefix + s.name for s in self.norm.tensor_specs()]
            self.norm.load({n[len(self.norm_prefix):]: tensors[n] for n in names}, dtype, device)

    def forward(self, token_ids: torch.Tensor, ctx=None) -> torch.Tensor:
        x = torch.empty((token_ids.shape[0], self.hidden_size), dtype=torch.float32, device=token_ids.device)
        ops.embedding(x, self.weight, token_ids, self.scale, self.positions, ctx.positions)
        if self.norm is None:
            return x
        out = torch.empty_like(x)
        ops.rmsnorm(out, x, self.norm.weight, self.norm.eps)
        return out


class LMHead(Part):
    graph_safe = True

    def __init__(self, vocab_size: int, hidden_size: int, tied: bool, tensor_name: str = "weight", softcap: Optional[float] = None):
        self.vocab_size = int(vocab_size)
        self.hidden_size = int(hidden_size)
        self.tied = bool(tied)
        self.softcap = float(softcap) if softcap else 0.0     # c > 0: logits become c * tanh(logits / c)
        self.tensor_name = tensor_name          # after the part's prefix; may be empty
        self.weight: Optional[torch.Tensor] = None

    def tensor_specs(self) -> List[TensorSpec]:
        return [] if self.tied else [TensorSpec(self.tensor_name, (self.vocab_size, self.hidden_size))]

    def load(self, tensors: Dict[str, torch.Tensor], dtype, device, tied_weight: Optional[torch.Tensor] = None) -> None:
        super().load(tensors, dtype, device)
        self.weight = tied_weight if self.tied else tensors[self.tensor_name]

    def streamed_weights(self) -> List[torch.Tensor]:
        return [self.weight]

    def forward(self, h: torch.Tensor, ctx=None) -> torch.Tensor:
        """activations [M, hidden] -> float32 logits [M, vocab]."""
        logits = torch.empty((h.shape[0], self.vocab_size), dtype=torch.float32, device=h.device)
        ops.gemm(logits, h, self.weight, ws=ctx.workspace if ctx is not None else None)
        if self.softcap > 0.0:
            ops.softcap_(logits, self.softcap)
        return logits
