"""Gated feed-forward (SwiGLU).

Formula (src/arch/transformer_block.cpp:282-295, include/photon/ops/kernels/swiglu_kernel.hpp:52-76):
``g = h W1^T``, ``u = h W3^T``, ``a = g / (1 + exp(-g)) * u``, ``x += a W2^T``; no bias.
Tensor names: ``gate_proj`` = W1, ``up_proj`` = W3, ``down_proj`` = W2.  The sigmoid
and the product run in float32.
"""
from __future__ import annotations

from typing import Dict, List

import torch

from .. import ops
from ..errors import UnsupportedModelError
from ..weights.loader import TensorSpec
from .base import FEED_FORWARDS, FeedForward, StepContext

INTERLEAVE = 16   # rows of a matrix-core tile


class SwiGLU(FeedForward):
    graph_safe = True

    def __init__(self, hidden_size: int, intermediate_size: int, activation: str = "silu",
                 names=("gate_proj.weight", "up_proj.weight", "down_proj.weight"), accumulate: bool = True):
        """``names``: the gate, up and down matrices' names after the part's prefix.
        ``accumulate`` False: ``forward`` writes its result into the tensor it is given instead of
        adding to it (for arrangements that normalise a sublayer's result before the residual add)."""
        if activation != "silu":
            raise UnsupportedModelError(f"gated feed-forward activation '{activation}' is not supported")
        self.hidden_size = int(hidden_size)
        self.intermediate_size = int(intermediate_size)
        self.names = tuple(names)
        self.accumulate = bool(accumulate)

    def tensor_specs(self) -> List[TensorSpec]:
        I, D = self.intermediate_size, self.hidden_size
        return [
            TensorSpec(self.names[0], (I, D)),
            TensorSpec(self.names[1], (I, D)),
            TensorSpec(self.names[2], (D, I)),
        ]

    def load(self, tensors: Dict[str, torch.Tensor], dtype, device) -> None:
        super().load(tensors, dtype, device)
        g, u = tensors[self.names[0]], tensors[self.names[1]]
        common = torch.float32 if torch.float32 in (g.dtype, u.dtype) else g.dtype
        g, u = g.to(common), u.to(common)
        I = self.intermediate_size
        if common == torch.bfloat16 and I % INTERLEAVE == 0:
            # one projection for gate and up, rows interleaved in blocks of 16 (gate block, up
            # block, ...): the matrix-core kernels then hold a feature's gate and up value in
            # the same lane and apply the activation before anything is stored
            self.interleave = INTERLEAVE
            self.w_gate_up = torch.stack([g.view(I // INTERLEAVE, INTERLEAVE, -1), u.view(I // INTERLEAVE, INTERLEAVE, -1)],
                                         dim=1).reshape(2 * I, -1).contiguous()
        else:
            self.interleave = 0                      # rows [gate | up]
            self.w_gate_up = torch.cat([g, u], dim=0).contiguous()
        self.w_down = tensors[self.names[2]]

    def streamed_weights(self) -> List[torch.Tensor]:
        return [self.w_gate_up, self.w_down]

    def forward(self, h: torch.Tensor, x: torch.Tensor, ctx: StepContext) -> None:
        act = torch.empty((h.shape[0], self.intermediate_size), dtype=self.dtype, device=h.device)
        ws = ctx.workspace if ctx is not None else None
        ops.gemm_swiglu(act, h, self.w_gate_up, self.interleave, ws=ws)
        ops.gemm(x, act, self.w_down, accumulate=self.accumulate,
                 may_defer=self.accumulate and getattr(ctx, "may_defer", False), ws=ws)


FEED_FORWARDS.register("swiglu", SwiGLU)


class ClampedGLU(FeedForward):
    """A gated feed-forward with biases, clamped before the gate's activation:

        g = min(W_gate h + b_gate, limit);  u = clamp(W_up h + b_up, -limit, limit)
        y = g * sigmoid(alpha * g) * (u + 1);  x += W_down y + b_down

    ``limit`` and ``alpha`` are parameters.  Biases are added and the unit is computed in float32
    from the float32 results of the one gate | up product; the down projection's bias joins the
    stream in the same kernel, so that the product only accumulates."""

    graph_safe = True

    def __init__(self, hidden_size: int, intermediate_size: int, limit: float, alpha: float = 1.702,
                 names=("gate", "up", "down"), bias_suffix: str = ".b"):
        self.hidden_size, self.intermediate_size = int(hidden_size), int(intermediate_size)
        self.limit, self.alpha = float(limit), float(alpha)
        self.names, self.bias_suffix = tuple(names), bias_suffix
        self.accumulate = True           # adds into the stream; there is no writing form

    def tensor_specs(self) -> List[TensorSpec]:
        I, D, b = self.intermediate_size, self.hidden_size, self.bias_suffix
        g, u, d = self.names
        return [TensorSpec(g, (I, D)), TensorSpec(g + b, (I,), "small_bias"), TensorSpec(u, (I, D)), TensorSpec(u + b, (I,), "small_bias"),
                TensorSpec(d, (D, I)), TensorSpec(d + b, (D,), "small_bias")]

    def load(self, tensors: Dict[str, torch.Tensor], dtype, device) -> None:
        super().load(tensors, dtype, device)
        g, u, d = self.names
        wg, wu = tensors[g], tensors[u]
        common = torch.float32 if torch.float32 in (wg.dtype, wu.dtype) else wg.dtype
        wg, wu, I = wg.to(common), wu.to(common), self.intermediate_size
        f32 = lambda t: t.to(torch.float32).contiguous()
        bg, bu = f32(tensors[g + self.bias_suffix]), f32(tensors[u + self.bias_suffix])
        if common == torch.bfloat16 and I % INTERLEAVE == 0:
            # one projection for gate and up, rows (and biases) interleaved in blocks of 16: the matrix-core kernels
            # then hold a feature's gate and up value in the same lane and apply the unit before anything is stored
            self.interleave = INTERLEAVE
            pair = lambda a, b: torch.stack([a.view(I // INTERLEAVE, INTERLEAVE, -1), b.view(I // INTERLEAVE, INTERLEAVE, -1)], dim=1)
            self.w_gate_up = pair(wg, wu).reshape(2 * I, -1).contiguous()
            self.b_gate_up = pair(bg, bu).reshape(2 * I).contiguous()
        else:
            self.interleave = 0                      # rows [gate | up]
            self.w_gate_up = torch.cat([wg, wu], dim=0).contiguous()
            self.b_gate_up = torch.cat([bg, bu]).contiguous()
        self.w_down, self.b_down = tensors[d], f32(tensors[d + self.bias_suffix])

    def streamed_weights(self) -> List[torch.Tensor]:
        return [self.w_gate_up, self.w_down]

    def forward(self, h: torch.Tensor, x: torch.Tensor, ctx: StepContext) -> None:
        ws = ctx.workspace if ctx is not None else None
        act = torch.empty((h.shape[0], self.intermediate_size), dtype=self.dtype, device=h.device)
        # the down projection's bias is added to the stream itself on the way, so that the product only accumulates
        ops.gemm_clamped_glu(act, h, self.w_gate_up, self.b_gate_up, self.limit, self.alpha, self.interleave, ws=ws,
                             x=x, x_bias=self.b_down)
        ops.gemm(x, act, self.w_down, accumulate=True, may_defer=getattr(ctx, "may_defer", False), ws=ws)


FEED_FORWARDS.register("clamped_glu", ClampedGLU)


class SquaredReluMLP(FeedForward):
    """A feed-forward without a gate: ``y = W_down act(W_up h)`` with ``act(z) = max(z, 0)^2``, no biases.  The square
    is taken on the product's float32 result, before the one rounding.  ``accumulate`` False: the result is written
    into the tensor handed to ``forward`` instead of added to it."""

    graph_safe = True

    def __init__(self, hidden_size: int, intermediate_size: int, names=("up", "down"), accumulate: bool = True):
        self.hidden_size, self.intermediate_size = int(hidden_size), int(intermediate_size)
        self.names, self.accumulate = tuple(names), bool(accumulate)

    def tensor_specs(self) -> List[TensorSpec]:
        I, D = self.intermediate_size, self.hidden_size
        return [TensorSpec(self.names[0], (I, D)), TensorSpec(self.names[1], (D, I))]

    def load(self, tensors: Dict[str, torch.Tensor], dtype, device) -> None:
        super().load(tensors, dtype, device)
        self.w_up, self.w_down = tensors[self.names[0]], tensors[self.names[1]]

    def streamed_weights(self) -> List[torch.Tensor]:
        return [self.w_up, self.w_down]

    def forward(self, h: torch.Tensor, x: torch.Tensor, ctx: StepContext) -> None:
        ws = ctx.workspace if ctx is not None else None
        act = torch.empty((h.shape[0], self.intermediate_size), dtype=self.dtype, device=h.device)
        ops.gemm_relu_squared(act, h, self.w_up, ws=ws)
        ops.gemm(x, act, self.w_down, accumulate=self.accumulate,
                 may_defer=self.accumulate and getattr(ctx, "may_defer", False), ws=ws)


FEED_FORWARDS.register("squared_relu_mlp", SquaredReluMLP)
