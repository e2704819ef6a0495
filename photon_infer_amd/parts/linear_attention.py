"""Gated linear attention: a matrix state per head whose key rows decay, each at its own rate (Yang, Wang, Shen, Panda
and Kim, "Gated Linear Attention Transformers with Hardware-Efficient Training").

With input h, ``heads`` heads with keys of ``key_dim`` and values of ``value_dim``:

* ``q = W_q h * key_dim^-1/2``, ``k = W_k h``, ``v = W_v h`` (no biases);
* a decay per head and key channel, ``alpha = sigmoid(W_a2 (W_a1 h) + b_a2)^(1 / tau)`` (a low-rank projection);
* per head, state S [key_dim, value_dim]: ``S <- diag(alpha) S + k v^T``, ``o = S^T q``;
* ``y = W_o (silu(W_g h) * concat_n(rms(o_n) * norm))``: one norm weight of ``value_dim`` for all heads, the gate over
  all heads' values at once.

Decays, the state and the norm are float32 in both compute modes; q, k and v enter the recurrence as the float32
results of their projection.  A request's state row holds S, is cleared when the request is admitted and carried from
step to step, so a prompt may be cut anywhere.
"""
from __future__ import annotations

from typing import Dict, List

import torch

from .. import ops
from ..errors import UnsupportedModelError
from ..weights.loader import TensorSpec
from .base import MIXERS, LayerCache, Mixer, StateSpec, StepContext


class GatedLinearAttention(Mixer):
    graph_safe = True        # slots and request boundaries are read on the device

    def __init__(self, hidden_size: int, num_heads: int, key_dim: int, value_dim: int, decay_rank: int, tau: float, eps: float,
                 accumulate: bool = True):
        self.hidden_size, self.num_heads = int(hidden_size), int(num_heads)
        self.key_dim, self.value_dim, self.decay_rank = int(key_dim), int(value_dim), int(decay_rank)
        self.tau, self.eps, self.accumulate = float(tau), float(eps), bool(accumulate)
        if not self.tau > 0.0:
            raise UnsupportedModelError(f"gated linear attention: tau must be positive, got {self.tau}")
        if self.key_dim > 256:
            raise UnsupportedModelError(f"gated linear attention: keys of {self.key_dim} (at most 256)")
        self.qk_size, self.v_size = self.num_heads * self.key_dim, self.num_heads * self.value_dim

    def tensor_specs(self) -> List[TensorSpec]:
        D = self.hidden_size
        return [TensorSpec("q", (self.qk_size, D)), TensorSpec("k", (self.qk_size, D)), TensorSpec("v", (self.v_size, D)),
                TensorSpec("g", (self.v_size, D)), TensorSpec("o", (D, self.v_size)), TensorSpec("norm", (self.value_dim,), "norm"),
                TensorSpec("a1", (self.decay_rank, D)), TensorSpec("a2", (self.qk_size, self.decay_rank)),
                TensorSpec("a2.b", (self.qk_size,), "bias")]

    def cache_spec(self):
        return StateSpec((ops.scan_state_floats(self.num_heads, self.key_dim, self.value_dim),), torch.float32)

    def load(self, tensors: Dict[str, torch.Tensor], dtype, device) -> None:
        super().load(tensors, dtype, device)
        # one projection with float32 results, rows [q | k | v | gate]; the decays' first factor gives results in the
        # activation type, which the second factor reads
        self.w_in = torch.cat([tensors[n] for n in ("q", "k", "v", "g")], dim=0).contiguous()
        self.w_a1, self.w_a2, self.w_o = tensors["a1"], tensors["a2"], tensors["o"]
        f32 = lambda t: t.to(torch.float32).contiguous()
        self.a_bias = f32(tensors["a2.b"])
        self.w_norm = f32(tensors["norm"]).repeat(self.num_heads).contiguous()      # per head, as the norm kernel indexes it

    def streamed_weights(self) -> List[torch.Tensor]:
        return [self.w_in, self.w_a1, self.w_a2, self.w_o]

    def forward(self, h: torch.Tensor, x: torch.Tensor, ctx: StepContext, cache: LayerCache) -> None:
        T, ws = h.shape[0], ctx.workspace
        f32 = lambda n: torch.empty((T, n), dtype=torch.float32, device=h.device)
        C = 2 * self.qk_size + self.v_size
        proj = f32(C + self.v_size)
        ops.gemm(proj, h, self.w_in, ws=ws)
        low = torch.empty((T, self.decay_rank), dtype=self.dtype, device=h.device)
        ops.gemm(low, h, self.w_a1, ws=ws)
        a = f32(self.qk_size)
        ops.gemm(a, low, self.w_a2, ws=ws)
        o = f32(self.v_size)
        ops.delta_scan(o, proj[:, :C], a, self.a_bias, None, None, ctx, cache.state, self.num_heads, self.num_heads, self.key_dim,
                       self.value_dim, self.key_dim ** -0.5, 0.0, kind="decayed_outer", tau=self.tau)
        y = torch.empty((T, self.v_size), dtype=self.dtype, device=h.device)
        ops.head_norm_gate(y, o, proj[:, C:], self.w_norm, self.eps, self.num_heads, self.value_dim, gate="silu")
        ops.gemm(x, y, self.w_o, accumulate=self.accumulate, may_defer=self.accumulate and getattr(ctx, "may_defer", False), ws=ws)


MIXERS.register("gated_linear_attention", GatedLinearAttention)
