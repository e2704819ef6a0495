"""A recurrent mixer that writes with the delta rule and forgets with one decay per head and key
channel (the gated delta rule of Yang, Kautz and Hatamizadeh, "Gated Delta Networks: Improving
Mamba2 with Delta Rule", with the scalar decay of a head made a vector over its key channels).

With input h, ``heads`` value heads of ``value_dim`` and ``kv_heads`` query / key heads of
``key_dim`` (value head n reads query / key head ``n // (heads / kv_heads)``):

* ``q = W_q h``, ``k = W_k h``, ``v = W_v h`` (no biases), each through a short causal convolution per
  channel (``q.conv`` ... [channels, taps], the last column on the current token, no bias, zeros
  before the start of a sequence) and silu;
* q and k become unit vectors per head, ``x / sqrt(sum x^2 + 1e-6)``; q is also times ``key_dim^-1/2``;
* ``beta = sigmoid(W_b h)`` per head; ``decay = exp(-exp(A_log_n) softplus(W_a2 (W_a1 h) + dt_bias))`` per
  head and key channel;
* per head, state S [key_dim, value_dim]: ``S <- diag(decay) S``, ``u = beta (v - S^T k)``, ``S <- S + k u^T``,
  ``o = S^T q`` (the read-out sees the current token's write);
* each head's o is RMS-normalised over value_dim with the weight ``norm`` (shared by the heads), times
  ``sigmoid(W_g2 (W_g1 h))``, then ``W_o``.

Unit vectors, beta, decays, the state and the norm are float32 in both compute modes.  A
request's state row holds the three convolutions' last taps - 1 inputs and S, is cleared when the
request is admitted and carried from step to step, so a prompt may be cut anywhere.
"""
from __future__ import annotations

from typing import Dict, List

import torch

from .. import ops
from ..errors import UnsupportedModelError
from ..weights.loader import TensorSpec
from .base import MIXERS, LayerCache, Mixer, StateSpec, StepContext

UNIT_EPS = 1e-6      # inside the root of the unit vectors' length


class ChannelDeltaRule(Mixer):
    graph_safe = True        # slots and request boundaries are read on the device

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, key_dim: int, value_dim: int, conv_taps: int,
                 decay_rank: int, gate_rank: int, eps: float, out_scale: float = 1.0, accumulate: bool = True):
        self.hidden_size, self.num_heads, self.num_kv_heads = int(hidden_size), int(num_heads), int(num_kv_heads)
        self.key_dim, self.value_dim, self.conv_taps = int(key_dim), int(value_dim), int(conv_taps)
        self.decay_rank, self.gate_rank = int(decay_rank), int(gate_rank)
        self.eps, self.out_scale, self.accumulate = float(eps), float(out_scale), bool(accumulate)
        if self.num_heads % self.num_kv_heads:
            raise UnsupportedModelError(f"delta rule: {self.num_heads} heads is not a multiple of {self.num_kv_heads} key heads")
        if not 1 <= self.conv_taps <= ops.CONV_MAX_TAPS or self.key_dim > 256:
            raise UnsupportedModelError(f"delta rule: {self.conv_taps} taps (at most {ops.CONV_MAX_TAPS}), keys of {self.key_dim} (at most 256)")
        self.qk_size, self.v_size = self.num_kv_heads * self.key_dim, self.num_heads * self.value_dim
        self.channels = 2 * self.qk_size + self.v_size                        # what the convolutions see: q | k | v
        self.a_size = self.num_heads * self.key_dim
        self.conv_floats = (self.conv_taps - 1) * self.channels

    def tensor_specs(self) -> List[TensorSpec]:
        D, H, t = self.hidden_size, self.num_heads, self.conv_taps
        return [TensorSpec("q", (self.qk_size, D)), TensorSpec("q.conv", (self.qk_size, t), "taps"),
                TensorSpec("k", (self.qk_size, D)), TensorSpec("k.conv", (self.qk_size, t), "taps"),
                TensorSpec("v", (self.v_size, D)), TensorSpec("v.conv", (self.v_size, t), "taps"),
                TensorSpec("b", (H, D)), TensorSpec("A_log", (H,), "bias"), TensorSpec("norm", (self.value_dim,), "norm"),
                TensorSpec("a1", (self.decay_rank, D)), TensorSpec("a2", (self.a_size, self.decay_rank)),
                TensorSpec("dt_bias", (self.a_size,), "bias"),
                TensorSpec("g1", (self.gate_rank, D)), TensorSpec("g2", (self.v_size, self.gate_rank)),
                TensorSpec("o", (D, self.v_size))]

    def cache_spec(self):
        return StateSpec((self.conv_floats + ops.scan_state_floats(self.num_heads, self.key_dim, self.value_dim),), torch.float32)

    def load(self, tensors: Dict[str, torch.Tensor], dtype, device) -> None:
        super().load(tensors, dtype, device)
        # one projection with float32 results, rows [q | k | v | beta]; one with results in the
        # activation type, rows [a1 | g1], which the two second factors read
        self.w_in = torch.cat([tensors[n] for n in ("q", "k", "v", "b")], dim=0).contiguous()
        self.w_low = torch.cat([tensors["a1"], tensors["g1"]], dim=0).contiguous()
        self.w_a2, self.w_g2, self.w_o = tensors["a2"], tensors["g2"], tensors["o"]
        self.w_conv = torch.cat([tensors[n] for n in ("q.conv", "k.conv", "v.conv")], dim=0).contiguous()
        f32 = lambda t: t.to(torch.float32).contiguous()
        self.dt_bias, self.a_log = f32(tensors["dt_bias"]), f32(tensors["A_log"])
        self.w_norm = f32(tensors["norm"]).repeat(self.num_heads).contiguous()      # per head, as the norm kernel indexes it

    def streamed_weights(self) -> List[torch.Tensor]:
        return [self.w_in, self.w_low, self.w_a2, self.w_g2, self.w_o]

    def forward(self, h: torch.Tensor, x: torch.Tensor, ctx: StepContext, cache: LayerCache) -> None:
        T, ws, C = h.shape[0], ctx.workspace, self.channels
        f32 = lambda n: torch.empty((T, n), dtype=torch.float32, device=h.device)
        proj = f32(C + self.num_heads)
        ops.gemm(proj, h, self.w_in, ws=ws)
        low = torch.empty((T, self.decay_rank + self.gate_rank), dtype=self.dtype, device=h.device)
        ops.gemm(low, h, self.w_low, ws=ws)
        a, gate = f32(self.a_size), f32(self.v_size)
        ops.gemm(a, low[:, :self.decay_rank], self.w_a2, ws=ws)
        ops.gemm(gate, low[:, self.decay_rank:], self.w_g2, ws=ws)
        qkv = f32(C)
        ops.causal_conv_silu(qkv, proj[:, :C], self.w_conv, None, ctx, cache.state[:, :self.conv_floats])
        o = f32(self.v_size)
        ops.delta_scan(o, qkv, a, self.dt_bias, self.a_log, proj[:, C:], ctx, cache.state[:, self.conv_floats:], self.num_heads,
                       self.num_kv_heads, self.key_dim, self.value_dim, self.key_dim ** -0.5, UNIT_EPS)
        y = torch.empty((T, self.v_size), dtype=self.dtype, device=h.device)
        ops.head_norm_gate(y, o, gate, self.w_norm, self.eps, self.num_heads, self.value_dim, self.out_scale)
        ops.gemm(x, y, self.w_o, accumulate=self.accumulate,
                 may_defer=self.accumulate and getattr(ctx, "may_defer", False), ws=ws)


MIXERS.register("channel_delta_rule", ChannelDeltaRule)


class GatedDeltaRule(Mixer):
    """The gated delta rule with one decay per head (the paper's own form), full-rank projections for the decay and
    for a silu output gate:

    * q, k, v as above (convolutions, silu, unit vectors, q times ``key_dim^-1/2``);
    * ``beta = sigmoid(W_b h)`` and ``decay = exp(-exp(A_log_n) softplus(W_a h + dt_bias_n))``, one each per head;
    * per head: ``S <- decay S``, ``u = beta (v - S^T k)``, ``S <- S + k u^T``, ``o = S^T q``;
    * ``y = W_o (silu(W_g h) * concat_n(rms(o_n) * norm))`` with one norm weight of ``value_dim`` for all heads.

    One projection gives everything that is read from h, as float32: rows [q | k | v | b | a | g]."""

    graph_safe = True

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, key_dim: int, value_dim: int, conv_taps: int, eps: float,
                 accumulate: bool = True):
        self.hidden_size, self.num_heads, self.num_kv_heads = int(hidden_size), int(num_heads), int(num_kv_heads)
        self.key_dim, self.value_dim, self.conv_taps = int(key_dim), int(value_dim), int(conv_taps)
        self.eps, self.accumulate = float(eps), bool(accumulate)
        if self.num_heads % self.num_kv_heads:
            raise UnsupportedModelError(f"delta rule: {self.num_heads} heads is not a multiple of {self.num_kv_heads} key heads")
        if not 1 <= self.conv_taps <= ops.CONV_MAX_TAPS or self.key_dim > 256:
            raise UnsupportedModelError(f"delta rule: {self.conv_taps} taps (at most {ops.CONV_MAX_TAPS}), keys of {self.key_dim} (at most 256)")
        self.qk_size, self.v_size = self.num_kv_heads * self.key_dim, self.num_heads * self.value_dim
        self.channels = 2 * self.qk_size + self.v_size
        self.conv_floats = (self.conv_taps - 1) * self.channels

    def tensor_specs(self) -> List[TensorSpec]:
        D, H, t = self.hidden_size, self.num_heads, self.conv_taps
        return [TensorSpec("q", (self.qk_size, D)), TensorSpec("q.conv", (self.qk_size, t), "taps"),
                TensorSpec("k", (self.qk_size, D)), TensorSpec("k.conv", (self.qk_size, t), "taps"),
                TensorSpec("v", (self.v_size, D)), TensorSpec("v.conv", (self.v_size, t), "taps"),
                TensorSpec("b", (H, D)), TensorSpec("A_log", (H,), "bias"), TensorSpec("norm", (self.value_dim,), "norm"),
                TensorSpec("a", (H, D)), TensorSpec("dt_bias", (H,), "bias"), TensorSpec("g", (self.v_size, D)),
                TensorSpec("o", (D, self.v_size))]

    def cache_spec(self):
        return StateSpec((self.conv_floats + ops.scan_state_floats(self.num_heads, self.key_dim, self.value_dim),), torch.float32)

    def load(self, tensors: Dict[str, torch.Tensor], dtype, device) -> None:
        super().load(tensors, dtype, device)
        self.w_in = torch.cat([tensors[n] for n in ("q", "k", "v", "b", "a", "g")], dim=0).contiguous()
        self.w_o = tensors["o"]
        self.w_conv = torch.cat([tensors[n] for n in ("q.conv", "k.conv", "v.conv")], dim=0).contiguous()
        f32 = lambda t: t.to(torch.float32).contiguous()
        self.dt_bias, self.a_log = f32(tensors["dt_bias"]), f32(tensors["A_log"])
        self.w_norm = f32(tensors["norm"]).repeat(self.num_heads).contiguous()      # per head, as the norm kernel indexes it

    def streamed_weights(self) -> List[torch.Tensor]:
        return [self.w_in, self.w_o]

    def forward(self, h: torch.Tensor, x: torch.Tensor, ctx: StepContext, cache: LayerCache) -> None:
        T, ws, C, H = h.shape[0], ctx.workspace, self.channels, self.num_heads
        f32 = lambda n: torch.empty((T, n), dtype=torch.float32, device=h.device)
        proj = f32(C + 2 * H + self.v_size)
        ops.gemm(proj, h, self.w_in, ws=ws)
        qkv = f32(C)
        ops.causal_conv_silu(qkv, proj[:, :C], self.w_conv, None, ctx, cache.state[:, :self.conv_floats])
        o = f32(self.v_size)
        ops.delta_scan(o, qkv, proj[:, C + H:C + 2 * H], self.dt_bias, self.a_log, proj[:, C:C + H], ctx, cache.state[:, self.conv_floats:],
                       H, self.num_kv_heads, self.key_dim, self.value_dim, self.key_dim ** -0.5, UNIT_EPS, kind="head_delta")
        y = torch.empty((T, self.v_size), dtype=self.dtype, device=h.device)
        ops.head_norm_gate(y, o, proj[:, C + 2 * H:], self.w_norm, self.eps, H, self.value_dim, gate="silu")
        ops.gemm(x, y, self.w_o, accumulate=self.accumulate, may_defer=self.accumulate and getattr(ctx, "may_defer", False), ws=ws)


MIXERS.register("gated_delta_rule", GatedDeltaRule)
