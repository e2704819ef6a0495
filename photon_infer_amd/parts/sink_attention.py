"""Windowed grouped-query attention without rotation: positions enter through a distance bias
and a query temperature; the softmax has a sink; every head has an output gate.

For a token at position p with input h (the constants are constructor parameters):

* ``q = Wq h``, ``k = Wk h``, ``v = Wv h`` (no biases); keys and queries of size ``head_dim``,
  values of size ``value_dim``; query head n reads kv head ``n // (heads / kv_heads)``;
* q and k are each RMS-normalised over their WHOLE projection (all heads at once, before the
  split into heads) with plain weights ``q.norm`` / ``k.norm``;
* q is multiplied by ``1 + temp_coef * ln(floor((p + 1) / temp_every) + 1)``;
* ``score(p, t) = scale * <q, k_t> - slope_n * (p - t)`` with ``slope_n = 2^(-8 (n + 1) / heads)``,
  for the keys ``p - window < t <= p``;
* weights ``exp(score) / (sum_t exp(score) + exp(sink_n))``: the sink has no key and no value;
* head n's output is multiplied by ``sigmoid(Wg h)_n``; then ``Wo`` on the concatenated heads.

Scores, softmax, norms, temperature and gates are float32 in both compute modes.  Keys are
stored normalised, values as they are, in pages; the window lets the cache manager give pages
back while a request runs.

Further options, each a constructor parameter:

* ``norm_per_head``: every head of q and of k is divided by the root mean square of its own
  ``head_dim`` entries instead of the whole projection's; ``norm_weights`` False: the norms have
  no weights (no tensors ``q.norm`` / ``k.norm``);
* ``softcap`` c: the scaled score s becomes ``c * tanh(s / c)`` before the softmax;
* ``chunk`` C: positions are cut into chunks of C, counted from position 0 of the sequence, and a
  token sees the keys ``floor(p / C) * C <= t <= p`` of its own chunk only;
* ``own_kv`` False: the layer has no k and v projections and attends, with its own queries, mask,
  sink and gate, over the keys (as cached, normalised) and values of the layer whose cache the
  run order hands it;
* ``cache_reach``: how many positions back the cache must keep (default: the window, or the chunk:
  a chunk never reaches further back than its own size; None with neither).  A layer whose cache
  other layers read names the longest reach among them.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from .. import ops
from ..errors import UnsupportedModelError
from ..weights.loader import TensorSpec
from .base import MIXERS, PAGE, LayerCache, Mixer, PagedCacheSpec, PagedTensor, StepContext


def distance_slopes(num_heads: int) -> torch.Tensor:
    """slope_n = 2^(-8 (n + 1) / heads), n = 0 .. heads-1, float32."""
    n = torch.arange(1, num_heads + 1, dtype=torch.float64)
    return torch.pow(2.0, -8.0 * n / num_heads).to(torch.float32)


class SinkWindowAttention(Mixer):
    graph_safe = True        # every kernel takes positions, requests and pages from device memory

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int, value_dim: int, scale: float,
                 window: Optional[int], eps: float, temp_coef: float = 0.0, temp_every: int = 1, qk_norm: bool = True,
                 distance_bias: bool = True, sink: bool = True, output_gate: bool = True, accumulate: bool = True,
                 norm_per_head: bool = False, norm_weights: bool = True, softcap: Optional[float] = None,
                 chunk: Optional[int] = None, own_kv: bool = True, cache_reach="own"):
        self.hidden_size, self.num_heads, self.num_kv_heads = int(hidden_size), int(num_heads), int(num_kv_heads)
        self.head_dim, self.value_dim = int(head_dim), int(value_dim)
        self.scale, self.eps = float(scale), float(eps)
        self.window = int(window) if window else None
        self.temp_coef, self.temp_every = float(temp_coef), int(temp_every)
        self.qk_norm, self.distance_bias, self.sink, self.output_gate = bool(qk_norm), bool(distance_bias), bool(sink), bool(output_gate)
        self.accumulate = bool(accumulate)     # False: forward writes its result instead of adding it
        self.norm_per_head, self.norm_weights = bool(norm_per_head), bool(norm_weights)
        if self.qk_norm and not self.norm_per_head and not self.norm_weights:
            raise UnsupportedModelError("the norm over a whole projection comes with weights; without them it is made per head")
        self.softcap = float(softcap) if softcap else 0.0
        self.chunk = int(chunk) if chunk else None
        self.own_kv = bool(own_kv)             # False: no k / v projection; reads the cache of another layer
        if cache_reach == "own":
            cache_reach = self.window if self.window else self.chunk
            if self.window and self.chunk:
                cache_reach = min(self.window, self.chunk)
        self.cache_reach = int(cache_reach) if cache_reach else None
        self.q_size, self.k_size = self.num_heads * self.head_dim, self.num_kv_heads * self.head_dim
        self.v_size, self.o_size = self.num_kv_heads * self.value_dim, self.num_heads * self.value_dim
        ops.check_general_attention_sizes(self.num_heads, self.num_kv_heads, self.head_dim, self.value_dim)

    def tensor_specs(self) -> List[TensorSpec]:
        D = self.hidden_size
        specs = [TensorSpec("q", (self.q_size, D))]
        if self.own_kv:
            specs += [TensorSpec("k", (self.k_size, D)), TensorSpec("v", (self.v_size, D))]
        if self.qk_norm and self.norm_weights:
            specs.append(TensorSpec("q.norm", (self.q_size,), "norm"))
            if self.own_kv:
                specs.append(TensorSpec("k.norm", (self.k_size,), "norm"))
        if self.sink:
            specs.append(TensorSpec("sink", (self.num_heads,), "bias"))
        if self.output_gate:
            specs.append(TensorSpec("g", (self.num_heads, D)))
        specs.append(TensorSpec("o", (D, self.o_size)))
        return specs

    def cache_spec(self):
        return PagedCacheSpec((PagedTensor("k", (self.num_kv_heads, PAGE, self.head_dim)),
                               PagedTensor("v", (self.num_kv_heads, self.value_dim, PAGE))), self.cache_reach)

    def step_planner(self, page_size: int):
        if self.value_dim != self.head_dim or self.head_dim % 16:     # only the general kernel takes such heads; it needs no work lists
            return None
        return ops.attention_planner(self.dtype, self.num_heads, self.num_kv_heads, self.head_dim, page_size, self.window or 0,
                                     self.device, self.chunk or 0)

    def load(self, tensors: Dict[str, torch.Tensor], dtype, device) -> None:
        super().load(tensors, dtype, device)
        mats = [tensors["q"]] + ([tensors["k"], tensors["v"]] if self.own_kv else []) + ([tensors["g"]] if self.output_gate else [])
        # one projection, rows [q heads | k heads | v heads | gates]
        common = torch.float32 if any(m.dtype == torch.float32 for m in mats) else mats[0].dtype
        self.w_in = torch.cat([m.to(common) for m in mats], dim=0).contiguous()
        self.w_o = tensors["o"]
        f32 = lambda t: t.to(torch.float32).contiguous()
        weighted = self.qk_norm and self.norm_weights
        self.w_qn = f32(tensors["q.norm"]) if weighted else None
        self.w_kn = f32(tensors["k.norm"]) if weighted and self.own_kv else None
        self.sinks = f32(tensors["sink"]) if self.sink else None
        self.slopes = distance_slopes(self.num_heads).to(device) if self.distance_bias else None

    def streamed_weights(self) -> List[torch.Tensor]:
        return [self.w_in, self.w_o]

    def forward(self, h: torch.Tensor, x: torch.Tensor, ctx: StepContext, cache: LayerCache) -> None:
        T, ws = h.shape[0], ctx.workspace
        table = ctx.block_tables[cache.group]
        # a float32 tensor, or - where the product was split over k - its pieces, which the next kernel adds
        proj = ops.qkv_projection(h, self.w_in, torch.float32, ws)
        q = torch.empty((T, self.q_size), dtype=self.dtype, device=h.device)
        gate = torch.empty((T, self.num_heads), dtype=torch.float32, device=h.device) if self.output_gate else None
        writes = self.own_kv and cache.writes
        ops.qk_norm_kv_write(q, gate, proj, self.w_qn, self.w_kn, ctx, self.eps, self.temp_coef, self.temp_every,
                             self.num_heads, self.num_kv_heads, self.head_dim, self.value_dim,
                             self.num_heads if self.output_gate else 0, cache.k if writes else None,
                             cache.v if writes else None, table, cache.page_size,
                             per_head=self.qk_norm and self.norm_per_head, has_kv=self.own_kv)
        attn = torch.empty((T, self.o_size), dtype=self.dtype, device=h.device)
        ops.paged_attention(attn, q, cache.k, cache.v, table, ctx, self.num_heads, self.num_kv_heads, self.head_dim,
                            cache.page_size, self.scale, self.window or 0, ws, value_dim=self.value_dim,
                            slopes=self.slopes, sinks=self.sinks, gate=gate, softcap=self.softcap, chunk=self.chunk or 0)
        ops.gemm(x, attn, self.w_o, accumulate=self.accumulate,
                 may_defer=self.accumulate and getattr(ctx, "may_defer", False), ws=ws)


MIXERS.register("sink_window_attention", SinkWindowAttention)
