"""Differential attention: every head holds two softmax maps over the same values and keeps their
difference (Ye et al., "Differential Transformer").

With input h, ``heads`` query heads and ``kv_heads`` key / value heads (query head n reads key / value
head ``n // (heads / kv_heads)``), keys of ``head_dim`` and values of ``value_dim``:

* ``q = W_q h + b_q`` (``heads * 2 * head_dim`` rows) and ``k = W_k h + b_k`` (``kv_heads * 2 * head_dim`` rows): a head's
  rows are map 1's, then map 2's; ``v = W_v h + b_v`` (``kv_heads * value_dim`` rows) serves both maps.  Positions enter
  through the causal mask alone.
* per head and map m: ``a_m = softmax(scale * q_m K_m^T) V`` over the keys at positions <= the query's;
* ``lam = exp(<lq1, lk1>) - exp(<lq2, lk2>) + diff`` (one number per layer, from four vectors of ``head_dim``);
* ``o = a_1 - lam * a_2``, divided by the root mean square of its ``value_dim`` entries (eps inside the root, no
  weight), times ``1 - diff``; heads concatenated, then ``W_o``.

The two maps are served by the attention kernels as heads of their own: query heads are regrouped at load into the
order [kv head][map][head within the group], so that map m of kv head g is kv head ``2 g + m`` of an attention with
``2 * heads`` query heads over ``2 * kv_heads`` key heads; the values of a kv head are cached once per map.  A kernel
behind the attention takes the difference and the norm in float32.

The matrix-core attention kernels want values as wide as keys.  Where the values are a small multiple of the keys'
width (twice, in the published models of this kind) and the compute type is bfloat16, a value vector is therefore cut into
``split`` pieces as wide as a key and every piece is attended as a head of its own, with the map's queries and keys
repeated for it: the order becomes [kv head][map][piece][head within the group], the scores are computed once per piece,
and the cache holds a map's keys once per piece.  Any other sizes, and float32, take the general kernel with the values
at their own width (``split`` 1).
"""
from __future__ import annotations

import math
from typing import Dict, List

import torch

from .. import ops
from ..errors import UnsupportedModelError
from ..weights.loader import TensorSpec
from .base import MIXERS, PAGE, KVCacheSpec, LayerCache, Mixer, PagedCacheSpec, PagedTensor, StepContext


class DifferentialAttention(Mixer):
    graph_safe = True        # positions, pages and request boundaries are read on the device

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int, value_dim: int, scale: float, diff: float,
                 eps: float, names=("q", "k", "v", "o"), lambda_names=("lq1", "lk1", "lq2", "lk2"), bias_suffix: str = ".b",
                 accumulate: bool = True):
        self.hidden_size, self.num_heads, self.num_kv_heads = int(hidden_size), int(num_heads), int(num_kv_heads)
        self.head_dim, self.value_dim = int(head_dim), int(value_dim)
        self.scale, self.diff, self.eps = float(scale), float(diff), float(eps)
        self.names, self.lambda_names, self.bias_suffix, self.accumulate = tuple(names), tuple(lambda_names), bias_suffix, bool(accumulate)
        if self.num_heads % self.num_kv_heads:
            raise UnsupportedModelError(f"differential attention: {self.num_heads} heads is not a multiple of {self.num_kv_heads} kv heads")
        # the projections as the model folder has them
        self.q_size, self.k_size = 2 * self.num_heads * self.head_dim, 2 * self.num_kv_heads * self.head_dim
        self.v_size, self.o_size = self.num_kv_heads * self.value_dim, self.num_heads * self.value_dim
        self._set_split(1)
        self.lam = None

    MAX_SPLIT = 4

    def _set_split(self, split: int) -> None:
        """As the attention kernels see it: every map, and every piece of its values, a head."""
        self.split = int(split)
        self.piece = self.value_dim // self.split
        self.map_heads, self.map_kv_heads = 2 * self.num_heads * self.split, 2 * self.num_kv_heads * self.split
        # heads whose values are as wide as their keys and a multiple of 16 may take the matrix-core kernels
        self.plain = self.piece == self.head_dim and self.head_dim % 16 == 0 and self.head_dim <= ops.MAX_HEAD_DIM
        if not self.plain:
            ops.check_general_attention_sizes(self.map_heads, self.map_kv_heads, self.head_dim, self.piece)

    def tensor_specs(self) -> List[TensorSpec]:
        q, k, v, o = self.names
        b, D = self.bias_suffix, self.hidden_size
        return ([TensorSpec(q, (self.q_size, D)), TensorSpec(q + b, (self.q_size,), "small_bias"),
                 TensorSpec(k, (self.k_size, D)), TensorSpec(k + b, (self.k_size,), "small_bias"),
                 TensorSpec(v, (self.v_size, D)), TensorSpec(v + b, (self.v_size,), "small_bias")]
                + [TensorSpec(n, (self.head_dim,), "small_bias") for n in self.lambda_names]
                + [TensorSpec(o, (D, self.o_size))])

    def cache_spec(self):
        """Before ``load`` (no compute type yet): the layout without pieces."""
        if self.plain:
            return KVCacheSpec(self.map_kv_heads, self.head_dim, None)
        return PagedCacheSpec((PagedTensor("k", (self.map_kv_heads, PAGE, self.head_dim)),
                               PagedTensor("v", (self.map_kv_heads, self.piece, PAGE))), None)

    def step_planner(self, page_size: int):
        if not self.plain:
            return None
        return ops.attention_planner(self.dtype, self.map_heads, self.map_kv_heads, self.head_dim, page_size, 0, self.device)

    def load(self, tensors: Dict[str, torch.Tensor], dtype, device) -> None:
        super().load(tensors, dtype, device)
        q, k, v, o = self.names
        H, G, d, dv, b = self.num_heads, self.num_kv_heads, self.head_dim, self.value_dim, self.bias_suffix
        per = H // G
        n = dv // d if d > 0 and dv % d == 0 else 0
        fits = dtype == torch.bfloat16 and ops.fast_kernels_enabled() and d % 16 == 0 and d <= ops.MAX_HEAD_DIM and 1 <= n <= self.MAX_SPLIT
        self._set_split(n if fits and all(tensors[x].dtype == torch.bfloat16 for x in (q, k, v)) else 1)
        n, w = self.split, self.piece

        def rows(t, *shape):
            return t.reshape(*shape, *t.shape[1:])

        def spread(t, at, times):      # a new axis of ``times`` equal copies
            t = t.unsqueeze(at)
            return t.expand(*t.shape[:at], times, *t.shape[at + 1:])

        def regroup(t):      # rows [kv head, head in group, map, d] -> [kv head, map, piece, head in group, d]
            return spread(rows(t, G, per, 2, d).transpose(1, 2), 2, n).reshape(2 * H * n * d, *t.shape[1:])

        def per_piece(t):    # a map's keys once per piece: [kv head, map, d] -> [kv head, map, piece, d]
            return spread(rows(t, G, 2, d), 2, n).reshape(2 * G * n * d, *t.shape[1:])

        def per_map(t):      # a kv head's values once per map: [kv head, piece, w] -> [kv head, map, piece, w]
            return spread(rows(t, G, n, w), 1, 2).reshape(2 * G * dv, *t.shape[1:])

        mats = [regroup(tensors[q]), per_piece(tensors[k]), per_map(tensors[v])]
        common = torch.float32 if any(m.dtype == torch.float32 for m in mats) else mats[0].dtype
        self.w_qkv = torch.cat([m.to(common) for m in mats], dim=0).contiguous()
        f32 = lambda t: t.to(torch.float32)
        self.b_qkv = torch.cat([regroup(f32(tensors[q + b])), per_piece(f32(tensors[k + b])), per_map(f32(tensors[v + b]))]).contiguous()
        self.w_o = tensors[o]
        lq1, lk1, lq2, lk2 = (tensors[n].to(torch.float64).cpu() for n in self.lambda_names)
        self.lam = math.exp(float((lq1 * lk1).sum())) - math.exp(float((lq2 * lk2).sum())) + self.diff

    def streamed_weights(self) -> List[torch.Tensor]:
        return [self.w_qkv, self.w_o]

    def forward(self, h: torch.Tensor, x: torch.Tensor, ctx: StepContext, cache: LayerCache) -> None:
        T, ws = h.shape[0], ctx.workspace
        table = ctx.block_tables[cache.group]
        dv = None if self.plain else self.piece
        # float32 results (a tensor, or the pieces of a product split over k): the bias joins before the one rounding
        proj = ops.qkv_projection(h, self.w_qkv, torch.float32, ws)
        if isinstance(proj, torch.Tensor):
            proj = ops.Partials(proj.view(1, T, proj.shape[1]), 1, T, proj.shape[1])
        q = torch.empty((T, self.map_heads * self.head_dim), dtype=self.dtype, device=h.device)
        ops.rope_kv_write(q, None, None, ctx.positions, ctx.req_of_token, None, self.map_heads, self.map_kv_heads, self.head_dim,
                          cache.k, cache.v, table, cache.page_size, pieces=proj, write_kv=cache.writes, value_dim=dv, bias=self.b_qkv)
        attn = torch.empty((T, 2 * self.o_size), dtype=self.dtype, device=h.device)
        ops.paged_attention(attn, q, cache.k, cache.v, table, ctx, self.map_heads, self.map_kv_heads, self.head_dim, cache.page_size,
                            self.scale, 0, ws, value_dim=dv)
        y = torch.empty((T, self.o_size), dtype=self.dtype, device=h.device)
        ops.diff_combine(y, attn, self.lam, self.eps, 1.0 - self.diff, self.num_heads, self.num_kv_heads, self.value_dim, self.split)
        ops.gemm(x, y, self.w_o, accumulate=self.accumulate, may_defer=self.accumulate and getattr(ctx, "may_defer", False), ws=ws)


MIXERS.register("differential_attention", DifferentialAttention)
