"""Causal grouped-query attention over the paged cache.

Formulas (include/photon/ops/kernels/mha_kernel.hpp:174-230): for a query at absolute
position p, head n, kv head ``g = n // (heads / kv_heads)``:
``s_t = scale * <q_n, K_g[t]>`` for t = 0..p (causality is the loop bound),
``P = softmax(s)``, ``o_n = sum_t P_t V_g[t]``; heads are concatenated and projected by
``o_proj``.  Projections have no bias and weights are ``[out, in]`` with ``y = x W^T``
(src/arch/transformer_block.cpp:204-211,262-270).  Keys are stored after the position
encoding, values as they are (src/ops/kernels/cuda/paged_kv_write.cu:27-77).

Unlike the reference's batched path (src/arch/transformer_block.cpp:443-509), every
token carries its own position and sees only keys at positions <= its own, so a
prompt may be cut into portions anywhere.

An optional ``window`` W restricts a query at p to keys p-W+1..p.

Further options, each a constructor parameter: values of another width than keys
(``value_dim``), a cap on the scores (``softcap`` c: the scaled score s becomes
``c * tanh(s / c)`` before the softmax), a factor on the mixer's result (``out_scale``, for
arrangements that weigh mixers side by side; applied to the attention's float32 output before
its one rounding, so that the output projection needs no second pass), other tensor names, biases on the
q, k and v projections (``qkv_bias``) and on the output projection (``o_bias``; tensor names with ``bias_suffix``
added; added in float32, the first three before the rotation), and ``accumulate`` False: the result is written into the
tensor handed to ``forward`` instead of added to it.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

from .. import ops
from ..errors import UnsupportedModelError
from ..weights.loader import TensorSpec
from .base import MIXERS, PAGE, KVCacheSpec, LayerCache, Mixer, PagedCacheSpec, PagedTensor, PositionEncoding, StepContext


POSITION_PREFIX = "position."


class PagedAttention(Mixer):
    def __init__(
        self,
        hidden_size: int,
        num_heads: int,
        num_kv_heads: int,
        head_dim: int,
        position: Optional[PositionEncoding] = None,
        scale: Optional[float] = None,
        window: Optional[int] = None,
        own_kv: bool = True,
        value_dim: Optional[int] = None,
        softcap: Optional[float] = None,
        out_scale: float = 1.0,
        names=("q_proj.weight", "k_proj.weight", "v_proj.weight", "o_proj.weight"),
        any_head_size: bool = False,
        qkv_bias: bool = False,
        o_bias: bool = False,
        bias_suffix: str = ".b",
        accumulate: bool = True,
        bias_to_caller: bool = False,
    ):
        self.hidden_size = int(hidden_size)
        self.num_heads = int(num_heads)
        self.num_kv_heads = int(num_kv_heads)
        self.head_dim = int(head_dim)
        self.position = position
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(self.head_dim)
        self.window = int(window) if window else None
        self.own_kv = bool(own_kv)  # False: the layer has no k/v projection and reads another's cache
        self.value_dim = int(value_dim) if value_dim else self.head_dim
        self.softcap = float(softcap) if softcap else 0.0
        self.out_scale = float(out_scale)
        self.names = tuple(names)          # the q, k, v and o matrices' names after the part's prefix
        self.qkv_bias, self.o_bias, self.bias_suffix, self.accumulate = bool(qkv_bias), bool(o_bias), bias_suffix, bool(accumulate)
        # True: the output projection's bias is not added here; whoever called reads it from ``pending_bias``
        # and adds it in a pass of its own (an arrangement that normalises the result anyway)
        self.bias_to_caller = bool(bias_to_caller) and self.o_bias
        self.pending_bias: Optional[torch.Tensor] = None
        self.q_size = self.num_heads * self.head_dim
        self.kv_size = self.num_kv_heads * self.head_dim
        self.v_size = self.num_kv_heads * self.value_dim
        self.o_size = self.num_heads * self.value_dim
        # what only the general kernels and the separate rotation serve
        self.with_options = self.value_dim != self.head_dim or self.softcap > 0.0 or self.out_scale != 1.0
        if any_head_size and self.head_dim % 16:     # a head size that only the general kernels take
            self.with_options = True
        if self.with_options:
            ops.check_general_attention_sizes(self.num_heads, self.num_kv_heads, self.head_dim, self.value_dim)
        else:
            ops.check_attention_sizes(self.num_heads, self.num_kv_heads, self.head_dim)

    def tensor_specs(self) -> List[TensorSpec]:
        specs = [TensorSpec(self.names[0], (self.q_size, self.hidden_size))]
        if self.own_kv:
            specs += [
                TensorSpec(self.names[1], (self.kv_size, self.hidden_size)),
                TensorSpec(self.names[2], (self.v_size, self.hidden_size)),
            ]
        specs.append(TensorSpec(self.names[3], (self.hidden_size, self.o_size)))
        if self.qkv_bias:
            sizes = [self.q_size] + ([self.kv_size, self.v_size] if self.own_kv else [])
            specs += [TensorSpec(n + self.bias_suffix, (size,), "small_bias") for n, size in zip(self.names, sizes)]
        if self.o_bias:
            specs.append(TensorSpec(self.names[3] + self.bias_suffix, (self.hidden_size,), "small_bias"))
        if self.position is not None:     # a position encoding with tensors of its own keeps them under "position."
            specs += [s.with_prefix(POSITION_PREFIX) for s in self.position.tensor_specs()]
        return specs

    def cache_spec(self):
        if self.value_dim != self.head_dim:
            return PagedCacheSpec((PagedTensor("k", (self.num_kv_heads, PAGE, self.head_dim)),
                                   PagedTensor("v", (self.num_kv_heads, self.value_dim, PAGE))), self.window)
        return KVCacheSpec(self.num_kv_heads, self.head_dim, self.window)

    @property
    def graph_safe(self) -> bool:
        # the kernels take the step's shape from device memory; a position encoding applied by
        # library calls must make the promise itself
        return self.position is None or bool(self.position.graph_safe)

    def step_planner(self, page_size: int):
        if self.value_dim != self.head_dim:      # only the general kernel takes such heads; it needs no work lists
            return None
        return ops.attention_planner(self.dtype, self.num_heads, self.num_kv_heads, self.head_dim, page_size,
                                     self.window or 0, self.device)

    def load(self, tensors: Dict[str, torch.Tensor], dtype, device) -> None:
        super().load(tensors, dtype, device)
        mats = [tensors[self.names[0]]]
        if self.own_kv:
            mats += [tensors[self.names[1]], tensors[self.names[2]]]
        # one projection for q, k and v: rows [q heads | k heads | v heads]
        common = torch.float32 if any(m.dtype == torch.float32 for m in mats) else mats[0].dtype
        self.w_qkv = torch.cat([m.to(common) for m in mats], dim=0).contiguous()
        self.w_o = tensors[self.names[3]]
        self.b_qkv = self.b_o = None
        if self.qkv_bias:
            self.b_qkv = torch.cat([tensors[n + self.bias_suffix].to(torch.float32) for n in self.names[:len(mats)]]).contiguous()
        if self.o_bias:
            self.b_o = tensors[self.names[3] + self.bias_suffix].to(torch.float32).contiguous()
            self.pending_bias = self.b_o if self.bias_to_caller else None
        if self.position is not None:
            own = {n[len(POSITION_PREFIX):]: t for n, t in tensors.items() if n.startswith(POSITION_PREFIX)}
            self.position.load(own, dtype, device)

    def streamed_weights(self) -> List[torch.Tensor]:
        return [self.w_qkv, self.w_o]

    def forward(self, h: torch.Tensor, x: torch.Tensor, ctx: StepContext, cache: LayerCache) -> None:
        T = h.shape[0]
        writes = self.own_kv and cache.writes
        rotary = self.position.rotary_params(ctx) if self.position is not None else None
        fused_position = self.position is None or rotary is not None
        table = ctx.block_tables[cache.group]
        ws = ctx.workspace
        if self.qkv_bias:
            if not fused_position:
                raise UnsupportedModelError("biased projections go with a rotation (or none), not with another position encoding")
            # float32 results (a tensor, or the pieces of a product split over k) so that the biased projection is
            # rounded once, after the rotation
            qkv = ops.qkv_projection(h, self.w_qkv, torch.float32, ws)
            if isinstance(qkv, torch.Tensor):
                qkv = ops.Partials(qkv.view(1, T, qkv.shape[1]), 1, T, qkv.shape[1])
        else:
            qkv = ops.qkv_projection(h, self.w_qkv, self.dtype, ws) if fused_position else None
        if qkv is not None and ctx.all_decode and not self.with_options and not self.qkv_bias:
            # single tokens only: one kernel rotates, writes the cache and attends
            attn = torch.empty((T, self.q_size), dtype=self.dtype, device=h.device)
            done = ops.decode_attention_from_projection(attn, qkv, ctx, rotary, self.num_heads, self.num_kv_heads,
                                                        self.head_dim, cache.k, cache.v, table, cache.page_size, self.scale,
                                                        self.window or 0, writes, ws,
                                                        leave_ranges=self.w_o.numel() * self.w_o.element_size())
            if done:
                # the output, or its key ranges still to be merged, which the product does as it reads them
                ops.gemm(x, done if isinstance(done, ops.KeyRanges) else attn, self.w_o, accumulate=self.accumulate,
                         may_defer=self.accumulate and not self.o_bias and getattr(ctx, "may_defer", False), ws=ws)
                if self.o_bias and not self.bias_to_caller:
                    ops.add_row_bias(x, self.b_o)
                return
        if qkv is not None and not isinstance(qkv, torch.Tensor):
            # the projection is still in pieces (split over k): the rotation kernel sums them
            q = torch.empty((T, self.q_size), dtype=self.dtype, device=h.device)
            ops.rope_kv_write(q, None, None, ctx.positions, ctx.req_of_token, rotary, self.num_heads,
                              self.num_kv_heads, self.head_dim, cache.k, cache.v, table, cache.page_size,
                              pieces=qkv, write_kv=writes, value_dim=self.value_dim, bias=self.b_qkv)
        else:
            if qkv is None:
                qkv = torch.empty((T, self.w_qkv.shape[0]), dtype=self.dtype, device=h.device)
                ops.gemm(qkv, h, self.w_qkv, ws=ws)
            q = qkv[:, : self.q_size]
            k = qkv[:, self.q_size : self.q_size + self.kv_size] if self.own_kv else None
            v = qkv[:, self.q_size + self.kv_size :] if self.own_kv else None
            if not fused_position:
                self.position.apply(q, k, ctx)
            ops.rope_kv_write(
                q, k if writes else None, v if writes else None, ctx.positions, ctx.req_of_token,
                rotary, self.num_heads, self.num_kv_heads, self.head_dim, cache.k, cache.v, table, cache.page_size,
                value_dim=self.value_dim,
            )
        attn = torch.empty((T, self.o_size), dtype=self.dtype, device=h.device)
        if self.with_options:
            ops.paged_attention(attn, q, cache.k, cache.v, table, ctx, self.num_heads, self.num_kv_heads, self.head_dim,
                                cache.page_size, self.scale, self.window or 0, ws, value_dim=self.value_dim,
                                softcap=self.softcap, out_scale=self.out_scale)
        else:
            ops.paged_attention(
                attn, q, cache.k, cache.v, table, ctx,
                self.num_heads, self.num_kv_heads, self.head_dim, cache.page_size,
                self.scale, self.window or 0, ws,
            )
        # where the arrangement allows it, the product stays in pieces for the stream's next reader
        ops.gemm(x, attn, self.w_o, accumulate=self.accumulate,
                 may_defer=self.accumulate and not self.o_bias and getattr(ctx, "may_defer", False), ws=ws)
        if self.o_bias and not self.bias_to_caller:
            ops.add_row_bias(x, self.b_o)


MIXERS.register("attention", PagedAttention)
