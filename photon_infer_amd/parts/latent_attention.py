"""Causal attention whose keys and values come through a low-rank latent, with one rotated key
part that all heads share.

For a token at position p with input h (sizes and constants are constructor parameters):

* queries through a latent of ``q_rank``: ``c_q = norm(W_dq h; dq.norm)``, ``q = W_uq c_q``, laid out head
  by head as [``head_dim`` plain | ``rot_dim`` rotated];
* ``W_dkv h`` has ``kv_rank + rot_dim`` rows: the first ``kv_rank``, normalised with ``dkv.norm``, are the
  latent ``c``; the last ``rot_dim`` (not normalised) are the rotated key part ``k_r`` of every head;
* head n's key is ``[W_uk_n c | k_r]`` and its value ``W_uv_n c``;
  ``score(p, t) = scale * (<q_plain, W_uk_n c_t> + <rotate(q_rot, p), rotate(k_r, t)>)`` for ``t <= p``;
* ordinary softmax; ``W_o`` on the concatenated heads.

Only ``c`` and the rotated ``k_r`` are kept per token.  Keys and values are never made: the
plain part of the score is ``<W_uk_n^T q_plain, c_t>``, so a head's query becomes
``q_lat = [W_uk_n^T q_plain | rotate(q_rot)]`` (``kv_rank + rot_dim`` numbers), every head attends over
the same cached rows ``[c | k_r]`` - one key/value head for all query heads - with ``c`` as the value,
and ``W_uv_n`` is applied to the result, head by head.  Norms, angles, rotations, scores and the
softmax are float32 in both compute modes.

The rotation is a ``PositionEncoding`` over ``rot_dim`` (any pairing rule and frequency scaling the
rotary part offers; its cos / sin table is made once per step).
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from .. import ops
from ..errors import UnsupportedModelError
from ..weights.loader import TensorSpec
from .base import MIXERS, PAGE, LayerCache, Mixer, PagedCacheSpec, PagedTensor, PositionEncoding, StepContext


class LatentAttention(Mixer):
    graph_safe = True        # every kernel takes positions, requests and pages from device memory

    def __init__(self, hidden_size: int, num_heads: int, head_dim: int, rot_dim: int, value_dim: int, q_rank: int, kv_rank: int,
                 scale: float, eps: float, position: Optional[PositionEncoding] = None, accumulate: bool = True,
                 names=("dq", "dq.norm", "uq", "dkv", "dkv.norm", "uk", "uv", "o")):
        self.hidden_size, self.num_heads = int(hidden_size), int(num_heads)
        self.head_dim, self.rot_dim, self.value_dim = int(head_dim), int(rot_dim), int(value_dim)
        self.q_rank, self.kv_rank = int(q_rank), int(kv_rank)
        self.scale, self.eps = float(scale), float(eps)
        self.position = position
        self.accumulate = bool(accumulate)
        self.names = tuple(names)
        if self.rot_dim % 2:
            raise UnsupportedModelError(f"latent attention: the rotated width {self.rot_dim} must be even")
        if self.rot_dim and position is None:
            raise UnsupportedModelError("latent attention: a rotated part needs its position encoding")
        if position is not None:
            params = position.rotary_params if hasattr(position, "rotary_params") else None
            if params is None or getattr(position, "rotary_dim", self.rot_dim) != self.rot_dim or not getattr(position, "interleaved", True):
                raise UnsupportedModelError("latent attention: the rotation must turn neighbouring pairs over the whole rotated part")
        self.latent_dim = self.kv_rank + self.rot_dim          # what a cached key row holds
        self.q_size = self.num_heads * (self.head_dim + self.rot_dim)
        self.o_size = self.num_heads * self.value_dim
        ops.check_general_attention_sizes(self.num_heads, 1, self.latent_dim, self.kv_rank)

    def tensor_specs(self) -> List[TensorSpec]:
        D, n = self.hidden_size, self.names
        return [TensorSpec(n[0], (self.q_rank, D)), TensorSpec(n[1], (self.q_rank,), "norm"),
                TensorSpec(n[2], (self.q_size, self.q_rank)),
                TensorSpec(n[3], (self.kv_rank + self.rot_dim, D)), TensorSpec(n[4], (self.kv_rank,), "norm"),
                TensorSpec(n[5], (self.num_heads * self.head_dim, self.kv_rank)),
                TensorSpec(n[6], (self.num_heads * self.value_dim, self.kv_rank)),
                TensorSpec(n[7], (D, self.o_size))]

    def value_rows(self, dtype) -> int:
        """Rows of a cached value page.  The latent alone is the value; where the matrix-core attention kernels can
        serve the heads (bfloat16, a latent row that is a multiple of 16 up to their largest head) the rotated part rides along, because those
        kernels want values as wide as keys; what it adds to a head's result is never read."""
        wide = dtype == torch.bfloat16 and self.latent_dim % 16 == 0 and self.latent_dim <= ops.MAX_HEAD_DIM and ops.fast_kernels_enabled()
        return self.latent_dim if wide else self.kv_rank

    def cache_spec(self):
        # one key/value head: the latent and the shared rotated part.  The compute dtype, known once the part is
        # loaded (the pools are made after that), decides the value rows.
        rows = self.value_rows(getattr(self, "dtype", None))
        return PagedCacheSpec((PagedTensor("k", (1, PAGE, self.latent_dim)), PagedTensor("v", (1, rows, PAGE))), None)

    def step_planner(self, page_size: int):
        if self.value_rows(self.dtype) != self.latent_dim:
            return None
        return ops.attention_planner(self.dtype, self.num_heads, 1, self.latent_dim, page_size, 0, self.device)

    def load(self, tensors: Dict[str, torch.Tensor], dtype, device) -> None:
        super().load(tensors, dtype, device)
        n = self.names
        mats = [tensors[n[0]], tensors[n[3]]]
        common = torch.float32 if any(m.dtype == torch.float32 for m in mats) else mats[0].dtype
        # one projection into [query latent | key/value latent | shared rotated part]
        self.w_in = torch.cat([m.to(common) for m in mats], dim=0).contiguous()
        self.w_uq = tensors[n[2]]
        f32 = lambda t: t.to(torch.float32).contiguous()
        self.w_qn, self.w_kvn = f32(tensors[n[1]]), f32(tensors[n[4]])
        H, d, dv, r = self.num_heads, self.head_dim, self.value_dim, self.kv_rank
        # per head, inputs as rows: W_uk_n as stored ([head_dim, kv_rank]: the query's plain part goes in, latent
        # coordinates come out) and W_uv_n transposed ([kv_rank, value_dim]: the attended latent goes in)
        self.w_uk = tensors[n[5]].to(dtype).reshape(H, d, r).contiguous()
        self.w_uv = tensors[n[6]].to(dtype).reshape(H, dv, r).transpose(1, 2).contiguous()
        # and with outputs as rows, which the matrix-core kernel reads for steps of many tokens
        fast = dtype == torch.bfloat16 and ops.fast_kernels_enabled()
        self.w_uk_rows = self.w_uk.transpose(1, 2).contiguous() if fast else None
        self.w_uv_rows = tensors[n[6]].to(dtype).reshape(H, dv, r).contiguous() if fast else None
        self.w_o = tensors[n[7]]
        if self.position is not None:
            self.position.load({}, dtype, device)

    def streamed_weights(self) -> List[torch.Tensor]:
        return [self.w_in, self.w_uq, self.w_o]

    def forward(self, h: torch.Tensor, x: torch.Tensor, ctx: StepContext, cache: LayerCache) -> None:
        T, ws, H = h.shape[0], ctx.workspace, self.num_heads
        table = ctx.block_tables[cache.group]
        rot_table = self.position.rotary_params(ctx)[0] if self.rot_dim else None
        # a float32 tensor, or - where the product was split over k - its pieces, which the next kernel adds
        proj = ops.qkv_projection(h, self.w_in, torch.float32, ws)
        cq = torch.empty((T, self.q_rank), dtype=self.dtype, device=h.device)
        ops.latent_kv_write(cq, proj, self.w_qn, self.w_kvn, rot_table, ctx, self.eps, self.q_rank, self.kv_rank, self.rot_dim,
                            cache.k if cache.writes else None, cache.v if cache.writes else None, table, cache.page_size)
        q = torch.empty((T, self.q_size), dtype=self.dtype, device=h.device)
        ops.gemm(q, cq, self.w_uq, ws=ws)
        # queries in the latent's coordinates, the rotated part behind them
        q_lat = torch.empty((T, H * self.latent_dim), dtype=self.dtype, device=h.device)
        ops.head_gemm(q_lat, q, self.w_uk, H, rot=self.rot_dim, table=rot_table, w_rows=self.w_uk_rows)
        v_rows = cache.v.shape[2]
        att = torch.empty((T, H * v_rows), dtype=self.dtype, device=h.device)
        if v_rows == self.latent_dim:
            ops.paged_attention(att, q_lat, cache.k, cache.v, table, ctx, H, 1, self.latent_dim, cache.page_size, self.scale, 0, ws)
        else:
            ops.paged_attention(att, q_lat, cache.k, cache.v, table, ctx, H, 1, self.latent_dim, cache.page_size, self.scale, 0, ws,
                                value_dim=v_rows)
        out = torch.empty((T, self.o_size), dtype=self.dtype, device=h.device)
        ops.head_gemm(out, att, self.w_uv, H, a_head=v_rows, w_rows=self.w_uv_rows)
        ops.gemm(x, out, self.w_o, accumulate=self.accumulate,
                 may_defer=self.accumulate and getattr(ctx, "may_defer", False), ws=ws)


MIXERS.register("latent_attention", LatentAttention)
