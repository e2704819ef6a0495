"""Arrangements of norm, mixer and feed-forward around the residual stream.

Pre-norm order of the reference (include/photon/arch/transformer_block.hpp:34-51,
src/arch/transformer_block.cpp:189-299):
``x += mixer(norm1(x)); x += ffn(norm2(x))``.
"""
from __future__ import annotations

from typing import Dict, List, Optional, Tuple

import torch

from .. import ops
from ..errors import UnsupportedModelError
from ..weights.loader import TensorSpec
from .base import BLOCKS, MIXERS, Block, FeedForward, LayerCache, Mixer, Norm, Part, StepContext


class SideBySide(Mixer):
    """Several mixers that read the same input, their results summed into the stream:
    ``x += sum_i scale_i * mixer_i(h)``.  Every mixer keeps a cache or state of its own
    (``mixers()``; ``forward`` takes their ``LayerCache`` in that order) and applies its own
    factor (its ``out_scale``) to its last activation, in float32, before the output projection
    that accumulates into the stream: the sum costs no kernel.

    ``branches``: [(prefix, mixer)]."""

    def __init__(self, branches):
        if not branches:
            raise UnsupportedModelError("mixers side by side: none given")
        self.branches: List[Tuple[str, Mixer]] = list(branches)
        for _, m in self.branches:
            if not getattr(m, "accumulate", True):
                raise UnsupportedModelError(f"{type(m).__name__} must add its result into the stream to stand beside other mixers")

    def mixers(self) -> List[Mixer]:
        return [m for _, m in self.branches]

    def tensor_specs(self) -> List[TensorSpec]:
        return [s.with_prefix(p) for p, m in self.branches for s in m.tensor_specs()]

    def load(self, tensors: Dict[str, torch.Tensor], dtype, device) -> None:
        super().load(tensors, dtype, device)
        for prefix, m in self.branches:
            names = [prefix + s.name for s in m.tensor_specs()]
            m.load({n[len(prefix):]: tensors[n] for n in names}, dtype, device)

    @property
    def graph_safe(self) -> bool:
        return all(m.graph_safe for _, m in self.branches)

    def streamed_weights(self) -> List[torch.Tensor]:
        return [w for _, m in self.branches for w in m.streamed_weights()]

    def forward(self, h: torch.Tensor, x: torch.Tensor, ctx: StepContext, cache) -> None:
        caches = cache if isinstance(cache, (list, tuple)) else [cache]
        for (_, m), c in zip(self.branches, caches):
            m.forward(h, x, ctx, c)


MIXERS.register("side_by_side", SideBySide)


class PreNormBlock(Block):
    """Each of the four parts comes with the name prefix of its tensors inside the block.  The
    mixer may be several side by side (``SideBySide``); ``norm2`` and ``ffn`` None: a layer without
    a feed-forward."""

    def __init__(self, norm1: Tuple[str, Norm], mixer: Tuple[str, Mixer],
                 norm2: Optional[Tuple[str, Norm]] = None, ffn: Optional[Tuple[str, FeedForward]] = None):
        if (ffn is None) != (norm2 is None):
            raise UnsupportedModelError("a feed-forward and its norm come together")
        self._named: List[Tuple[str, Part]] = [norm1, mixer] + ([norm2, ffn] if ffn is not None else [])
        self.norm1, self.mixer = norm1[1], mixer[1]
        self.norm2, self.ffn = (norm2[1], ffn[1]) if ffn is not None else (None, None)

    def mixers(self) -> List[Mixer]:
        inner = getattr(self.mixer, "mixers", None)
        return inner() if inner is not None else [self.mixer]

    def tensor_specs(self) -> List[TensorSpec]:
        return [s.with_prefix(p) for p, part in self._named for s in part.tensor_specs()]

    def load(self, tensors: Dict[str, torch.Tensor], dtype, device) -> None:
        super().load(tensors, dtype, device)
        # a part's tensors: those named by its own list (a prefix may be a prefix of another)
        for prefix, part in self._named:
            names = [prefix + s.name for s in part.tensor_specs()]
            part.load({n[len(prefix):]: tensors[n] for n in names}, dtype, device)

    @property
    def graph_safe(self) -> bool:
        return all(part.graph_safe for _, part in self._named)

    def streamed_weights(self) -> List[torch.Tensor]:
        return [w for _, part in self._named for w in part.streamed_weights()]

    @property
    def reads_deferred(self) -> bool:
        return bool(getattr(self.norm1, "consumes_deferred", False))

    def forward(self, x: torch.Tensor, ctx: StepContext, cache: LayerCache) -> None:
        # A mixer or feed-forward may leave its update of x in pieces (ops.gemm(..., may_defer=True))
        # when the stream's next reader adds them: norm2 after the mixer; after the feed-forward,
        # whoever the model says reads the stream next.
        if self.ffn is None:
            ctx.may_defer = ctx.after_block_consumes
            self.mixer.forward(self.norm1.forward(x, ctx), x, ctx, cache)
            ctx.may_defer = False
            return
        ctx.may_defer = bool(getattr(self.norm2, "consumes_deferred", False))
        self.mixer.forward(self.norm1.forward(x, ctx), x, ctx, cache)
        ctx.may_defer = ctx.after_block_consumes
        self.ffn.forward(self.norm2.forward(x, ctx), x, ctx)
        ctx.may_defer = False


BLOCKS.register("prenorm", PreNormBlock)


class OutputNormBlock(Block):
    """Sublayers that read the stream itself and are normalised on the way out:

        x <- x + mult * norm1(mix(x));   x <- x + mult * norm2(ffn(x))   (no feed-forward: the first only)

    ``mix`` is one mixer, or two side by side that read the same input: then each result is first
    normalised with a weight of its own and the two are averaged.  The norms, the mean, the scaled
    add and the copy of the new stream in the activation type are one kernel per sublayer.  The
    mixers and the feed-forward write their result (``accumulate=False``) instead of adding it.

    ``branches``: [(prefix, mixer, (prefix, norm) or None)]; ``norm1`` / ``norm2`` / ``ffn``: (prefix, part).
    """

    reads_deferred = False
    _STREAM = "stream in the activation type"     # key in ctx.scratch: (stream, its copy) left for the next reader

    def __init__(self, branches, norm1: Tuple[str, Norm], mult: float, norm2=None, ffn=None):
        if not 1 <= len(branches) <= 2:
            raise UnsupportedModelError(f"an output-norm block holds one mixer or two side by side, not {len(branches)}")
        if len(branches) == 2 and any(b[2] is None for b in branches):
            raise UnsupportedModelError("two mixers side by side each need the norm of their result")
        if (ffn is None) != (norm2 is None):
            raise UnsupportedModelError("a feed-forward and its norm come together")
        self.branches = list(branches)
        self.norm1, self.norm2, self.ffn = norm1[1], norm2[1] if norm2 else None, ffn[1] if ffn else None
        self.mult = float(mult)
        self._named: List[Tuple[str, Part]] = [(p, m) for p, m, _ in branches] + [n for _, _, n in branches if n is not None] + [norm1]
        if ffn is not None:
            self._named += [norm2, ffn]
        for _, part in self._named:
            if getattr(part, "accumulate", False):
                raise UnsupportedModelError(f"{type(part).__name__} must be built with accumulate=False inside an output-norm block")

    def mixers(self) -> List[Mixer]:
        return [m for _, m, _ in self.branches]

    def tensor_specs(self) -> List[TensorSpec]:
        return [s.with_prefix(p) for p, part in self._named for s in part.tensor_specs()]

    def load(self, tensors: Dict[str, torch.Tensor], dtype, device) -> None:
        super().load(tensors, dtype, device)
        # a part's tensors: those named by its own list (prefixes here may be prefixes of one another)
        for prefix, part in self._named:
            names = [prefix + s.name for s in part.tensor_specs()]
            part.load({n[len(prefix):]: tensors[n] for n in names}, dtype, device)

    @property
    def graph_safe(self) -> bool:
        return all(part.graph_safe for _, part in self._named)

    def streamed_weights(self) -> List[torch.Tensor]:
        return [w for _, part in self._named for w in part.streamed_weights()]

    def forward(self, x: torch.Tensor, ctx: StepContext, cache) -> None:
        left = ctx.scratch.pop(self._STREAM, None)
        h = left[1] if left is not None and left[0] is x else ops.cast_stream(x, self.dtype)
        caches = cache if isinstance(cache, (list, tuple)) else [cache]
        ctx.may_defer = False
        outs = []
        for (_, mixer, _), c in zip(self.branches, caches):
            out = torch.empty_like(x)
            mixer.forward(h, out, ctx, c)
            outs.append(out)
        norms = [n[1] if n is not None else None for _, _, n in self.branches]
        eps = self.norm1.eps
        if len(outs) == 2:
            h = ops.branch_norm_add(x, outs[0], self.norm1.weight_f32(), eps, self.mult, norms[0].weight_f32(), outs[1],
                                    norms[1].weight_f32(), h_dtype=self.dtype)
        else:
            h = ops.branch_norm_add(x, outs[0], self.norm1.weight_f32(), eps, self.mult,
                                    norms[0].weight_f32() if norms[0] is not None else None, h_dtype=self.dtype)
        if self.ffn is not None:
            out = torch.empty_like(x)
            self.ffn.forward(h, out, ctx)
            h = ops.branch_norm_add(x, out, self.norm2.weight_f32(), self.norm2.eps, self.mult, h_dtype=self.dtype)
        ctx.scratch[self._STREAM] = (x, h)


BLOCKS.register("output_norm", OutputNormBlock)


class SandwichBlock(Block):
    """A norm in front of every sublayer and another behind it:

        x <- x + post1(mix(pre1(x)));   x <- x + post2(ffn(pre2(x)))     (no feed-forward: the first only)

    ``mix`` is one mixer, or two side by side that read the same input: then each result is first RMS-normalised
    over the width with a weight of its own and the two are averaged.  The four norms are layer norms with weight and
    bias (``LayerNorm``).  The branch norms, the mean, the norm behind the sublayer, the add and the norm in front of the
    next sublayer of the block are one kernel.  The mixers and the feed-forward write their result
    (``accumulate=False``) instead of adding it.

    ``branches``: [(prefix, mixer, (prefix, rmsnorm) or None)]; ``pre1`` / ``post1`` / ``pre2`` / ``post2`` / ``ffn``: (prefix, part).
    """

    reads_deferred = False

    def __init__(self, branches, pre1: Tuple[str, Norm], post1: Tuple[str, Norm], pre2=None, post2=None, ffn=None):
        if not 1 <= len(branches) <= 2:
            raise UnsupportedModelError(f"a sandwich block holds one mixer or two side by side, not {len(branches)}")
        if len(branches) == 2 and any(b[2] is None for b in branches):
            raise UnsupportedModelError("two mixers side by side each need the norm of their result")
        if not ((ffn is None) == (pre2 is None) == (post2 is None)):
            raise UnsupportedModelError("a feed-forward and its two norms come together")
        self.branches = list(branches)
        self.pre1, self.post1 = pre1[1], post1[1]
        self.pre2, self.post2, self.ffn = (pre2[1], post2[1], ffn[1]) if ffn is not None else (None, None, None)
        self._named: List[Tuple[str, Part]] = [pre1, post1] + [(p, m) for p, m, _ in branches] + [n for _, _, n in branches if n is not None]
        if ffn is not None:
            self._named += [pre2, post2, ffn]
        for _, part in [(p, m) for p, m, _ in branches] + ([ffn] if ffn is not None else []):
            if getattr(part, "accumulate", True):
                raise UnsupportedModelError(f"{type(part).__name__} must be built with accumulate=False inside a sandwich block")
        for n in (self.pre1, self.post1, self.pre2, self.post2):
            if n is not None and not hasattr(n, "weight_bias_f32"):
                raise UnsupportedModelError(f"a sandwich block's norms are layer norms with weight and bias, not {type(n).__name__}")

    def mixers(self) -> List[Mixer]:
        return [m for _, m, _ in self.branches]

    def tensor_specs(self) -> List[TensorSpec]:
        return [s.with_prefix(p) for p, part in self._named for s in part.tensor_specs()]

    def load(self, tensors: Dict[str, torch.Tensor], dtype, device) -> None:
        super().load(tensors, dtype, device)
        # a part's tensors: those named by its own list (prefixes here may be prefixes of one another)
        for prefix, part in self._named:
            names = [prefix + s.name for s in part.tensor_specs()]
            part.load({n[len(prefix):]: tensors[n] for n in names}, dtype, device)

    @property
    def graph_safe(self) -> bool:
        return all(part.graph_safe for _, part in self._named)

    def streamed_weights(self) -> List[torch.Tensor]:
        return [w for _, part in self._named for w in part.streamed_weights()]

    def forward(self, x: torch.Tensor, ctx: StepContext, cache) -> None:
        caches = cache if isinstance(cache, (list, tuple)) else [cache]
        ctx.may_defer = False
        h = self.pre1.forward(x, ctx)
        outs = []
        for (_, mixer, _), c in zip(self.branches, caches):
            out = torch.empty_like(x)
            mixer.forward(h, out, ctx, c)
            outs.append(out)
        norms = [n[1] if n is not None else None for _, _, n in self.branches]
        nxt = self.pre2.weight_bias_f32() if self.ffn is not None else None
        # a mixer may leave the bias of its last product to this kernel (``pending_bias``)
        a_bias = getattr(self.branches[0][1], "pending_bias", None)
        w_a = norms[0].weight_f32() if norms[0] is not None else None
        if len(outs) == 2:
            h = ops.sandwich_norm_add(x, outs[0], self.post1.weight_bias_f32(), self.post1.eps, nxt, self.dtype, w_a=w_a, b=outs[1],
                                      w_b=norms[1].weight_f32(), a_bias=a_bias)
        else:
            h = ops.sandwich_norm_add(x, outs[0], self.post1.weight_bias_f32(), self.post1.eps, nxt, self.dtype, w_a=w_a, a_bias=a_bias)
        if self.ffn is not None:
            out = torch.empty_like(x)
            self.ffn.forward(h, out, ctx)
            ops.sandwich_norm_add(x, out, self.post2.weight_bias_f32(), self.post2.eps)


BLOCKS.register("sandwich", SandwichBlock)
