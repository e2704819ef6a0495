"""Routed experts (mixture of experts) feed-forward.

Router logits ``z = Wr h`` in float32; scores ``s = softmax(z)`` over all experts.  Experts form
``groups`` equal groups of neighbours; a group's score is its largest expert score and only
experts of the ``keep`` best groups can be chosen.  Each token uses the ``top`` allowed experts
with the largest scores, weighted by those scores as they are (``renormalize``: divided by
their sum plus ``renorm_eps``).  An expert is a gated feed-forward ``Wdown (silu(Wgate h) * (Wup h))`` without
biases (``activation`` "silu"), or ``Wdown max(Wup h, 0)^2`` (``activation`` "relu2": no gate matrix); the result is
the weighted sum of the chosen experts' outputs (float32).

Further options, each a constructor parameter: ``correction`` (a tensor of one number per router output that is
added to the scores for the choice only; the weights stay the scores), ``identity`` (so many identity experts, which take
the last places among the router's outputs, own no matrices and contribute ``weight * h``), and ``shared``
((prefix, feed-forward): one more feed-forward that every token goes through, added to the routed sum).

The step's (token, choice) entries are sorted by expert on the device and each expert's rows go
through grouped products; nothing is counted on the host.
"""
from __future__ import annotations

from typing import Dict, List

import torch

from .. import ops
from ..errors import UnsupportedModelError
from ..weights.loader import TensorSpec
from .base import FEED_FORWARDS, FeedForward, StepContext
from .mlp import INTERLEAVE


class RoutedExperts(FeedForward):
    def __init__(self, hidden_size: int, expert_size: int, num_experts: int, top: int, groups: int = 1, keep: int = 1,
                 renormalize: bool = False, activation: str = "silu", accumulate: bool = True,
                 expert_prefix: str = "e", names=("gate", "up", "down"), router_name: str = "router", identity: int = 0,
                 correction: str = "", renorm_eps: float = 0.0, shared=None):
        if activation not in ("silu", "relu2"):
            raise UnsupportedModelError(f"expert activation '{activation}' is not supported (silu, relu2)")
        self.gated = activation == "silu"
        self.identity, self.correction_name, self.renorm_eps = int(identity), correction, float(renorm_eps)
        self.shared_prefix, self.shared = shared if shared is not None else ("", None)
        if self.identity < 0:
            raise UnsupportedModelError(f"routed experts: {self.identity} identity experts")
        self.hidden_size, self.expert_size = int(hidden_size), int(expert_size)
        self.num_experts, self.top, self.groups, self.keep = int(num_experts), int(top), int(groups), int(keep)
        self.router_size = self.num_experts + self.identity       # router outputs: real experts, then identity experts
        if not 0 < self.top <= self.router_size:
            raise UnsupportedModelError(f"routed experts: {self.top} choices among {self.router_size} experts")
        if self.groups > 1 and self.identity:
            raise UnsupportedModelError("routed experts: groups of experts and identity experts do not go together")
        if self.groups > 1 and (self.num_experts % self.groups or not 0 < self.keep <= self.groups
                                or self.keep * (self.num_experts // self.groups) < self.top):
            raise UnsupportedModelError(f"routed experts: {self.num_experts} experts in {self.groups} groups of which {self.keep} "
                                        f"are kept cannot give {self.top} choices")
        self.renormalize, self.accumulate = bool(renormalize), bool(accumulate)
        self.expert_prefix, self.names, self.router_name = expert_prefix, tuple(names), router_name
        if self.shared is not None and bool(getattr(self.shared, "accumulate", True)) is not True:
            raise UnsupportedModelError("routed experts: the shared expert adds its result (accumulate=True)")

    def tensor_specs(self) -> List[TensorSpec]:
        F, D = self.expert_size, self.hidden_size
        specs = []
        for e in range(self.num_experts):
            p = f"{self.expert_prefix}{e}."
            if self.gated:
                specs.append(TensorSpec(p + self.names[0], (F, D)))
            specs += [TensorSpec(p + self.names[1], (F, D)), TensorSpec(p + self.names[2], (D, F))]
        specs.append(TensorSpec(self.router_name, (self.router_size, D)))
        if self.correction_name:
            specs.append(TensorSpec(self.correction_name, (self.router_size,), "small_bias"))
        if self.shared is not None:
            specs += [s.with_prefix(self.shared_prefix) for s in self.shared.tensor_specs()]
        return specs

    def load(self, tensors: Dict[str, torch.Tensor], dtype, device) -> None:
        super().load(tensors, dtype, device)
        E, p = self.num_experts, self.expert_prefix
        F, b = self.expert_size, INTERLEAVE
        self.w_router = tensors[self.router_name]
        self.correction = tensors[self.correction_name].to(torch.float32).contiguous() if self.correction_name else None
        if self.shared is not None:
            sp = self.shared_prefix
            self.shared.load({n[len(sp):]: tensors[n] for n in (sp + s.name for s in self.shared.tensor_specs())}, dtype, device)
        self.w_down = torch.stack([tensors[f"{p}{e}.{self.names[2]}"] for e in range(E)]).contiguous()   # [E, D, F]
        if not self.gated:
            self.interleave = 0
            self.w_up = torch.stack([tensors[f"{p}{e}.{self.names[1]}"] for e in range(E)]).contiguous()   # [E, F, D]
            self.tile = ops.grouped_tile_rows(self.w_up.dtype if self.w_down.dtype == self.w_up.dtype else torch.float32)
            return
        mats = []
        for e in range(E):
            g, u = tensors[f"{p}{e}.{self.names[0]}"], tensors[f"{p}{e}.{self.names[1]}"]
            if g.dtype == torch.bfloat16 and u.dtype == torch.bfloat16 and F % b == 0:
                # gate and up rows interleaved in blocks of 16, as the dense gated feed-forward keeps them: the
                # matrix-core product then applies the activation before anything is stored
                mats.append(torch.stack([g.view(F // b, b, -1), u.view(F // b, b, -1)], dim=1).reshape(2 * F, -1))
            else:
                mats.append(torch.cat([g, u], dim=0))
        self.interleave = b if all(t.dtype == torch.bfloat16 for t in mats) and F % b == 0 else 0
        self.w_gate_up = torch.stack(mats).contiguous()                   # [E, 2F, D]
        self.tile = ops.grouped_tile_rows(self.w_gate_up.dtype if self.w_down.dtype == self.w_gate_up.dtype else torch.float32)

    def streamed_weights(self) -> List[torch.Tensor]:
        return self.shared.streamed_weights() if self.shared is not None else []

    @property
    def graph_safe(self) -> bool:
        return self.shared is None or bool(self.shared.graph_safe)

    def forward(self, h: torch.Tensor, x: torch.Tensor, ctx: StepContext) -> None:
        T, ws = h.shape[0], ctx.workspace if ctx is not None else None
        logits = torch.empty((T, self.router_size), dtype=torch.float32, device=h.device)
        ops.gemm(logits, h, self.w_router, ws=ws)
        ids, weights = ops.route(logits, self.top, self.groups, self.keep, self.renormalize, self.correction, self.renorm_eps)
        rows = ops.group_entries(ids, self.num_experts, self.tile)
        a = ops.gather_rows(h, rows)
        act = torch.empty((rows.rows, self.expert_size), dtype=self.dtype, device=h.device)
        if self.gated:
            ops.grouped_gemm_swiglu(act, a, self.w_gate_up, rows, self.interleave)
        else:
            ops.grouped_gemm_relu_squared(act, a, self.w_up, rows)
        y = torch.empty((rows.rows, self.hidden_size), dtype=torch.float32, device=h.device)
        ops.grouped_gemm(y, act, self.w_down, rows)
        if self.accumulate:
            ops.materialize(x, ws)
        if self.identity:
            ops.combine_choices(x, y, weights, rows, accumulate=self.accumulate, ids=ids, num_real=self.num_experts, h=h)
        else:
            ops.combine_choices(x, y, weights, rows, accumulate=self.accumulate)
        if self.shared is not None:
            may_defer, ctx.may_defer = ctx.may_defer, False
            self.shared.forward(h, x, ctx)
            ctx.may_defer = may_defer


FEED_FORWARDS.register("routed_experts", RoutedExperts)
