"""Plain implementation of the Muretar design: whole sequences, no cache, float64, loops over
positions and heads, one function per mechanism.  It shares nothing with the engine: it takes
the raw config.json mapping and a dict of tensors by their names in a model folder.

    x_0 = embed[token]
    per layer:  x <- x + LN(mixer(LN(x; norm1)); norm1b);  x <- x + LN(ff(LN(x; norm2)); norm2b)
    logits = head . LN(x; final.norm)

LN is a layer norm with weight and bias.  A layer's mixer is one of

* ``attention``: differential attention.  Every head holds two score maps over the same values,
  ``o = A1 v - lam * A2 v``, ``lam = exp(<lq1, lk1>) - exp(<lq2, lk2>) + diff``, then a unit root
  mean square over the head's values and a factor ``1 - diff``; no rotation; biases on q, k, v.
* ``parallel``: grouped-query attention with partly rotated heads (neighbouring pairs, all
  frequencies divided by a constant) beside a gated delta rule with one decay per head; each
  result is RMS-normalised over the width with a weight of its own, and the two are averaged.
* ``gla``: gated linear attention, ``S <- diag(alpha) S + k v^T``, ``o = S^T q``, with a decay per
  key channel ``alpha = sigmoid(W2 W1 h + b)^(1 / tau)``.

A feed-forward is dense and gated (silu), or routed: a softmax router over real and identity
experts, a correction added for the choice only, the chosen scores divided by their sum, experts
``W_down relu(W_up h)^2``, identity experts that hand the input through, and a shared expert.
``weights_of: j`` in a layer's entry: the layer is run with the tensors named ``l<j>.`` and keeps its own cache or state.
"""
from __future__ import annotations

import json
import math
import os
from typing import Callable, Dict, List, Optional

import torch

F64 = torch.float64
Round = Optional[Callable[[torch.Tensor], torch.Tensor]]
UNIT_EPS = 1e-6
WEIGHT_SUM_EPS = 1e-20


def bf16_round(t: torch.Tensor) -> torch.Tensor:
    return t.to(torch.bfloat16).to(t.dtype)


def _r(t: torch.Tensor, act_round: Round) -> torch.Tensor:
    """Activations rounded where an engine that computes in a 16-bit type rounds them (None: not at all)."""
    return act_round(t.to(torch.float32)).to(F64) if act_round is not None else t


def read_model_folder(model_dir: str):
    from safetensors.torch import load_file
    with open(os.path.join(model_dir, "config.json"), encoding="utf-8") as f:
        config = json.load(f)
    return config, load_file(os.path.join(model_dir, "model.safetensors"))


# ------------------------------------------------------------------ small functions
def layer_norm(x: torch.Tensor, w: torch.Tensor, b: torch.Tensor, eps: float) -> torch.Tensor:
    """(x - mean) / sqrt(mean of squared deviations + eps) * w + b over the last axis."""
    mu = x.mean(dim=-1, keepdim=True)
    dev = x - mu
    return dev / torch.sqrt((dev * dev).mean(dim=-1, keepdim=True) + eps) * w + b


def rms_norm(x: torch.Tensor, w: Optional[torch.Tensor], eps: float) -> torch.Tensor:
    y = x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)
    return y if w is None else y * w


def silu(x: torch.Tensor) -> torch.Tensor:
    return x / (1.0 + torch.exp(-x))


def sigmoid(x: torch.Tensor) -> torch.Tensor:
    return 1.0 / (1.0 + torch.exp(-x))


def softplus(x: torch.Tensor) -> torch.Tensor:
    return torch.where(x > 30.0, x, torch.log1p(torch.exp(torch.clamp(x, max=30.0))))


def causal_conv(u: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """u [T, C]; w [C, taps], the last column weighs the current token; zeros before the start."""
    T, C = u.shape
    taps = w.shape[1]
    out = torch.zeros((T, C), dtype=F64)
    for t in range(T):
        for j in range(taps):
            src = t - (taps - 1) + j
            if src >= 0:
                out[t] += w[:, j] * u[src]
    return out


def rotate_pairs(x: torch.Tensor, pos: int, dims: int, base: float, divide: float = 1.0) -> torch.Tensor:
    """x [heads, dim]: pairs (2i, 2i+1), i < dims / 2, turned by pos * base^(-2i / dims) / divide; the rest unchanged."""
    y = x.clone()
    for i in range(dims // 2):
        a = pos * (base ** (-2.0 * i / dims) / divide)
        c, s = math.cos(a), math.sin(a)
        u, v = x[:, 2 * i].clone(), x[:, 2 * i + 1].clone()
        y[:, 2 * i] = u * c - v * s
        y[:, 2 * i + 1] = v * c + u * s
    return y


def causal_softmax_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float) -> torch.Tensor:
    """One head: q, k [T, d], v [T, dv]; position i sees j <= i; ordinary softmax."""
    T = q.shape[0]
    out = torch.zeros((T, v.shape[1]), dtype=F64)
    for i in range(T):
        s = (k[: i + 1] @ q[i]) * scale
        p = torch.exp(s - s.max())
        out[i] = (p / p.sum()) @ v[: i + 1]
    return out


# ------------------------------------------------------------------ mixers
def differential_attention(h: torch.Tensor, m: dict, W: Dict[str, torch.Tensor], p: str, eps: float, act_round: Round = None) -> torch.Tensor:
    H, G, d, dv, diff, scale = m["heads"], m["kv_heads"], m["dim"], m["vdim"], float(m["diff"]), float(m["scale"])
    T = h.shape[0]
    q = _r(h @ W[p + "q"].T + W[p + "q.b"], act_round).view(T, H, 2, d)
    k = _r(h @ W[p + "k"].T + W[p + "k.b"], act_round).view(T, G, 2, d)
    v = _r(h @ W[p + "v"].T + W[p + "v.b"], act_round).view(T, G, dv)
    lam = math.exp(float((W[p + "lq1"] * W[p + "lk1"]).sum())) - math.exp(float((W[p + "lq2"] * W[p + "lk2"]).sum())) + diff
    out = torch.zeros((T, H, dv), dtype=F64)
    for n in range(H):
        g = n // (H // G)
        a1 = causal_softmax_attention(q[:, n, 0], k[:, g, 0], v[:, g], scale)
        a2 = causal_softmax_attention(q[:, n, 1], k[:, g, 1], v[:, g], scale)
        out[:, n] = rms_norm(a1 - lam * a2, None, eps) * (1.0 - diff)
    return _r(out.reshape(T, H * dv), act_round) @ W[p + "o"].T


def rotary_attention(h: torch.Tensor, m: dict, W: Dict[str, torch.Tensor], p: str, act_round: Round = None) -> torch.Tensor:
    H, G, d, dv, scale = m["heads"], m["kv_heads"], m["dim"], m["vdim"], float(m["scale"])
    rot = m.get("rot")
    T = h.shape[0]
    q = (h @ W[p + "q"].T + W[p + "q.b"]).view(T, H, d)
    k = (h @ W[p + "k"].T + W[p + "k.b"]).view(T, G, d)
    v = _r(h @ W[p + "v"].T + W[p + "v.b"], act_round).view(T, G, dv)
    if rot:
        divide = float((rot.get("scaling") or {}).get("factor", 1.0))
        q = torch.stack([rotate_pairs(q[t], t, rot["dims"], float(rot["base"]), divide) for t in range(T)])
        k = torch.stack([rotate_pairs(k[t], t, rot["dims"], float(rot["base"]), divide) for t in range(T)])
    q, k = _r(q, act_round), _r(k, act_round)
    out = torch.zeros((T, H, dv), dtype=F64)
    for n in range(H):
        g = n // (H // G)
        out[:, n] = causal_softmax_attention(q[:, n], k[:, g], v[:, g], scale)
    return _r(out.reshape(T, H * dv), act_round) @ W[p + "o"].T + W[p + "o.b"]


def delta_rule_walk(q, k, v, beta, decay):
    """One head: q, k [T, d] (already unit vectors), v [T, dv], beta, decay [T]:
    S <- decay S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q."""
    T, d = q.shape
    S = torch.zeros((d, v.shape[1]), dtype=F64)
    out = torch.zeros((T, v.shape[1]), dtype=F64)
    for t in range(T):
        S = decay[t] * S
        u = beta[t] * (v[t] - S.T @ k[t])
        S = S + torch.outer(k[t], u)
        out[t] = S.T @ q[t]
    return out


def gated_delta_rule(h: torch.Tensor, m: dict, W: Dict[str, torch.Tensor], p: str, eps: float, act_round: Round = None) -> torch.Tensor:
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q = silu(causal_conv(h @ W[p + "q"].T, W[p + "q.conv"])).view(T, G, d)
    k = silu(causal_conv(h @ W[p + "k"].T, W[p + "k.conv"])).view(T, G, d)
    v = silu(causal_conv(h @ W[p + "v"].T, W[p + "v.conv"])).view(T, H, dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + UNIT_EPS) * d ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + UNIT_EPS)
    beta = sigmoid(h @ W[p + "b"].T)                                                        # [T, H]
    decay = torch.exp(-torch.exp(W[p + "A_log"]) * softplus(h @ W[p + "a"].T + W[p + "dt_bias"]))   # [T, H]
    gate = silu(h @ W[p + "g"].T).view(T, H, dv)
    out = torch.zeros((T, H, dv), dtype=F64)
    for n in range(H):
        g = n // (H // G)
        o = delta_rule_walk(q[:, g], k[:, g], v[:, n], beta[:, n], decay[:, n])
        out[:, n] = rms_norm(o, W[p + "norm"], eps) * gate[:, n]
    return _r(out.reshape(T, H * dv), act_round) @ W[p + "o"].T


def parallel_mixer(h: torch.Tensor, m: dict, W: Dict[str, torch.Tensor], p: str, eps: float, act_round: Round = None) -> torch.Tensor:
    left = rotary_attention(h, m["left"], W, p + "left.", act_round)
    right = gated_delta_rule(h, m["right"], W, p + "right.", eps, act_round)
    return 0.5 * (rms_norm(left, W[p + "left.out"], eps) + rms_norm(right, W[p + "right.out"], eps))


def decayed_outer_walk(q, k, v, alpha):
    """One head: q, k, alpha [T, d], v [T, dv]: S <- diag(alpha) S + k v^T; o = S^T q."""
    T, d = q.shape
    S = torch.zeros((d, v.shape[1]), dtype=F64)
    out = torch.zeros((T, v.shape[1]), dtype=F64)
    for t in range(T):
        S = alpha[t][:, None] * S + torch.outer(k[t], v[t])
        out[t] = S.T @ q[t]
    return out


def gated_linear_attention(h: torch.Tensor, m: dict, W: Dict[str, torch.Tensor], p: str, eps: float, act_round: Round = None) -> torch.Tensor:
    H, d, dv, tau = m["heads"], m["dim"], m["vdim"], float(m["tau"])
    T = h.shape[0]
    q = (h @ W[p + "q"].T).view(T, H, d) * d ** -0.5
    k = (h @ W[p + "k"].T).view(T, H, d)
    v = (h @ W[p + "v"].T).view(T, H, dv)
    z = _r(h @ W[p + "a1"].T, act_round) @ W[p + "a2"].T + W[p + "a2.b"]
    alpha = (sigmoid(z) ** (1.0 / tau)).view(T, H, d)
    gate = silu(h @ W[p + "g"].T).view(T, H, dv)
    out = torch.zeros((T, H, dv), dtype=F64)
    for n in range(H):
        out[:, n] = rms_norm(decayed_outer_walk(q[:, n], k[:, n], v[:, n], alpha[:, n]), W[p + "norm"], eps) * gate[:, n]
    return _r(out.reshape(T, H * dv), act_round) @ W[p + "o"].T


# ------------------------------------------------------------------ feed-forwards
def gated_unit(h, W, p, act_round: Round = None):
    return _r(silu(h @ W[p + "gate"].T) * (h @ W[p + "up"].T), act_round) @ W[p + "down"].T


def squared_relu_unit(h, W, p, act_round: Round = None):
    a = torch.clamp(h @ W[p + "up"].T, min=0.0)
    return _r(a * a, act_round) @ W[p + "down"].T


def route(z: torch.Tensor, correction: torch.Tensor, top: int):
    """z [E] router logits -> (chosen indices, weights): softmax over all, the choice by score + correction
    (the lower index among equals), the weights the chosen scores over their sum."""
    s = torch.exp(z - z.max())
    s = s / s.sum()
    choice = s + correction
    order = sorted(range(z.shape[0]), key=lambda e: (-float(choice[e]), e))[:top]
    w = torch.stack([s[e] for e in order])
    return order, w / (w.sum() + WEIGHT_SUM_EPS)


def routed_experts(h: torch.Tensor, mlp: dict, W: Dict[str, torch.Tensor], p: str, act_round: Round = None, choices: Optional[list] = None,
                   margins: Optional[list] = None, chosen: Optional[list] = None) -> torch.Tensor:
    """``choices``: per token the experts to use instead of the router's own choice (weights still from the scores).
    ``chosen`` / ``margins``: lists that receive, per token, the router's own choice and by how much (in choice score) its
    last chosen expert beat the best one left out."""
    real, ident, top = mlp["router"]["experts"], mlp["router"].get("identity", 0), mlp["router"]["top"]
    T = h.shape[0]
    z = h @ W[p + "router"].T
    out = torch.zeros_like(h)
    for t in range(T):
        order, w = route(z[t], W[p + "correction"], top)
        if chosen is not None:
            chosen.append(list(order))
        if margins is not None:
            sc = torch.exp(z[t] - z[t].max())
            sc = sc / sc.sum() + W[p + "correction"]
            ranked = sorted((float(v) for v in sc), reverse=True)
            margins.append(ranked[top - 1] - ranked[top] if top < len(ranked) else float("inf"))
        if choices is not None:
            s = torch.exp(z[t] - z[t].max())
            s = s / s.sum()
            order = list(choices[t])
            w = torch.stack([s[e] for e in order])
            w = w / (w.sum() + WEIGHT_SUM_EPS)
        for e, we in zip(order, w):
            if e >= real:
                assert e < real + ident
                out[t] += we * h[t]
            else:
                out[t] += we * squared_relu_unit(h[t:t + 1], W, f"{p}e{e}.", act_round)[0]
    if mlp.get("shared"):
        out = out + squared_relu_unit(h, W, p + "shared.", act_round)
    return out


# ------------------------------------------------------------------ the model
def forward(config: dict, W: Dict[str, torch.Tensor], tokens: List[int], act_round: Round = None, streams: Optional[list] = None,
            choices: Optional[dict] = None, margins: Optional[dict] = None, chosen: Optional[dict] = None) -> torch.Tensor:
    """Logits [T, vocab] (float64) of the whole sequence.  ``streams``: a list that receives the residual
    stream after every layer.  ``choices``: {layer index: per token the experts to use}; ``margins`` / ``chosen``: dicts
    that receive, per routed layer, what ``routed_experts`` reports."""
    W = {n: t.to(F64) for n, t in W.items()}
    eps = float(config["norm"]["eps"])
    x = W["embed"][torch.tensor(tokens, dtype=torch.long)]
    for i, layer in enumerate(config["layers"]):
        j = layer.get("weights_of", i)
        if j is None:
            j = i
        p = f"l{j}."
        ln = lambda v, name: layer_norm(v, W[p + name], W[p + name + ".b"], eps)
        h = _r(ln(x, "norm1"), act_round)
        kind, m = layer["type"], layer["mixer"]
        if kind == "attention":
            y = differential_attention(h, m, W, p + "mix.", eps, act_round)
        elif kind == "parallel":
            y = parallel_mixer(h, m, W, p + "mix.", eps, act_round)
        elif kind == "gla":
            y = gated_linear_attention(h, m, W, p + "mix.", eps, act_round)
        else:
            raise ValueError(f"unknown layer type {kind}")
        x = x + ln(y, "norm1b")
        mlp = layer.get("mlp")
        if mlp is not None:
            h = _r(ln(x, "norm2"), act_round)
            if mlp["kind"] == "dense":
                y = gated_unit(h, W, p + "mlp.", act_round)
            else:
                y = routed_experts(h, mlp, W, p + "mlp.", act_round, None if choices is None else choices.get(i),
                                   None if margins is None else margins.setdefault(i, []), None if chosen is None else chosen.setdefault(i, []))
            x = x + ln(y, "norm2b")
        if streams is not None:
            streams.append(x.clone())
    h = _r(layer_norm(x, W["final.norm"], W["final.norm.b"], eps), act_round)
    return h @ W["head"].T


def greedy(config: dict, W: Dict[str, torch.Tensor], prompt: List[int], new_tokens: int) -> List[int]:
    tokens, out = list(prompt), []
    for _ in range(new_tokens):
        nxt = int(torch.argmax(forward(config, W, tokens)[-1]))
        out.append(nxt)
        tokens.append(nxt)
    return out
