"""Plain implementation of the Dokanex design: whole sequences, no cache, float64, one function
per mechanism.  It shares nothing with the engine: it takes the raw config.json mapping and a dict
of tensors by their names in a model folder.

    x_0 = embed[token] * scale
    per layer:  x <- x + mixer(norm(x; norm1));  x <- x + ff(norm(x; norm2))     (layers with a feed-forward)
    logits = cap * tanh((embed . norm(x; final.norm)) / cap)

A layer's mixer is grouped-query attention within chunks of positions (unit queries and keys,
capped scores, a sink in the softmax, a gate per head, optionally on the keys and values of an
earlier layer), or attention through a low-rank latent with a rotated part that all heads share.
"""
from __future__ import annotations

import json
import math
import os
from typing import Callable, Dict, List, Optional

import torch

F64 = torch.float64
Round = Optional[Callable[[torch.Tensor], torch.Tensor]]


def bf16_round(t: torch.Tensor) -> torch.Tensor:
    return t.to(torch.bfloat16).to(t.dtype)


def _r(t: torch.Tensor, act_round: Round) -> torch.Tensor:
    """Activations rounded where an engine that computes in a 16-bit type rounds them (None: not at all)."""
    return act_round(t.to(torch.float32)).to(F64) if act_round is not None else t


def read_model_folder(model_dir: str):
    """(raw config.json, tensors by name) of a model folder written with safetensors."""
    from safetensors.torch import load_file
    with open(os.path.join(model_dir, "config.json"), encoding="utf-8") as f:
        config = json.load(f)
    return config, load_file(os.path.join(model_dir, "model.safetensors"))


def rms_norm(x: torch.Tensor, w: Optional[torch.Tensor], eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) [* w] over the last axis."""
    y = x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)
    return y if w is None else y * w


def silu(x: torch.Tensor) -> torch.Tensor:
    return x / (1.0 + torch.exp(-x))


def sigmoid(x: torch.Tensor) -> torch.Tensor:
    return 1.0 / (1.0 + torch.exp(-x))


def capped(s: torch.Tensor, cap: Optional[float]) -> torch.Tensor:
    return s if not cap else cap * torch.tanh(s / cap)


def chunk_mask(T: int, size: Optional[int]) -> torch.Tensor:
    """[T, T] bool: query i sees key j when j <= i and, with chunks, both lie in the same chunk of ``size`` positions."""
    i = torch.arange(T).unsqueeze(1)
    j = torch.arange(T).unsqueeze(0)
    seen = j <= i
    if size:
        seen = seen & (torch.div(i, size, rounding_mode="floor") == torch.div(j, size, rounding_mode="floor"))
    return seen


def softmax_with_sink(s: torch.Tensor, seen: torch.Tensor, sink: Optional[float]) -> torch.Tensor:
    """Rows of weights exp(s) / (sum over the seen keys of exp(s) [+ exp(sink)]); unseen keys weigh nothing."""
    s = torch.where(seen, s, torch.full_like(s, -math.inf))
    m = s.max(dim=-1, keepdim=True).values
    if sink is not None:
        m = torch.clamp(m, min=float(sink))
    e = torch.exp(s - m)
    den = e.sum(dim=-1, keepdim=True)
    if sink is not None:
        den = den + torch.exp(torch.tensor(float(sink), dtype=F64) - m)
    return e / den


def yarn_frequencies(dims: int, base: float, scaling: Optional[dict]):
    """(frequencies [dims / 2], factor on cos and sin).  Without scaling base^(-2i / dims) and 1.  With it, pair i's
    frequency is blended between f_i and f_i / factor by a ramp over the pair index that runs from the pair whose
    wavelength fits ``fast`` times into the original length to the one that fits ``slow`` times."""
    f = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    if not scaling:
        return f, 1.0
    factor, orig = float(scaling["factor"]), float(scaling["original"])
    where = lambda turns: dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
    lo = max(math.floor(where(float(scaling["fast"]))), 0)
    hi = min(math.ceil(where(float(scaling["slow"]))), dims - 1)
    out = []
    for i, fi in enumerate(f):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(fi / factor * ramp + fi * (1.0 - ramp))
    return out, 0.1 * math.log(factor) + 1.0


def rotate_pairs(x: torch.Tensor, positions: torch.Tensor, freqs: List[float], mult: float) -> torch.Tensor:
    """x [T, ..., dims]: the pair (2i, 2i + 1) at position p turned by p * freqs[i]; cos and sin times ``mult``."""
    y = x.clone()
    shape = [x.shape[0]] + [1] * (x.dim() - 2)
    for i, f in enumerate(freqs):
        a = positions.to(F64) * f
        c, s = (torch.cos(a) * mult).reshape(shape), (torch.sin(a) * mult).reshape(shape)
        u, v = x[..., 2 * i], x[..., 2 * i + 1]
        y[..., 2 * i] = u * c - v * s
        y[..., 2 * i + 1] = v * c + u * s
    return y


def chunk_attention_keys(h: torch.Tensor, m: dict, W: Dict[str, torch.Tensor], eps: float, act_round: Round = None):
    """(unit keys [T, G, dim], values [T, G, vdim]) of a layer that has projections of its own."""
    T, G, d, dv = h.shape[0], m["kv_heads"], m["dim"], m["vdim"]
    k = rms_norm((h @ W["k"].T).reshape(T, G, d), None, eps)
    v = (h @ W["v"].T).reshape(T, G, dv)
    return _r(k, act_round), _r(v, act_round)


def chunk_attention(h: torch.Tensor, m: dict, W: Dict[str, torch.Tensor], eps: float, kv, act_round: Round = None) -> torch.Tensor:
    """The attention mixer on input h [T, D] with keys and values ``kv`` (its own, or an earlier layer's)."""
    T, H, G, d, dv = h.shape[0], m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    k, v = kv
    q = _r(rms_norm((h @ W["q"].T).reshape(T, H, d), None, eps), act_round)
    gate = sigmoid(h @ W["g"].T)                                  # [T, H]
    size = (m.get("mask") or {}).get("size")
    seen = chunk_mask(T, size)
    out = torch.zeros((T, H, dv), dtype=F64)
    for n in range(H):
        g = n // (H // G)
        s = capped((q[:, n] @ k[:, g].T) * m["scale"], m.get("softcap"))
        p = softmax_with_sink(s, seen, float(W["sink"][n]))
        out[:, n] = (p @ v[:, g]) * gate[:, n:n + 1]
    return _r(out.reshape(T, H * dv), act_round) @ W["o"].T


def latent_attention(h: torch.Tensor, m: dict, W: Dict[str, torch.Tensor], eps: float, positions: torch.Tensor,
                     act_round: Round = None) -> torch.Tensor:
    """Attention whose queries come through a latent of q_rank and whose keys and values through one of kv_rank;
    a head's key is [its own unrotated part | one rotated part for all heads]."""
    T, H, d, dr, dv, rank = h.shape[0], m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    freqs, mult = yarn_frequencies(m["rot"]["dims"], m["rot"]["base"], m["rot"].get("scaling"))
    cq = _r(rms_norm(h @ W["dq"].T, W["dq.norm"], eps), act_round)
    q = _r(cq @ W["uq"].T, act_round).reshape(T, H, d + dr)
    q_plain, q_rot = q[..., :d], rotate_pairs(q[..., d:], positions, freqs, mult)
    down = h @ W["dkv"].T
    c = _r(rms_norm(down[:, :rank], W["dkv.norm"], eps), act_round)
    k_rot = _r(rotate_pairs(down[:, rank:], positions, freqs, mult), act_round)        # [T, dr]
    k_plain = (c @ W["uk"].T).reshape(T, H, d)
    v = (c @ W["uv"].T).reshape(T, H, dv)
    seen = chunk_mask(T, None)
    out = torch.zeros((T, H, dv), dtype=F64)
    for n in range(H):
        s = (q_plain[:, n] @ k_plain[:, n].T + q_rot[:, n] @ k_rot.T) * m["scale"]
        out[:, n] = softmax_with_sink(s, seen, None) @ v[:, n]
    return _r(out.reshape(T, H * dv), act_round) @ W["o"].T


def dense_ff(h: torch.Tensor, W: Dict[str, torch.Tensor], act_round: Round = None) -> torch.Tensor:
    return _r(silu(h @ W["gate"].T) * (h @ W["up"].T), act_round) @ W["down"].T


def _sub(tensors: Dict[str, torch.Tensor], prefix: str) -> Dict[str, torch.Tensor]:
    return {n[len(prefix):]: t.to(F64) for n, t in tensors.items() if n.startswith(prefix)}


def forward(config: dict, tensors: Dict[str, torch.Tensor], tokens, act_round: Round = None, streams: Optional[list] = None) -> torch.Tensor:
    """float64 logits [T, vocab] of one whole sequence; ``streams`` collects the stream after every layer."""
    eps = float(config["norm"]["eps"])
    embed = tensors["embed"].to(F64)
    ids = torch.as_tensor(list(tokens), dtype=torch.long)
    positions = torch.arange(len(ids))
    x = embed[ids] * float(config["embedding"]["scale"])
    kept = {}
    for i, layer in enumerate(config["layers"]):
        m = layer["mixer"]
        h = _r(rms_norm(x, tensors[f"l{i}.norm1"].to(F64), eps), act_round)
        W = _sub(tensors, f"l{i}.mix.")
        if layer["type"] == "attention":
            src = m.get("kv_from")
            kv = kept[src] if src is not None else chunk_attention_keys(h, m, W, eps, act_round)
            kept[i] = kv
            x = x + chunk_attention(h, m, W, eps, kv, act_round)
        elif layer["type"] == "latent_attention":
            x = x + latent_attention(h, m, W, eps, positions, act_round)
        else:
            raise ValueError(f"layer type {layer['type']!r}")
        if layer.get("mlp") is not None:
            h = _r(rms_norm(x, tensors[f"l{i}.norm2"].to(F64), eps), act_round)
            x = x + dense_ff(h, _sub(tensors, f"l{i}.mlp."), act_round)
        if streams is not None:
            streams.append(x.clone())
    h = _r(rms_norm(x, tensors["final.norm"].to(F64), eps), act_round)
    logits = h @ embed.T
    cap = config.get("logit_softcap")
    return capped(logits, cap)


def greedy(config: dict, tensors: Dict[str, torch.Tensor], prompt, new_tokens: int) -> List[int]:
    """Greedy continuation, the whole sequence run again for every token."""
    seq = list(prompt)
    for _ in range(new_tokens):
        seq.append(int(torch.argmax(forward(config, tensors, seq)[-1])))
    return seq[len(prompt):]
