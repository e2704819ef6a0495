"""Dokanex: a pre-norm decoder with a scaled embedding, a tied and capped head, and two kinds of
attention layers - grouped-query attention within chunks of positions (unit queries and keys per
head, capped scores, a sink in the softmax, a gate per head; a layer may attend over the keys and
values of an earlier layer), and attention through a low-rank latent with one rotated key part
for all heads (neighbouring pairs, frequencies scaled by a ramp).

    x = embed[token] * scale
    per layer:  x <- x + mixer(norm(x; norm1));  x <- x + ffn(norm(x; norm2))     (layers with a feed-forward)
    logits = cap * tanh((embed . norm(x; final.norm)) / cap)

Layer i's tensors start with ``l<i>.``; the mixer's with ``mix.``, the feed-forward's with ``mlp.``;
norms are named by themselves (``l<i>.norm1``, ``final.norm``); the head is the embedding's table.
"""
from __future__ import annotations

from ..config.dokanex import ChunkAttentionConfig, DokanexConfig, LatentAttentionConfig
from ..errors import UnsupportedModelError
from ..parts import BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITION_ENCODINGS
from ..parts.embedding import LMHead, TokenEmbedding
from ..parts.model import ModelSpec, RunEntry
from ..parts.rope import RampScaling
from ..registry import register_architecture


def _cache_reach(cfg: DokanexConfig, owner: int):
    """How far back the keys of layer ``owner`` are read, by itself or by the layers that attend over them: the
    longest chunk among them, or None (everything) when one of them sees all earlier positions."""
    chunks = [l.mixer.chunk for i, l in enumerate(cfg.layers)
              if isinstance(l.mixer, ChunkAttentionConfig) and (i == owner or l.mixer.kv_from == owner)]
    return None if any(c is None for c in chunks) else max(chunks)


def _mixer(cfg: DokanexConfig, i: int, ropes: dict):
    m, D, eps = cfg.layers[i].mixer, cfg.width, cfg.norm_eps
    if isinstance(m, ChunkAttentionConfig):
        own = m.kv_from is None
        return MIXERS.make("sink_window_attention", hidden_size=D, num_heads=m.heads, num_kv_heads=m.kv_heads, head_dim=m.dim,
                           value_dim=m.vdim, scale=m.scale, window=None, eps=eps, distance_bias=False, norm_per_head=True,
                           norm_weights=False, softcap=m.softcap, chunk=m.chunk, own_kv=own,
                           cache_reach=_cache_reach(cfg, i) if own else None)
    if isinstance(m, LatentAttentionConfig):
        s = m.rot_scaling
        key = (m.rot_dim, m.rot_base, s)
        if key not in ropes:      # layers that rotate alike share the part, and with it a step's table of cosines and sines
            scaling = RampScaling(s.factor, s.original, s.fast, s.slow) if s is not None else None
            ropes[key] = POSITION_ENCODINGS.make("rope", head_dim=m.rot_dim, theta=m.rot_base, scaling=scaling, interleaved=True)
        return MIXERS.make("latent_attention", hidden_size=D, num_heads=m.heads, head_dim=m.dim, rot_dim=m.rot_dim,
                           value_dim=m.vdim, q_rank=m.q_rank, kv_rank=m.kv_rank, scale=m.scale, eps=eps, position=ropes[key])
    raise UnsupportedModelError(f"no mixer for {type(m).__name__}")


def build_dokanex(cfg: DokanexConfig) -> ModelSpec:
    D, eps = cfg.width, cfg.norm_eps
    norm = lambda: NORMS.make("rmsnorm", dim=D, eps=eps, tensor_name="")
    layers, order, ignorable, ropes = [], [], [], {}
    for i, layer in enumerate(cfg.layers):
        norm2 = ffn = None
        if layer.mlp is not None:
            norm2 = ("norm2", norm())
            ffn = ("mlp.", FEED_FORWARDS.make("swiglu", hidden_size=D, intermediate_size=layer.mlp.ff, names=("gate", "up", "down")))
        else:
            ignorable.append(f"l{i}.norm2")      # a layer without a feed-forward has no use for its norm
        block = BLOCKS.make("prenorm", norm1=("norm1", norm()), mixer=("mix.", _mixer(cfg, i, ropes)), norm2=norm2, ffn=ffn)
        layers.append((f"l{i}.", block))
        # every layer runs once, in order: the entry's index is the layer's
        order.append(RunEntry(i, cache_of=getattr(layer.mixer, "kv_from", None)))
    return ModelSpec(
        hidden_size=D, vocab_size=cfg.vocab, max_positions=cfg.max_positions,
        embedding=("embed", TokenEmbedding(cfg.vocab, D, tensor_name="", scale=cfg.embedding_scale)), layers=layers, run_order=order,
        final_norm=("final.norm", norm()), head=("head", LMHead(cfg.vocab, D, tied=True, tensor_name="", softcap=cfg.logit_softcap)),
        ignorable=tuple(ignorable),
    )


register_architecture("Dokanex", DokanexConfig, build_dokanex)
