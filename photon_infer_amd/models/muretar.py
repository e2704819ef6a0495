"""Muretar: a decoder whose every sublayer sits between two layer norms, with three kinds of mixer - differential
attention, rotary attention beside a gated delta rule, gated linear attention - and feed-forwards that are dense and
gated or routed (real and identity experts, a shared expert).

    x = embed[token]
    per layer:  x <- x + LN(mixer(LN(x; norm1)); norm1b);  x <- x + LN(ff(LN(x; norm2)); norm2b)   (layers with a feed-forward)
    logits = head . LN(x; final.norm)

    mixer of an "attention" layer:  two softmax maps per head over the same values, their difference normalised
    mixer of a "parallel" layer:    (rms(attention(h); left.out) + rms(delta_rule(h); right.out)) / 2
    mixer of a "gla" layer:         gated linear attention with a decay per key channel

A layer with ``weights_of: j`` has no tensors: the run order names layer j's block again, and every entry of the
run order gets a cache or state of its own.  Layer i's tensors start with ``l<i>.``; the mixers' with ``mix.``
(``mix.left.`` / ``mix.right.``), the feed-forward's with ``mlp.``; norms are named by themselves (``l<i>.norm1``,
``final.norm``) with their bias at ``<name>.b``.
"""
from __future__ import annotations

from ..config.llama import RopeScaling
from ..config.muretar import DiffAttentionConfig, GlaConfig, MuretarConfig, ParallelConfig
from ..errors import UnsupportedModelError
from ..parts import BLOCKS, FEED_FORWARDS, MIXERS, NORMS, POSITION_ENCODINGS
from ..parts.embedding import LMHead, TokenEmbedding
from ..parts.model import ModelSpec, RunEntry
from ..registry import register_architecture


def _branches(cfg: MuretarConfig, m, ropes: dict):
    """[(prefix, mixer, norm of its result or None)] of one layer."""
    D, eps = cfg.width, cfg.norm_eps
    if isinstance(m, DiffAttentionConfig):
        mixer = MIXERS.make("differential_attention", hidden_size=D, num_heads=m.heads, num_kv_heads=m.kv_heads, head_dim=m.dim,
                            value_dim=m.vdim, scale=m.scale, diff=m.diff, eps=eps, accumulate=False)
        return [("mix.", mixer, None)]
    if isinstance(m, GlaConfig):
        if m.decay_rank is None:
            raise UnsupportedModelError("the decay projection's inner size is open: a model folder gives it by its tensors "
                                        "(registry.load_config), a bare configuration names 'decay_rank'")
        mixer = MIXERS.make("gated_linear_attention", hidden_size=D, num_heads=m.heads, key_dim=m.dim, value_dim=m.vdim,
                            decay_rank=m.decay_rank, tau=m.tau, eps=eps, accumulate=False)
        return [("mix.", mixer, None)]
    if isinstance(m, ParallelConfig):
        a, r = m.left, m.right
        rope = None
        if a.rot_dims:
            # layers that rotate alike share the part, and with it a step's table of cosines and sines
            key = (a.dim, a.rot_dims, a.rot_base, a.rot_factor)
            if key not in ropes:
                scaling = RopeScaling("linear", a.rot_factor) if a.rot_factor is not None else None
                ropes[key] = POSITION_ENCODINGS.make("rope", head_dim=a.dim, theta=a.rot_base, scaling=scaling, interleaved=True,
                                                     rotary_dim=a.rot_dims)
            rope = ropes[key]
        left = MIXERS.make("attention", hidden_size=D, num_heads=a.heads, num_kv_heads=a.kv_heads, head_dim=a.dim, position=rope,
                           scale=a.scale, value_dim=a.vdim, names=("q", "k", "v", "o"), any_head_size=True, qkv_bias=True, o_bias=True,
                           accumulate=False, bias_to_caller=True)
        right = MIXERS.make("gated_delta_rule", hidden_size=D, num_heads=r.heads, num_kv_heads=r.kv_heads, key_dim=r.dim,
                            value_dim=r.vdim, conv_taps=r.conv, eps=eps, accumulate=False)
        rms = lambda: NORMS.make("rmsnorm", dim=D, eps=eps, tensor_name="")
        return [("mix.left.", left, ("mix.left.out", rms())), ("mix.right.", right, ("mix.right.out", rms()))]
    raise UnsupportedModelError(f"no mixer for {type(m).__name__}")


def _feed_forward(cfg: MuretarConfig, mlp):
    D = cfg.width
    if mlp.kind == "dense":
        return FEED_FORWARDS.make("swiglu", hidden_size=D, intermediate_size=mlp.ff, names=("gate", "up", "down"), accumulate=False)
    shared = None
    if mlp.shared_ff is not None:
        shared = ("shared.", FEED_FORWARDS.make("squared_relu_mlp", hidden_size=D, intermediate_size=mlp.shared_ff))
    return FEED_FORWARDS.make("routed_experts", hidden_size=D, expert_size=mlp.ff, num_experts=mlp.experts, top=mlp.top,
                              renormalize=True, renorm_eps=1e-20, activation="relu2", accumulate=False, identity=mlp.identity,
                              correction="correction", shared=shared)


def build_muretar(cfg: MuretarConfig) -> ModelSpec:
    D, eps = cfg.width, cfg.norm_eps
    norm = lambda: NORMS.make("layernorm", dim=D, eps=eps, tensor_name="")
    layers, place, ropes = [], {}, {}
    for i, layer in enumerate(cfg.layers):
        if layer.weights_of is not None:
            continue                      # no tensors of its own
        pre2 = post2 = ffn = None
        if layer.mlp is not None:
            pre2, post2, ffn = ("norm2", norm()), ("norm2b", norm()), ("mlp.", _feed_forward(cfg, layer.mlp))
        block = BLOCKS.make("sandwich", branches=_branches(cfg, layer.mixer, ropes), pre1=("norm1", norm()), post1=("norm1b", norm()),
                            pre2=pre2, post2=post2, ffn=ffn)
        place[i] = len(layers)
        layers.append((f"l{i}.", block))
    return ModelSpec(
        hidden_size=D, vocab_size=cfg.vocab, max_positions=cfg.max_positions,
        embedding=("", TokenEmbedding(cfg.vocab, D, tensor_name="embed")), layers=layers,
        run_order=[RunEntry(place[cfg.owner(i)]) for i in range(len(cfg.layers))],
        final_norm=("final.norm", norm()), head=("head", LMHead(cfg.vocab, D, tied=False, tensor_name="")),
    )


register_architecture("Muretar", MuretarConfig, build_muretar)
