"""Muretar on the GPU against the plain implementation (``plain_muretar``): each mechanism's kernels alone, with inputs made so
that a fault shows (a loud token far back, a write that must be recalled after hundreds of tokens, a routing choice that only
the correction makes), then whole models under every cutting, batching, page and slot reuse, long decoding, and greedy
generation through the engine's own entry point."""
import json
import math
import os
from types import SimpleNamespace

import numpy as np
import pytest
import torch

import plain_muretar as P
import tiny_muretar as TM
from gpu_tools import DEV, attention_ctx, cut_steps, live_token_need, run_trace
from tiny_models import random_tokens

pytestmark = pytest.mark.gpu
DTYPES = ["float32", "bfloat16"]
TORCH = {"float32": torch.float32, "bfloat16": torch.bfloat16}
F64 = torch.float64


def randn(*shape, seed=0, scale=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=F64) * scale


def close(got, ref, what, tol=2e-5):
    tol = tol * max(1.0, float(ref.abs().max()))
    err = float((got.double().cpu() - ref).abs().max())
    assert err <= tol, f"{what}: error {err:.3e} > {tol:.3e}"


def dev32(t):
    return t.float().to(DEV).contiguous()


def state_ctx(q_lens, slots):
    """The fields of a StepContext that the kernels of mixers with a state read."""
    q_start = np.zeros(len(q_lens) + 1, np.int32)
    np.cumsum(q_lens, out=q_start[1:])
    return SimpleNamespace(T=int(sum(q_lens)), R=len(q_lens), max_q_len=max(q_lens), q_lens=list(q_lens),
                           q_start=torch.from_numpy(q_start).to(DEV), slots=torch.tensor(slots, dtype=torch.int32, device=DEV))


def in_steps(seqs, cuts):
    """Steps over several sequences at once: ``cuts[name]`` are the portion sizes of sequence ``name`` (cycled); a step
    holds the next portion of every sequence that has tokens left.  Yields [(name, begin, end)]."""
    at = {n: 0 for n in seqs}
    k = 0
    while any(at[n] < seqs[n] for n in seqs):
        step = []
        for n in seqs:
            if at[n] < seqs[n]:
                size = min(cuts[n][k % len(cuts[n])], seqs[n] - at[n])
                step.append((n, at[n], at[n] + size))
                at[n] += size
        k += 1
        yield step


def paged(lengths, page, seed=0):
    """(block table [requests, width] on the device, pages in the pool): pages dealt out of order, three to spare."""
    blocks = [-(-n // page) for n in lengths]
    total = sum(blocks) + 3
    order = torch.randperm(total, generator=torch.Generator().manual_seed(seed)).tolist()
    table = torch.full((len(lengths), max(blocks)), -1, dtype=torch.int32)
    it = iter(order)
    for r, b in enumerate(blocks):
        for j in range(b):
            table[r, j] = next(it)
    return table.to(DEV), total


# ----------------------------------------------------------------------------- norms
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("D", [64, 100, 1030])
def test_layer_norm_with_bias_and_chosen_rows(dtype, D):
    from photon_infer_amd import ops
    x = randn(9, D, seed=1, scale=3.0) + 1.5
    w, b = randn(D, seed=2) * 0.3 + 1.0, randn(D, seed=3)
    want = P.layer_norm(x, w, b, 1e-5)
    tol = 3e-5 if dtype == "float32" else 2e-2
    out = torch.empty((9, D), dtype=TORCH[dtype], device=DEV)
    ops.layer_norm(out, dev32(x), dev32(w), dev32(b), 1e-5)
    close(out, want, "all rows", tol)
    rows = torch.tensor([7, 0, 3], dtype=torch.int32, device=DEV)
    out = torch.empty((3, D), dtype=TORCH[dtype], device=DEV)
    ops.layer_norm(out, dev32(x), dev32(w), dev32(b), 1e-5, rows)
    close(out, want[[7, 0, 3]], "chosen rows", tol)


def test_layer_norm_of_a_row_far_from_zero_keeps_its_digits():
    """A row at 1000 +- 1: the deviations are taken from the mean before they are squared."""
    from photon_infer_amd import ops
    x = randn(4, 256, seed=4) + 1000.0
    w, b = torch.ones(256, dtype=F64), torch.zeros(256, dtype=F64)
    out = torch.empty((4, 256), dtype=torch.float32, device=DEV)
    ops.layer_norm(out, dev32(x), dev32(w), dev32(b), 1e-6)
    close(out, P.layer_norm(x.float().double(), w, b, 1e-6), "offset rows", 2e-4)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("D", [64, 100, 520])
def test_a_result_joins_the_stream_through_a_norm_and_the_next_norm_is_made_on_the_way(dtype, D):
    from photon_infer_amd import ops
    T, eps = 7, 1e-5
    x, a, b = randn(T, D, seed=1, scale=2.0), randn(T, D, seed=2, scale=0.05), randn(T, D, seed=3, scale=5.0)
    a_bias = randn(D, seed=4, scale=0.1)
    wa, wb = randn(D, seed=5) * 0.2 + 1, randn(D, seed=6) * 0.2 + 1
    pw, pb, nw, nb = randn(D, seed=7) * 0.2 + 1, randn(D, seed=8), randn(D, seed=9) * 0.2 + 1, randn(D, seed=10)
    post, nxt = (dev32(pw), dev32(pb)), (dev32(nw), dev32(nb))
    cases = {"one result": a, "one result with a bias": a + a_bias,
             "two normalised results": 0.5 * (P.rms_norm(a + a_bias, wa, eps) + P.rms_norm(b, wb, eps)), "one normalised result": P.rms_norm(a, wa, eps)}
    for what, y in cases.items():
        want_x = x + P.layer_norm(y, pw, pb, eps)
        want_h = P.layer_norm(want_x, nw, nb, eps)
        xd = dev32(x)
        kw = {}
        if "bias" in what or "two" in what:
            kw["a_bias"] = dev32(a_bias)
        if "normalised" in what:
            kw["w_a"] = dev32(wa)
        if "two" in what:
            kw.update(b=dev32(b), w_b=dev32(wb))
        h = ops.sandwich_norm_add(xd, dev32(a), post, eps, nxt, TORCH[dtype], **kw)
        close(xd, want_x, f"{what}: stream")
        close(h, want_h, f"{what}: next input", 3e-5 if dtype == "float32" else 2e-2)
        xd = dev32(x)
        assert ops.sandwich_norm_add(xd, dev32(a), post, eps, **kw) is None
        close(xd, want_x, f"{what}: stream, nothing follows")


# ----------------------------------------------------------------------------- attention with two maps
def make_part(kind, tensors, tdt, **params):
    from photon_infer_amd.parts import MIXERS
    part = MIXERS.make(kind, **params)
    names = {s.name: s for s in part.tensor_specs()}
    assert set(names) == set(tensors), (sorted(names), sorted(tensors))
    part.load({n: t.to(tdt if t.dim() == 2 else torch.float32).to(DEV) for n, t in tensors.items()}, tdt, torch.device(DEV))
    return part


def run_paged_part(part, h, want, cuts_list, tdt, page, tol, what, D):
    """A mixer with pages as a part, on pages dealt out of order: under each cutting of the sequence its result must be the plain one."""
    from photon_infer_amd.parts import LayerCache
    T = h.shape[0]
    table, pages = paged([T], page, seed=2)
    spec = part.cache_spec()
    pools = {t.name: torch.zeros((pages, *t.page_shape(page)), dtype=tdt, device=DEV) for t in spec.tensors}
    cache = LayerCache(group=0, k=pools["k"], v=pools["v"], page_size=page, writes=True, tensors=pools)
    for cuts in cuts_list:
        for t in pools.values():
            t.fill_(50.0)                     # what a page held before must not show
        done = 0
        for n in cuts:
            ctx = attention_ctx([n], [done + n], tdt)
            ctx.block_tables, ctx.may_defer = {0: table}, False
            x = torch.full((n, D), 3.0, dtype=torch.float32, device=DEV)          # the part writes its result, it does not add
            part.forward(h[done:done + n].to(tdt).to(DEV).contiguous(), x, ctx, cache)
            close(x, want[done:done + n], f"{what} tokens {done} .. {done + n} of cuts {cuts[:4]}", tol)
            done += n


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("sizes", [(4, 2, 16, 24), (4, 1, 64, 64), (6, 3, 12, 10), (1, 1, 48, 48), (2, 2, 32, 64), (8, 2, 128, 128), (2, 1, 16, 48),
                                   (4, 2, 64, 128), (2, 1, 128, 384)])
def test_differential_attention_whole_in_portions_and_token_by_token(dtype, sizes):
    """One token far back is loud; the second map's vectors make a lambda far from ``diff``.  Values two and three times as
    wide as keys are attended in pieces by the bfloat16 engine."""
    H, G, d, dv = sizes
    D, T, page, eps, scale, diff = 72, 150, 16, 1e-5, 0.11, 0.35
    tdt = TORCH[dtype]
    rnd = lambda *s, seed, scale=0.2: randn(*s, seed=seed, scale=scale).to(torch.bfloat16).double()
    W = {"q": rnd(H * 2 * d, D, seed=1), "k": rnd(G * 2 * d, D, seed=2), "v": rnd(G * dv, D, seed=3), "o": rnd(D, H * dv, seed=4),
         "q.b": rnd(H * 2 * d, seed=5), "k.b": rnd(G * 2 * d, seed=6), "v.b": rnd(G * dv, seed=7),
         "lq1": rnd(d, seed=8, scale=0.4), "lk1": rnd(d, seed=9, scale=0.4), "lq2": rnd(d, seed=10, scale=0.4), "lk2": rnd(d, seed=11, scale=0.4)}
    h = randn(T, D, seed=12).to(tdt).double()
    h[5] *= 4.0
    m = {"heads": H, "kv_heads": G, "dim": d, "vdim": dv, "diff": diff, "scale": scale}
    want = P.differential_attention(h, m, W, "", eps, P.bf16_round if dtype == "bfloat16" else None)
    lam = math.exp(float(W["lq1"] @ W["lk1"])) - math.exp(float(W["lq2"] @ W["lk2"])) + diff
    assert abs(lam - diff) > 0.01
    part = make_part("differential_attention", W, tdt, hidden_size=D, num_heads=H, num_kv_heads=G, head_dim=d, value_dim=dv, scale=scale, diff=diff,
                     eps=eps, accumulate=False)
    assert abs(part.lam - lam) < 1e-12
    assert part.split == (dv // d if dtype == "bfloat16" and d % 16 == 0 and dv % d == 0 else 1)
    run_paged_part(part, h, want, ([T], [64, 7, 2, 77], [T - 12] + [1] * 12), tdt, page, 1e-4 if dtype == "float32" else 5e-2, f"{sizes}", D)


def test_the_two_maps_are_told_apart_and_share_their_values():
    """Map 1 of every head looks at the first token only, map 2 at the token itself: o = v_0 - lam v_t, whatever the head."""
    from photon_infer_amd import ops
    H, G, d, dv, T, page = 4, 2, 16, 8, 40, 16
    v = randn(T, G, dv, seed=1)
    q = torch.zeros(T, H, 2, d, dtype=F64)
    k = torch.zeros(T, G, 2, d, dtype=F64)
    q[:, :, 0, 0], q[:, :, 1, 1] = 1.0, 1.0
    k[0, :, 0, 0] = 60.0                                         # map 1: the first token's key is loud
    k[:, :, 1, 1] = torch.arange(T, dtype=F64)[:, None] * 60.0   # map 2: every later key is louder than all before it
    per = H // G
    regroup = lambda t: t.reshape(T, G, per, 2, -1).transpose(2, 3).reshape(T, -1)
    proj = torch.cat([regroup(q), k.reshape(T, -1), v[:, :, None, :].expand(T, G, 2, dv).reshape(T, -1)], dim=1)
    table, pages = paged([T], page, seed=3)
    kc = torch.zeros((pages, 2 * G, page, d), device=DEV)
    vc = torch.zeros((pages, 2 * G, dv, page), device=DEV)
    ctx = attention_ctx([T], [T], torch.float32)
    qd = torch.empty((T, 2 * H * d), device=DEV)
    pieces = ops.Partials(dev32(proj).view(1, T, -1), 1, T, proj.shape[1])
    ops.rope_kv_write(qd, None, None, ctx.positions, ctx.req_of_token, None, 2 * H, 2 * G, d, kc, vc, table, page, pieces=pieces, write_kv=True,
                      value_dim=dv, bias=torch.zeros(proj.shape[1], device=DEV))
    attn = torch.empty((T, 2 * H * dv), device=DEV)
    ops.paged_attention(attn, qd, kc, vc, table, ctx, 2 * H, 2 * G, d, page, 1.0, 0, None, value_dim=dv)
    out = torch.empty((T, H * dv), device=DEV)
    lam = 0.7
    ops.diff_combine(out, attn, lam, 0.0, 1.0, H, G, dv)
    for n in range(H):
        o = v[0, n // per] - lam * v[1:, n // per]
        close(out[1:, n * dv:(n + 1) * dv], o / torch.sqrt((o * o).mean(-1, keepdim=True)), f"head {n}", 1e-4)


# ----------------------------------------------------------------------------- attention with biases beside it
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("sizes", [(4, 2, 16, 32, 8, 3.0), (4, 1, 64, 64, 64, None), (6, 3, 24, 12, 0, None), (1, 1, 32, 32, 16, 1.0), (8, 1, 64, 48, 64, 2.0),
                                   (2, 2, 128, 128, 128, 4.0)])
def test_attention_with_biases_part_rotation_and_divided_frequencies(dtype, sizes):
    from photon_infer_amd.config.llama import RopeScaling
    from photon_infer_amd.parts import POSITION_ENCODINGS
    H, G, d, dv, rd, factor = sizes
    D, T, page, scale, base = 72, 150, 16, 0.13, 300.0
    tdt = TORCH[dtype]
    rnd = lambda *s, seed, scale=0.2: randn(*s, seed=seed, scale=scale).to(torch.bfloat16).double()
    W = {"q": rnd(H * d, D, seed=1), "k": rnd(G * d, D, seed=2), "v": rnd(G * dv, D, seed=3), "o": rnd(D, H * dv, seed=4),
         "q.b": rnd(H * d, seed=5, scale=0.5), "k.b": rnd(G * d, seed=6, scale=0.5), "v.b": rnd(G * dv, seed=7, scale=0.5), "o.b": rnd(D, seed=8, scale=0.5)}
    h = randn(T, D, seed=12).to(tdt).double()
    h[5] *= 4.0
    m = {"heads": H, "kv_heads": G, "dim": d, "vdim": dv, "scale": scale}
    if rd:
        m["rot"] = {"base": base, "dims": rd}
        if factor is not None:
            m["rot"]["scaling"] = {"factor": factor}
    want = P.rotary_attention(h, m, W, "", P.bf16_round if dtype == "bfloat16" else None)
    rope = None
    if rd:
        rope = POSITION_ENCODINGS.make("rope", head_dim=d, theta=base, interleaved=True, rotary_dim=rd,
                                       scaling=RopeScaling("linear", factor) if factor is not None else None)
        rope.load({}, tdt, torch.device(DEV))
    part = make_part("attention", W, tdt, hidden_size=D, num_heads=H, num_kv_heads=G, head_dim=d, position=rope, scale=scale, value_dim=dv,
                     names=("q", "k", "v", "o"), any_head_size=True, qkv_bias=True, o_bias=True, accumulate=False)
    run_paged_part(part, h, want, ([T], [64, 7, 2, 77], [T - 12] + [1] * 12), tdt, page, 1e-4 if dtype == "float32" else 5e-2, f"{sizes}", D)


# ----------------------------------------------------------------------------- walks over a state
def walk(kind, data, T, slot, cuts, sizes, consts):
    """Run ``ops.delta_scan`` of ``kind`` over the sequences of ``data`` in the steps that ``cuts`` give; {name: outputs}, states."""
    from photon_infer_amd import ops
    H, G, d, dv = sizes
    floats = ops.scan_state_floats(H, d, dv)
    state = torch.zeros((4, floats + 3), device=DEV)
    got = {n: [] for n in T}
    for step in in_steps(T, cuts):
        qkv = dev32(torch.cat([data[n][0][i:j] for n, i, j in step]))
        a = dev32(torch.cat([data[n][1][i:j] for n, i, j in step]))
        ctx = state_ctx([j - i for _, i, j in step], [slot[n] for n, _, _ in step])
        o = torch.empty((qkv.shape[0], H * dv), device=DEV)
        if kind == "head_delta":
            b = dev32(torch.cat([data[n][2][i:j] for n, i, j in step]))
            ops.delta_scan(o, qkv, a, dev32(consts["dt_bias"]), dev32(consts["A_log"]), b, ctx, state[:, :floats], H, G, d, dv, d ** -0.5, 1e-6,
                           kind="head_delta")
        else:
            ops.delta_scan(o, qkv, a, dev32(consts["a_bias"]), None, None, ctx, state[:, :floats], H, G, d, dv, d ** -0.5, 0.0,
                           kind="decayed_outer", tau=consts["tau"])
        for (n, i, j), part in zip(step, torch.split(o, [j - i for _, i, j in step])):
            got[n].append(part)
    return {n: torch.cat(p) for n, p in got.items()}, state


CUTS = ({"a": [83], "b": [10]}, {"a": [1], "b": [1]}, {"a": [2, 17, 1, 40], "b": [3, 2]}, {"a": [9], "b": [10]})


@pytest.mark.parametrize("sizes", [(4, 2, 16, 24), (4, 4, 32, 32), (3, 1, 20, 28), (1, 1, 48, 80), (5, 5, 8, 8), (2, 1, 128, 64), (2, 2, 3, 200)])
def test_delta_rule_with_a_decay_per_head_whole_in_portions_and_token_by_token(sizes):
    H, G, d, dv = sizes
    T = {"a": 83, "b": 10}
    consts = {"A_log": randn(H, seed=1, scale=0.5) - 1.0, "dt_bias": randn(H, seed=2, scale=0.5)}
    data, want = {}, {}
    for i, (n, t) in enumerate(T.items()):
        q, k, v = randn(t, G, d, seed=10 + i), randn(t, G, d, seed=20 + i), randn(t, H, dv, seed=30 + i)
        a, b = randn(t, H, seed=40 + i), randn(t, H, seed=50 + i)
        data[n] = (torch.cat([q.reshape(t, -1), k.reshape(t, -1), v.reshape(t, -1)], dim=1), a, b)
        qu = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * d ** -0.5
        ku = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
        decay = torch.exp(-torch.exp(consts["A_log"]) * P.softplus(a + consts["dt_bias"]))
        want[n] = torch.stack([P.delta_rule_walk(qu[:, h // (H // G)], ku[:, h // (H // G)], v[:, h], P.sigmoid(b[:, h]), decay[:, h]) for h in range(H)], 1)
    slot = {"a": 3, "b": 1}
    for cuts in CUTS:
        got, state = walk("head_delta", data, T, slot, cuts, sizes, consts)
        for n in T:
            close(got[n], want[n].reshape(T[n], -1), f"{sizes} {n} cut {cuts[n]}", 5e-5)
        assert bool((state[0] == 0).all()) and bool((state[2] == 0).all())


@pytest.mark.parametrize("sizes", [(2, 24, 16, 8.0), (4, 32, 64, 16.0), (3, 20, 28, 3.5), (1, 40, 40, 1.0), (2, 128, 64, 2.0), (2, 3, 200, 5.0)])
def test_gated_linear_attention_walk_whole_in_portions_and_token_by_token(sizes):
    H, d, dv, tau = sizes
    T = {"a": 83, "b": 10}
    consts = {"a_bias": randn(H * d, seed=2), "tau": tau}
    data, want = {}, {}
    for i, (n, t) in enumerate(T.items()):
        q, k, v, z = randn(t, H, d, seed=10 + i), randn(t, H, d, seed=20 + i), randn(t, H, dv, seed=30 + i), randn(t, H, d, seed=40 + i, scale=2.0)
        data[n] = (torch.cat([q.reshape(t, -1), k.reshape(t, -1), v.reshape(t, -1)], dim=1), z.reshape(t, -1))
        alpha = P.sigmoid(z + consts["a_bias"].view(H, d)) ** (1.0 / tau)
        want[n] = torch.stack([P.decayed_outer_walk(q[:, h] * d ** -0.5, k[:, h], v[:, h], alpha[:, h]) for h in range(H)], 1)
    slot = {"a": 0, "b": 2}
    for cuts in CUTS:
        got, state = walk("decayed_outer", data, T, slot, cuts, (H, H, d, dv), consts)
        for n in T:
            close(got[n], want[n].reshape(T[n], -1), f"{sizes} {n} cut {cuts[n]}", 5e-5)
        assert bool((state[1] == 0).all()) and bool((state[3] == 0).all())


@pytest.mark.parametrize("sizes", [(2, 24, 16, 8.0), (3, 20, 28, 3.5), (2, 128, 64, 2.0), (1, 40, 200, 1.0)])
def test_long_portions_of_the_linear_walk_beside_short_ones(sizes):
    """Portions of hundreds of tokens (many chunks of the walk) beside single tokens and a short portion; the state a portion
    leaves is the one the next step starts from, whatever the cutting."""
    from photon_infer_amd import ops
    H, d, dv, tau = sizes
    T = {"a": 700, "b": 300, "c": 9}
    consts = {"a_bias": randn(H * d, seed=2), "tau": tau}
    data, want = {}, {}
    for i, (n, t) in enumerate(T.items()):
        q, k, v, z = randn(t, H, d, seed=10 + i), randn(t, H, d, seed=20 + i), randn(t, H, dv, seed=30 + i), randn(t, H, d, seed=40 + i, scale=2.0) + 3.0
        data[n] = (torch.cat([q.reshape(t, -1), k.reshape(t, -1), v.reshape(t, -1)], dim=1), z.reshape(t, -1))
        alpha = P.sigmoid(z + consts["a_bias"].view(H, d)) ** (1.0 / tau)
        want[n] = torch.stack([P.decayed_outer_walk(q[:, h] * d ** -0.5, k[:, h], v[:, h], alpha[:, h]) for h in range(H)], 1)
    slot = {"a": 0, "b": 2, "c": 3}
    for cuts in ({"a": [700], "b": [300], "c": [9]}, {"a": [256, 1, 300, 143], "b": [1, 299], "c": [1]}, {"a": [129, 571], "b": [44, 256], "c": [3]}):
        got, state = walk("decayed_outer", data, T, slot, cuts, (H, H, d, dv), consts)
        for n in T:
            close(got[n], want[n].reshape(T[n], -1), f"{sizes} {n} cut {cuts[n]}", 1e-4)
        assert bool((state[1] == 0).all())


@pytest.mark.parametrize("decode", [False, True])
def test_a_write_is_recalled_after_hundreds_of_tokens_and_fades_by_its_channel_alone(decode):
    """Token 3 writes v into key channel 0 (which does not decay) and into channel 1 (which halves every token); 600 tokens
    later channel 0 still holds it whole and channel 1 nothing; the tokens between write nothing."""
    from photon_infer_amd import ops
    H, d, dv, T, tau = 1, 16, 16, 604, 4.0
    q, k, v = torch.zeros(T, d, dtype=F64), torch.zeros(T, d, dtype=F64), randn(T, dv, seed=1)
    k[3, 0], k[3, 1] = 2.0, 2.0
    z = torch.full((T, d), -3.0, dtype=F64)
    z[:, 0] = 40.0                                              # sigmoid = 1
    z[:, 1] = math.log(1.0 / (2.0 ** tau - 1.0))                # sigmoid^(1 / tau) = 1 / 2
    q[:, 0], q[T - 1, 1] = 4.0, 4.0                             # times d^-1/2 = 1
    qkv = torch.cat([q, k, v], dim=1)
    cuts = [T] if not decode else [4, 300] + [1] * 300
    state = torch.zeros((2, ops.scan_state_floats(H, d, dv)), device=DEV)
    outs, done = [], 0
    for n in cuts:
        o = torch.empty((n, dv), device=DEV)
        ops.delta_scan(o, dev32(qkv[done:done + n]), dev32(z[done:done + n]), torch.zeros(d, device=DEV), None, None, state_ctx([n], [1]), state, H, H, d, dv,
                       d ** -0.5, 0.0, kind="decayed_outer", tau=tau)
        outs.append(o)
        done += n
    out = torch.cat(outs).double().cpu()
    assert float(out[:3].abs().max()) == 0.0
    close(out[3], 2.0 * v[3], "the token itself")
    close(out[4], 2.0 * v[3], "one token later: channel 0 alone is read")
    close(out[T - 2], 2.0 * v[3], "599 tokens later")
    close(out[T - 1], 2.0 * v[3] * (1.0 + 0.5 ** 600), "600 tokens later, both channels read")


def test_head_norm_with_a_silu_gate():
    from photon_infer_amd import ops
    T, H, dv = 5, 3, 20
    o, g, w = randn(T, H, dv, seed=1, scale=3.0), randn(T, H, dv, seed=2, scale=2.0), randn(dv, seed=3) * 0.2 + 1.0
    want = (P.rms_norm(o, w, 1e-5) * P.silu(g)).reshape(T, -1)
    for dtype in DTYPES:
        y = torch.empty((T, H * dv), dtype=TORCH[dtype], device=DEV)
        ops.head_norm_gate(y, dev32(o.reshape(T, -1)), dev32(g.reshape(T, -1)), dev32(w.repeat(H)), 1e-5, H, dv, gate="silu")
        close(y, want, dtype, 3e-5 if dtype == "float32" else 2e-2)


# ----------------------------------------------------------------------------- routed experts
def test_routing_with_a_correction_and_renormalised_weights():
    from photon_infer_amd import ops
    T, E, top = 200, 11, 4
    z, corr = randn(T, E, seed=1, scale=1.5), randn(E, seed=2, scale=0.1)
    ids, w = ops.route(dev32(z), top, 1, 1, True, dev32(corr), 1e-20)
    plain_ids, w0 = ops.route(dev32(z), top, 1, 1, True)
    changed = 0
    for t in range(T):
        order, weights = P.route(z[t].float().double(), corr.float().double(), top)
        assert ids[t].tolist() == order, t
        close(w[t], weights, f"weights of token {t}", 1e-5)
        changed += ids[t].tolist() != plain_ids[t].tolist()
    assert changed > 20                                          # the correction decides many choices


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("sizes", [(5, 2, 3, 40, 56), (8, 0, 4, 128, 64), (9, 3, 1, 36, None), (1, 3, 4, 48, None), (3, 1, 2, 32, 16)])
@pytest.mark.parametrize("T", [1, 9, 150])
def test_routed_experts_with_identities_and_a_shared_expert(dtype, sizes, T):
    from photon_infer_amd import ops
    from photon_infer_amd.parts import FEED_FORWARDS
    E, ident, top, F, shared = sizes
    D = 64
    tdt = TORCH[dtype]
    rnd = lambda *s, seed, scale=0.2: randn(*s, seed=seed, scale=scale).to(torch.bfloat16).double()
    W = {"router": rnd(E + ident, D, seed=1, scale=0.5), "correction": rnd(E + ident, seed=2, scale=0.1)}
    for e in range(E):
        W[f"e{e}.up"], W[f"e{e}.down"] = rnd(F, D, seed=10 + e), rnd(D, F, seed=40 + e)
    mlp = {"router": {"experts": E, "identity": ident, "top": top}, "expert": {"ff": F}}
    part_shared = None
    if shared:
        W["shared.up"], W["shared.down"] = rnd(shared, D, seed=80), rnd(D, shared, seed=81)
        mlp["shared"] = {"ff": shared}
        part_shared = ("shared.", FEED_FORWARDS.make("squared_relu_mlp", hidden_size=D, intermediate_size=shared))
    part = FEED_FORWARDS.make("routed_experts", hidden_size=D, expert_size=F, num_experts=E, top=top, renormalize=True, renorm_eps=1e-20,
                              activation="relu2", accumulate=False, identity=ident, correction="correction", shared=part_shared)
    assert {s.name for s in part.tensor_specs()} == set(W)
    part.load({n: t.to(tdt if t.dim() == 2 else torch.float32).to(DEV) for n, t in W.items()}, tdt, torch.device(DEV))
    h = randn(T, D, seed=3).to(tdt).double()
    seen = []
    real = ops.route
    ops.route = lambda *a, **k: (seen.append(real(*a, **k)), seen[-1])[1]
    try:
        out = torch.full((T, D), 7.0, device=DEV)
        part.forward(h.to(tdt).to(DEV), out, SimpleNamespace(workspace=None, may_defer=False))
    finally:
        ops.route = real
    ids = seen[0][0].cpu()
    if ident:
        assert int((ids >= E).sum()) > 0 or T == 1
    margins, chosen = [], []
    P.routed_experts(h, mlp, W, "", margins=margins, chosen=chosen)
    for t in range(T):
        if sorted(ids[t].tolist()) != sorted(chosen[t]):
            assert dtype == "bfloat16" and margins[t] < 0.01, (t, ids[t].tolist(), chosen[t], margins[t])
    want = P.routed_experts(h, mlp, W, "", P.bf16_round if dtype == "bfloat16" else None, choices=[r.tolist() for r in ids])
    close(out, want, f"{sizes} {T} tokens", 3e-5 if dtype == "float32" else 3e-2)


@pytest.mark.parametrize("M,N,K", [(5, 96, 128), (200, 96, 128), (129, 520, 320), (300, 40, 64)])
def test_product_and_squared_relu(M, N, K):
    """Few rows: the product's float32 result through the activation's kernel; many rows in bfloat16: the tile product's epilogue."""
    from photon_infer_amd import ops
    a, w = randn(M, K, seed=1).to(torch.bfloat16), randn(N, K, seed=2, scale=0.1).to(torch.bfloat16)
    want = torch.clamp(a.double() @ w.double().T, min=0.0) ** 2
    for dtype in DTYPES:
        tdt = TORCH[dtype]
        out = torch.empty((M, N), dtype=tdt, device=DEV)
        ops.gemm_relu_squared(out, a.to(tdt).to(DEV), w.to(tdt).to(DEV))
        close(out, want, f"{dtype} {M} x {N} x {K}", 3e-5 if dtype == "float32" else 1e-2)


# ----------------------------------------------------------------------------- whole models
@pytest.fixture(scope="module")
def model_dirs(tmp_path_factory):
    root = tmp_path_factory.mktemp("muretar")
    return {name: TM.make_model_dir(root, name, seed=5, ranks_in_config=(name != "C")) for name in TM.ALL}


_plain = {}
CLOSE_CALL = 0.01      # choice scores (a share of 1 among the experts): a bfloat16 choice that differs from the plain one must be this close to a tie


class RouteRecorder:
    """Records the experts the engine chooses (every call of ``ops.route``, in order), so that the plain implementation can be
    asked for the logits of the same choices: among hundreds of routing decisions some are near ties, which bfloat16 rounding
    decides either way, and one flipped expert changes everything after it."""

    def __enter__(self):
        from photon_infer_amd import ops
        self.ops, self.real, self.calls = ops, ops.route, []

        def route(*a, **k):
            ids, w = self.real(*a, **k)
            self.calls.append(ids.cpu())
            return ids, w
        ops.route = route
        return self

    def __exit__(self, *exc):
        self.ops.route = self.real

    def by_request(self, steps, config):
        """{request: {routed layer: [tokens, top] expert ids}} from the calls, given the trace's steps."""
        layers = [i for i, l in enumerate(config["layers"]) if l["mlp"] and l["mlp"]["kind"] == "moe"]
        out, k = {}, 0
        for s in steps:
            sizes = [len(e["tokens"]) for e in s["entries"]]
            for i in layers:
                for e, part in zip(s["entries"], torch.split(self.calls[k], sizes)):
                    out.setdefault(e["id"], {}).setdefault(i, []).append(part)
                k += 1
        assert k == len(self.calls)
        return {rid: {i: [r.tolist() for r in torch.cat(p)] for i, p in per.items()} for rid, per in out.items()}


def plain_logits(model_dir, tokens, emulate=False, forced=None):
    key = (model_dir, tuple(tokens), emulate)
    if forced is not None or key not in _plain:
        cfg, W = P.read_model_folder(model_dir)
        out = P.forward(cfg, W, list(tokens), P.bf16_round if emulate else None, choices=forced).float()
        if forced is not None:
            return out
        _plain[key] = out
    return _plain[key]


def runner_for(model_dir, name, dtype, max_tokens):
    from photon_infer_amd.engine.replay import make_runner
    return make_runner(model_dir, dtype, max(max_tokens, 64), TM.ALL[name][1]["block_size"])


def check_choices(model_dir, toks, forced, what):
    """The engine's experts are those of the plain implementation with activations rounded where a 16-bit engine rounds them
    (a sublayer's result is normalised before it joins the stream, which can blow a rounding up to a tenth of the stream at a
    token; the unrounded router then sees another input), or differ only where that router was within a whisker of choosing
    otherwise."""
    cfg, W = P.read_model_folder(model_dir)
    margins, chosen = {}, {}
    P.forward(cfg, W, list(toks), P.bf16_round, choices=forced, margins=margins, chosen=chosen)
    for i, ids in forced.items():
        for t in range(len(toks)):
            if sorted(ids[t]) != sorted(chosen[i][t]):
                assert margins[i][t] < CLOSE_CALL, f"{what}: layer {i} token {t}: experts {ids[t]} instead of {chosen[i][t]} (margin {margins[i][t]:.4f})"


def check(got, model_dir, reqs, dtype, what, choices=None):
    """``choices`` (bfloat16 runs): the experts the engine chose per request; the plain logits are then those of the same
    choices, which must be the plain ones up to close calls."""
    assert got, "no logits came back"
    for rid, toks in reqs.items():
        forced = choices.get(rid) if choices else None
        if forced:
            check_choices(model_dir, toks, forced, what)
        ref = plain_logits(model_dir, toks, forced=forced)
        if dtype == "float32":
            tol = 1e-4 * max(1.0, float(ref.abs().max()))
        else:       # three times what rounding activations to bfloat16 does to the plain implementation itself
            tol = 3.0 * float((plain_logits(model_dir, toks, True, forced=forced) - ref).abs().max())
        over = []
        for p in range(len(toks)):
            assert (rid, p) in got, f"{what}: logits of {rid} position {p} are missing"
            err = float((got[(rid, p)] - ref[p]).abs().max())
            if dtype == "float32" or err > 3.0 * tol:
                assert err <= tol, f"{what}: {rid} position {p}: error {err:.3e} > {tol:.3e} (first wrong position)"
            elif err > tol:
                over.append(p)
        # bfloat16: a sublayer's result is normalised before it is added, so where a result happens to be small rounding noise is
        # blown up to full size at that one position; such positions are rare, stay within three times the bound, and leave their
        # neighbours alone - a fault of cache, state or batch does none of the three
        assert len(over) <= max(1, len(toks) // 50), f"{what}: {rid}: positions {over} are over {tol:.3e}"


def run_checked(runner, steps, out_dir, model_dir, reqs, dtype, what):
    """Replay ``steps`` and compare; in bfloat16 the plain implementation follows the engine's routing choices."""
    if dtype == "float32":
        return check(run_trace(runner, steps, out_dir), model_dir, reqs, dtype, what)
    with RouteRecorder() as rec:
        got = run_trace(runner, steps, out_dir)
    check(got, model_dir, reqs, dtype, what, rec.by_request(steps, P.read_model_folder(model_dir)[0]))


LENGTHS = {"A": [1, 26, 90], "B": [3, 130, 210], "C": [2, 30, 75], "D": [2, 45, 100]}


def requests_for(name, seed=0):
    vocab = TM.ALL[name][0]["vocab"]
    return {f"r{i}": random_tokens(n, vocab, seed * 100 + i) for i, n in enumerate(LENGTHS[name])}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(TM.ALL))
def test_whole_prompts_and_the_stream_after_every_layer(name, dtype, model_dirs, tmp_path):
    reqs = requests_for(name)
    steps = []
    for rid, toks in reqs.items():
        steps += cut_steps(rid, toks, [len(toks)], first_step=len(steps))
    runner = runner_for(model_dirs[name], name, dtype, live_token_need(steps))
    run_checked(runner, steps, str(tmp_path), model_dirs[name], reqs, dtype, "whole")
    if dtype == "float32":         # the stream after every layer (a layer that runs another's tensors counts for itself), for the longest request
        from photon_infer_amd.engine.step import StepEntry
        toks = reqs["r2"]
        cfg, W = P.read_model_folder(model_dirs[name])
        want, got = [], []
        P.forward(cfg, W, toks, streams=want)
        for blk in set(runner.model.blocks):
            def wrapped(x, ctx, cache, f=blk.forward):
                f(x, ctx, cache)
                got.append(x.detach().double().cpu())
            blk.forward = wrapped
        runner.admit("s")
        runner.step([StepEntry("s", toks, [])])
        assert len(got) == len(want) == len(cfg["layers"])
        for i, (g, w) in enumerate(zip(got, want)):
            close(g, w, f"stream after layer {i}", 1e-4)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(TM.ALL))
def test_prefill_then_token_by_token_and_all_token_by_token(name, dtype, model_dirs, tmp_path):
    reqs = requests_for(name, seed=1)
    steps = []
    for rid, toks in reqs.items():
        head = max(0, len(toks) - 40)
        sizes = ([head] if head else []) + [1] * (len(toks) - head)
        steps += cut_steps(rid, toks, sizes, first_step=len(steps))
    steps += cut_steps("all", reqs["r1"], [1], first_step=len(steps))
    runner = runner_for(model_dirs[name], name, dtype, live_token_need(steps))
    run_checked(runner, steps, str(tmp_path), model_dirs[name], dict(reqs, all=reqs["r1"]), dtype, "decoding")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(TM.ALL))
@pytest.mark.parametrize("sizes", [[2], [7, 2, 31, 1, 3], [64, 5], [17]])
def test_portions_of_changing_size(name, dtype, sizes, model_dirs, tmp_path):
    reqs = {"r2": requests_for(name, seed=2)["r2"]}
    steps = cut_steps("r2", reqs["r2"], sizes)
    runner = runner_for(model_dirs[name], name, dtype, live_token_need(steps))
    run_checked(runner, steps, str(tmp_path), model_dirs[name], reqs, dtype, f"portions {sizes}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(TM.ALL))
def test_mixed_batches_with_pages_and_slots_used_again(name, dtype, model_dirs, tmp_path):
    """Seven unequal requests through four slots: portions of some beside single tokens of others; a request may sit out a
    step; a finished request's pages and slot go to the next one.  Each must come out as it does alone."""
    vocab = TM.ALL[name][0]["vocab"]
    lengths = [70, 33, 5, 120, 64, 18, 91]
    reqs = {f"m{i}": random_tokens(n, vocab, 50 + i) for i, n in enumerate(lengths)}
    rng = np.random.default_rng(7)
    waiting, live, at, steps = list(reqs), [], {}, []
    while waiting or live:
        while waiting and len(live) < 4:
            live.append(waiting.pop(0))
            at[live[-1]] = 0
        entries, end = [], []
        for rid in list(live):
            left = len(reqs[rid]) - at[rid]
            if len(live) > 1 and rng.random() < 0.2:
                continue                               # sits this step out
            n = 1 if left <= 12 else int(min(left - 12, rng.choice([2, 3, 16, 29, 40])))
            entries.append({"id": rid, "tokens": reqs[rid][at[rid]:at[rid] + n], "want": list(range(n))})
            at[rid] += n
            if at[rid] == len(reqs[rid]):
                end.append(rid)
                live.remove(rid)
        if entries:
            steps.append({"step": len(steps), "entries": entries, "end": end})
    runner = runner_for(model_dirs[name], name, dtype, live_token_need(steps))
    assert runner.cache.max_slots == 4
    run_checked(runner, steps, str(tmp_path), model_dirs[name], reqs, dtype, "mixed")
    assert all(g.pool.num_allocated == 0 for g in runner.cache.groups)


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_long_prompt_whole_and_in_two_long_portions(dtype, model_dirs, tmp_path):
    """600 tokens whole, and in two long portions and a single token."""
    vocab = TM.ALL["A"][0]["vocab"]
    reqs = {"w": random_tokens(600, vocab, 11), "p": random_tokens(600, vocab, 11)}
    steps = cut_steps("w", reqs["w"], [600])
    steps += cut_steps("p", reqs["p"], [301, 298, 1], first_step=len(steps))
    runner = runner_for(model_dirs["A"], "A", dtype, live_token_need(steps))
    run_checked(runner, steps, str(tmp_path), model_dirs["A"], reqs, dtype, "long prompt")


@pytest.mark.parametrize("name", ["A", "C"])
def test_long_decoding_keeps_its_state(name, model_dirs, tmp_path):
    """250 tokens one by one after a portion of three: the states and pages carry everything from step to step."""
    vocab = TM.ALL[name][0]["vocab"]
    toks = random_tokens(250, vocab, 9)
    steps = cut_steps("long", toks, [3] + [1] * 247)
    runner = runner_for(model_dirs[name], name, "float32", 256)
    run_checked(runner, steps, str(tmp_path), model_dirs[name], {"long": toks}, "float32", "long decoding")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(TM.ALL))
def test_greedy_generation_through_the_engine(name, dtype, model_dirs):
    """The engine's own entry point, scheduler, sampling and decode steps: unequal prompts at once, more requests than slots,
    prompts longer than a portion; every request must generate what the plain implementation generates alone."""
    from photon_infer_amd.engine import ContinuousBatchEngine, EngineOptions
    cfg, W = P.read_model_folder(model_dirs[name])
    vocab = cfg["vocab"]
    prompts = [random_tokens(n, vocab, 70 + i) for i, n in enumerate([5, 41, 18, 70, 2])]
    engine = ContinuousBatchEngine(model_dirs[name], EngineOptions(dtype=dtype, block_size=TM.ALL[name][1]["block_size"], max_batch=3,
                                                                   max_cache_tokens=1024, chunk_size=32, max_model_len=200))
    got = engine.generate(prompts, max_new_tokens=10)
    for prompt, out in zip(prompts, got):
        want = P.greedy(cfg, W, prompt, 10)
        if dtype == "float32":
            assert list(out) == want
        else:       # bfloat16: a near tie may fall the other way; everything before the first difference must agree and the
            # differing token must be a close second of the plain logits: within twice the bound that the logits themselves
            # are held to (three times what rounding activations does to the plain implementation at that position)
            for i, (a, b) in enumerate(zip(out, want)):
                if a != b:
                    lg = P.forward(cfg, W, prompt + want[:i])[-1]
                    tol = 3.0 * float((P.forward(cfg, W, prompt + want[:i], P.bf16_round)[-1] - lg).abs().max())
                    assert float(lg[b] - lg[a]) <= 2.0 * tol, f"token {i}: {a} instead of {b} ({float(lg[b] - lg[a]):.3f} apart, bound {tol:.3f})"
                    break


def test_command_line_and_replayed_decode_steps(model_dirs, tmp_path):
    """The framework's commands serve the design as they serve its others (from a folder, and from a bare configuration with
    random weights); and decode steps replayed as HIP graphs give the tokens of eager steps, with new requests' prompts in
    between and states in slots that are used again."""
    import subprocess
    from photon_infer_amd.engine import ContinuousBatchEngine, EngineOptions
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    cfg, W = P.read_model_folder(model_dirs["A"])
    prompt = random_tokens(9, cfg["vocab"], 81)
    want = P.greedy(cfg, W, prompt, 5)
    proc = subprocess.run([os.path.join(root, "bin", "llama_infer"), model_dirs["A"], "--dtype", "fp32", "--prompt-ids",
                           ",".join(map(str, prompt)), "--max-new-tokens", "5", "--temperature", "0", "--ignore-eos"],
                          capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert "Architecture: Muretar" in proc.stdout and f"Generated ids: {','.join(map(str, want))}" in proc.stdout
    (tmp_path / "cfg").mkdir()
    json.dump(TM.TINY_D, open(tmp_path / "cfg" / "config.json", "w"))
    proc = subprocess.run([os.path.join(root, "bin", "llama_infer"), str(tmp_path / "cfg"), "--random-weights", "--seed", "3",
                           "--prompt-ids", "5,6,7", "--max-new-tokens", "4", "--ignore-eos"], capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert "Generated ids:" in proc.stdout
    # the trace replay as a command, from the folder (whose configuration leaves a size to the tensors)
    cfgc, _ = P.read_model_folder(model_dirs["C"])
    toks = random_tokens(12, cfgc["vocab"], 82)
    lines = "\n".join(json.dumps(s) for s in cut_steps("x", toks, [5, 1, 6])) + "\n"
    proc = subprocess.run([os.path.join(root, "bin", "trace_run"), "--model", model_dirs["C"], "--dtype", "float32", "--out", str(tmp_path / "out"),
                           "--max-tokens", "64"], input=lines, capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [l for l in proc.stdout.split("\n") if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    last = torch.from_numpy(np.fromfile(tmp_path / "out" / "2.f32", dtype="<f4").reshape(6, cfgc["vocab"]))
    close(last, plain_logits(model_dirs["C"], toks)[6:].double(), "trace_run", 1e-4)

    prompts = [random_tokens(n, cfg["vocab"], 90 + n) for n in (3, 40, 17, 9, 26)]

    def run(use_graphs):
        eng = ContinuousBatchEngine(model_dirs["A"], EngineOptions(dtype="bfloat16", block_size=16, max_batch=3, max_cache_tokens=1024,
                                                                   chunk_size=8, max_step_tokens=24, max_model_len=200, use_graphs=use_graphs))
        assert eng.runner.graph_safe
        out = eng.generate(prompts, max_new_tokens=20, ignore_eos=True)
        return out, eng.runner.graphs_captured

    graphs, captured = run(True)
    eager, none = run(False)
    assert captured > 0 and none == 0
    assert [list(o) for o in graphs] == [list(o) for o in eager]


def wide_config():
    diff = dict(heads=8, kv_heads=2, dim=64, vdim=64, scale=0.1, diff=0.5)
    left = dict(heads=16, kv_heads=4, dim=64, vdim=64, scale=0.1, rot={"base": 10000.0, "dims": 32, "scaling": {"factor": 2.0}})
    right = dict(heads=8, kv_heads=4, dim=64, vdim=128, conv=4)
    gla = dict(heads=4, dim=128, vdim=256, tau=16.0, decay_rank=16)
    moe = {"kind": "moe", "expert": {"ff": 512}, "router": {"experts": 8, "identity": 2, "top": 3}, "shared": {"ff": 1024}}
    return {"architecture": "Muretar", "vocab": 1000, "width": 1024, "norm": {"eps": 1e-5},
            "layers": [{"type": "gla", "mixer": gla, "mlp": {"kind": "dense", "ff": 2048}}, {"type": "attention", "mixer": diff, "mlp": moe},
                       {"type": "parallel", "mixer": {"left": left, "right": right}, "mlp": moe}]}


def test_kernels_chosen_at_real_widths_against_the_general_kernels(tmp_path):
    """A model wide enough that the bfloat16 engine takes what it takes at real sizes (tile products for the prompt with their
    epilogues, weight-streaming products for single tokens, the matrix-core attention, grouped tile products) against the same
    engine on the general kernels: a 300-token prompt, a mixed step and decode steps of a batch.  Both follow the same experts."""
    from photon_infer_amd import ops
    from photon_infer_amd.config import MuretarConfig
    from photon_infer_amd.engine.replay import make_runner
    from photon_infer_amd.engine.step import StepEntry
    from photon_infer_amd.weights import write_random_model
    d = write_random_model(MuretarConfig.from_dict(wide_config()), str(tmp_path / "wide"), seed=2, std=0.03, norm_init="uniform", dtype="bfloat16")
    prompts = {"a": random_tokens(300, 1000, 1), "b": random_tokens(70, 1000, 2), "c": random_tokens(5, 1000, 3)}
    outs, routes = [], []
    real = ops.route
    for fast in (True, False):
        prev = ops.use_fast_kernels(fast)
        calls = []

        def route(*a, **k):
            # the second run follows the first run's experts (a near tie may fall either way between the kernels)
            ids, w = real(*a, **k)
            if fast:
                routes.append(ids)
                return ids, w
            forced = routes[len(calls)]
            calls.append(1)
            scores = torch.softmax(a[0], dim=-1).gather(1, forced.long())
            return forced, (scores / scores.sum(-1, keepdim=True)).contiguous()
        ops.route = route
        try:
            r = make_runner(d, "bfloat16", 1024, 16)
            for rid in prompts:
                r.admit(rid)
            got = [r.step([StepEntry("a", prompts["a"], [0, 150, 299])]),
                   r.step([StepEntry("b", prompts["b"][:60], [59]), StepEntry("c", prompts["c"], [4]), StepEntry("a", [7], [0])])]
            for k in range(3):
                got.append(r.step([StepEntry("a", [8 + k], [0]), StepEntry("b", [prompts["b"][60 + k]], [0]), StepEntry("c", [9 + k], [0])]))
            outs.append(torch.cat(got).float().cpu())
        finally:
            ops.route = real
            ops.use_fast_kernels(prev)
    err = float((outs[0] - outs[1]).abs().max())
    assert err <= 0.04 * float(outs[1].std()) + 0.02, (err, float(outs[1].std()))
