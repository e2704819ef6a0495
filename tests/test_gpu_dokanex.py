"""Dokanex on the GPU against the plain implementation (``plain_dokanex``): each mechanism's kernels alone, with inputs made
so that a fault shows (a loud key just inside and just outside a chunk, a loud key far back in a latent cache, a lone key
beside the sink), then whole models under every cutting, batching, page and slot reuse, long decoding, and greedy generation
through the engine's own entry point."""
import json
import math
import os
from types import SimpleNamespace

import numpy as np
import pytest
import torch

import plain_dokanex as P
import tiny_dokanex as TD
from gpu_tools import DEV, PagedKV, attention_ctx, cut_steps, live_token_need, run_trace
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


def chunk_attend(q, k, v, scale, cap, size, sinks, gate):
    """The plain attention of [T, H, d] queries over [T, G, d] keys and [T, G, dv] values, from the oracle's mechanisms."""
    T, H, G = q.shape[0], q.shape[1], k.shape[1]
    seen = P.chunk_mask(T, size)
    out = torch.zeros((T, H, v.shape[2]), dtype=F64)
    for n in range(H):
        g = n // (H // G)
        s = P.capped((q[:, n] @ k[:, g].T) * scale, cap)
        w = P.softmax_with_sink(s, seen, None if sinks is None else float(sinks[n]))
        out[:, n] = (w @ v[:, g]) * (1.0 if gate is None else gate[:, n:n + 1])
    return out


# ----------------------------------------------------------------------------- mechanisms alone
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("sizes", [(4, 2, 16, 32), (4, 1, 64, 64), (6, 3, 24, 12), (3, 3, 40, 40), (1, 1, 48, 80)])
def test_unit_heads_into_the_cache_and_gates(dtype, sizes):
    """Every head of q and k divided by the root mean square of its own entries, keys and values into pages, gates through
    a sigmoid; then the same rows without keys and values (a layer that reads another's)."""
    from photon_infer_amd import ops
    H, G, d, dv = sizes
    T, page, eps = 45, 8, 3e-3
    tdt = TORCH[dtype]
    row = randn(T, H * d + G * d + G * dv + H, seed=4, scale=2.0)
    row[:, :d] *= 30.0                                     # one loud head must not change its neighbours' norms
    proj = row.float().to(DEV).contiguous()
    table, pages = paged([T], page)
    kc = torch.zeros((pages, G, page, d), dtype=tdt, device=DEV)
    vc = torch.zeros((pages, G, dv, page), dtype=tdt, device=DEV)
    ctx = attention_ctx([T], [T], tdt)
    q = torch.empty((T, H * d), dtype=tdt, device=DEV)
    gate = torch.empty((T, H), dtype=torch.float32, device=DEV)
    ops.qk_norm_kv_write(q, gate, proj, None, None, ctx, eps, 0.0, 1, H, G, d, dv, H, kc, vc, table, page, per_head=True)
    row = proj.double().cpu()
    want_q = P.rms_norm(row[:, :H * d].reshape(T, H, d), None, eps).reshape(T, -1)
    want_k = P.rms_norm(row[:, H * d:H * d + G * d].reshape(T, G, d), None, eps)
    want_v = row[:, H * d + G * d:H * d + G * d + G * dv].reshape(T, G, dv)
    tol = 1e-5 if dtype == "float32" else 1e-2
    close(q, want_q, "unit queries", tol)
    close(gate, P.sigmoid(row[:, -H:]), "gates", 1e-6)
    for t in (0, 7, 8, 44):
        pg, slot = int(table[0, t // page]), t % page
        close(kc[pg, :, slot], want_k[t], f"unit key {t} in its page", tol)
        close(vc[pg, :, :, slot], want_v[t], f"value {t} in its page", tol)
    # the reader's rows: [q | gates] only; nothing is written
    proj2 = torch.cat([proj[:, :H * d], proj[:, -H:]], dim=1).contiguous()
    q2, gate2 = torch.empty_like(q), torch.empty_like(gate)
    before = kc.clone()
    ops.qk_norm_kv_write(q2, gate2, proj2, None, None, ctx, eps, 0.0, 1, H, G, d, dv, H, None, None, table, page, per_head=True, has_kv=False)
    assert torch.equal(q2, q) and torch.equal(gate2, gate) and torch.equal(kc, before)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("sizes", [(4, 2, 16, 32, 24), (4, 1, 64, 64, 32), (6, 3, 24, 12, 7), (2, 2, 128, 128, 100), (3, 3, 40, 40, 1), (8, 2, 48, 48, 64)])
def test_chunks_capped_scores_sink_and_gate(dtype, sizes):
    """Attention within chunks over pages dealt out of order: a whole prompt, then its last tokens alone and four at a time.
    The last token's query is loud towards two keys: the first of its own chunk (seen) and the last of the chunk before
    (not seen): a mask that is one position off moves the result by far more than the tolerance."""
    from photon_infer_amd import ops
    H, G, d, dv, size = sizes
    T, page, cap, scale = 333, 16, 6.0, 0.3
    tdt = TORCH[dtype]
    q, k, v = randn(T, H, d, seed=1), randn(T, G, d, seed=2), randn(T, G, dv, seed=3)
    start = (T - 1) // size * size
    mark = randn(d, seed=9)
    q[-1] = mark * 1.5
    k[start] = mark                                        # just inside
    if start > 0:
        k[start - 1] = mark * 1.2                          # just outside, and louder
    v[start] += 4.0
    if start > 0:
        v[start - 1] -= 4.0
    sinks, gate = randn(H, seed=5), P.sigmoid(randn(T, H, seed=6))
    rnd = lambda t: t.to(tdt).double()
    want = chunk_attend(rnd(q), rnd(k), rnd(v), scale, cap, size, sinks, gate)
    if start > 0 and size > 1:        # one position more, or one less, is another result
        off_by_one = chunk_attend(rnd(q), rnd(k), rnd(v), scale, cap, None, sinks, gate)
        assert float((want[-1] - off_by_one[-1]).abs().max()) > 0.05
    kv = PagedKV([(k, v)], page, tdt, seed=3)
    sk, gt = sinks.float().to(DEV), gate.float().to(DEV).contiguous()
    tol = 3e-5 if dtype == "float32" else 3e-2
    for q_len in (T, 1, 4, 70):
        ctx = attention_ctx([q_len], [T], tdt)
        rows = slice(T - q_len, T)
        qd = q[rows].reshape(q_len, -1).to(tdt).to(DEV).contiguous()
        out = torch.empty((q_len, H * dv), dtype=tdt, device=DEV)
        ops.paged_attention(out, qd, kv.k, kv.v, kv.table, ctx, H, G, d, page, scale, 0, None, value_dim=dv, sinks=sk,
                            gate=gt[rows].contiguous(), softcap=cap, chunk=size)
        close(out, want[rows].reshape(q_len, -1), f"{sizes} {q_len} tokens ending the sequence", tol)


def test_a_lone_key_beside_the_sink_in_closed_form():
    """The first token of a chunk sees itself and the sink: its weight is e^s / (e^s + e^sink) with the capped score s."""
    from photon_infer_amd import ops
    H, d, size, page, scale, cap = 2, 32, 16, 16, 0.5, 3.0
    T = 2 * size + 1
    q, k, v = randn(T, H, d, seed=1), randn(T, H, d, seed=2), randn(T, H, d, seed=3)
    sinks = torch.tensor([0.7, -1.1], dtype=F64)
    kv = PagedKV([(k, v)], page, torch.float32)
    ctx = attention_ctx([1], [T], torch.float32)
    out = torch.empty((1, H * d), dtype=torch.float32, device=DEV)
    ops.paged_attention(out, q[-1:].reshape(1, -1).float().to(DEV), kv.k, kv.v, kv.table, ctx, H, H, d, page, scale, 0, None,
                        value_dim=d, sinks=sinks.float().to(DEV), softcap=cap, chunk=size)
    for n in range(H):
        s = cap * math.tanh(float(q[-1, n] @ k[-1, n]) * scale / cap)
        w = math.exp(s) / (math.exp(s) + math.exp(float(sinks[n])))
        close(out[0, n * d:(n + 1) * d], v[-1, n] * w, f"head {n}", 1e-5)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("sizes", [(2, 16, 8, 24, 20, 24), (4, 32, 16, 32, 64, 48), (3, 20, 6, 28, 10, 30), (1, 24, 16, 40, 32, 272), (5, 8, 2, 8, 8, 8),
                                   (20, 8, 8, 8, 16, 24), (16, 16, 16, 16, 32, 112)])
def test_latent_attention_mixer_whole_in_portions_and_token_by_token(dtype, sizes):
    """The mixer as a part on pages dealt out of order: a prompt whole, then in portions, then its end token by token; the
    rotation's frequencies are scaled over an original length that the prompt passes.  One latent far back is loud."""
    from photon_infer_amd.parts import MIXERS, POSITION_ENCODINGS, LayerCache
    from photon_infer_amd.parts.rope import RampScaling
    H, d, dr, dv, qr, rank = sizes
    D, T, page, eps, scale, base = 72, 150, 16, 1e-5, 0.12, 300.0
    scaling = {"factor": 4.0, "original": 48, "fast": 6.0, "slow": 1.0}
    m = {"heads": H, "dim": d, "rot_dim": dr, "vdim": dv, "q_rank": qr, "kv_rank": rank, "scale": scale,
         "rot": {"base": base, "dims": dr, "scaling": scaling}}
    tdt = TORCH[dtype]
    shapes = {"dq": (qr, D), "uq": (H * (d + dr), qr), "dkv": (rank + dr, D), "uk": (H * d, rank), "uv": (H * dv, rank), "o": (D, H * dv)}
    W = {n: randn(*s, seed=10 + i, scale=0.2).to(torch.bfloat16).double() for i, (n, s) in enumerate(shapes.items())}
    W["dq.norm"], W["dkv.norm"] = 0.5 + torch.rand(qr, dtype=F64), 0.5 + torch.rand(rank, dtype=F64)
    h = randn(T, D, seed=3).to(tdt).double()
    h[5] *= 4.0                                            # far back, and loud
    want = P.latent_attention(h, m, W, eps, torch.arange(T))
    rope = POSITION_ENCODINGS.make("rope", head_dim=dr, theta=base, interleaved=True, scaling=RampScaling(4.0, 48, 6.0, 1.0))
    mixer = MIXERS.make("latent_attention", hidden_size=D, num_heads=H, head_dim=d, rot_dim=dr, value_dim=dv, q_rank=qr, kv_rank=rank,
                        scale=scale, eps=eps, position=rope)
    mixer.load({n: t.to(tdt if t.dim() == 2 else torch.float32).to(DEV) for n, t in W.items()}, tdt, torch.device(DEV))
    table, pages = paged([T], page, seed=2)
    spec = mixer.cache_spec()
    pools = {t.name: torch.zeros((pages, *t.page_shape(page)), dtype=tdt, device=DEV) for t in spec.tensors}
    cache = LayerCache(group=0, k=pools["k"], v=pools["v"], page_size=page, writes=True, tensors=pools)
    tol = 1e-4 if dtype == "float32" else 4e-2
    for cuts in ([T], [64, 7, 2, 77], [T - 12] + [1] * 12):
        for t in pools.values():
            t.zero_()
        done = 0
        for n in cuts:
            ctx = attention_ctx([n], [done + n], tdt)
            ctx.block_tables, ctx.may_defer = {0: table}, False
            x = torch.zeros((n, D), dtype=torch.float32, device=DEV)
            mixer.forward(h[done:done + n].to(tdt).to(DEV).contiguous(), x, ctx, cache)
            close(x, want[done:done + n], f"{sizes} tokens {done} .. {done + n} of cuts {cuts[:4]}", tol)
            done += n


def test_scaled_rotation_table_and_the_ramp_ends():
    """cos and sin of the step's table against the plain frequencies, at positions far beyond the original length; pairs below
    the ramp keep their frequency, pairs above it turn ``factor`` times slower, and both are stretched by 0.1 ln(factor) + 1."""
    from photon_infer_amd import ops
    from photon_infer_amd.parts.rope import RampScaling, rope_frequencies
    dims, base, sc = 32, 10000.0, {"factor": 8.0, "original": 256, "fast": 32.0, "slow": 1.0}
    f, mult = P.yarn_frequencies(dims, base, sc)
    plain = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    assert f[0] == plain[0] and abs(f[-1] - plain[-1] / 8.0) < 1e-18 and any(plain[i] / 8.0 < f[i] < plain[i] for i in range(dims // 2))
    assert abs(mult - (0.1 * math.log(8.0) + 1.0)) < 1e-15
    scaling = RampScaling(8.0, 256, 32.0, 1.0)
    inv = rope_frequencies(dims, base, scaling)
    close(inv, torch.tensor(f, dtype=F64), "frequencies", 1e-12)
    pos = torch.tensor([0, 1, 255, 256, 4097, 30000], dtype=torch.int32, device=DEV)
    table = ops.rope_table(pos, inv.float().to(DEV), scaling.magnitude)
    ang = (pos.cpu().float().unsqueeze(1) * inv.float().unsqueeze(0)).double()      # the angle is a float32 product, as the design asks
    close(table[:, :dims // 2], torch.cos(ang) * mult, "cosines", 3e-6)
    close(table[:, dims // 2:], torch.sin(ang) * mult, "sines", 3e-6)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("sizes", [(1, 3, 24, 30, 0), (9, 4, 16, 24, 8), (77, 2, 128, 200, 16), (8, 5, 7, 65, 2), (130, 1, 64, 64, 0),
                                   (300, 3, 64, 96, 16), (257, 4, 40, 72, 0)])
def test_a_product_per_head_with_a_rotated_tail(dtype, sizes):
    """Few tokens take the general kernel; in bfloat16, from 129 tokens on, heads that start at multiples of 8 columns take
    the matrix-core kernel (one launch, every head a group at columns of its own), the rotated tails a launch of their own."""
    from photon_infer_amd import ops
    M, H, K, N, rot = sizes
    tdt = TORCH[dtype]
    a, w = randn(M, H * (K + rot) + (8 if M > 128 else 3), seed=1).to(tdt), randn(H, K, N, seed=2).to(tdt)
    freqs = [0.37 ** i for i in range(rot // 2)]
    pos = torch.arange(M) * 3
    want = torch.zeros((M, H, N + rot), dtype=F64)
    ah = a[:, :H * (K + rot)].double().reshape(M, H, K + rot)
    want[..., :N] = torch.einsum("mhk,hkn->mhn", ah[..., :K], w.double())
    table = None
    if rot:
        want[..., N:] = P.rotate_pairs(ah[..., K:], pos, freqs, 1.3)
        table = ops.rope_table(pos.to(torch.int32).to(DEV), torch.tensor(freqs, dtype=torch.float32, device=DEV), 1.3)
    out = torch.full((M, H * (N + rot) + 5), 7.0, dtype=tdt, device=DEV)
    rows = w.transpose(1, 2).contiguous().to(DEV) if dtype == "bfloat16" else None
    ops.head_gemm(out, a.to(DEV), w.to(DEV).contiguous(), H, rot=rot, table=table, w_rows=rows)
    close(out[:, :H * (N + rot)], want.reshape(M, -1), f"{sizes}", 2e-5 if dtype == "float32" else 2e-2)
    assert bool((out[:, H * (N + rot):] == 7.0).all())


def test_scaled_embedding_and_capped_logits():
    from photon_infer_amd import ops
    table = randn(50, 24, seed=1).to(torch.bfloat16)
    ids = torch.tensor([3, 49, 0, 3], dtype=torch.int32, device=DEV)
    x = torch.empty((4, 24), dtype=torch.float32, device=DEV)
    ops.embedding(x, table.to(DEV), ids, 2.5)
    close(x, table.double()[ids.cpu().long()] * 2.5, "scaled rows", 1e-6)
    lg = randn(3, 1000, seed=2, scale=20.0)
    dev = lg.float().to(DEV).contiguous()
    ops.softcap_(dev, 9.0)
    close(dev, 9.0 * torch.tanh(lg / 9.0), "capped logits", 1e-6)


# ----------------------------------------------------------------------------- whole models
@pytest.fixture(scope="module")
def model_dirs(tmp_path_factory):
    base = tmp_path_factory.mktemp("dokanex")
    return {name: TD.make_model_dir(base, name) for name in TD.ALL}


_plain = {}


def plain_logits(model_dir, tokens, emulate=False):
    key = (model_dir, tuple(tokens), emulate)
    if key not in _plain:
        cfg, W = P.read_model_folder(model_dir)
        _plain[key] = P.forward(cfg, W, list(tokens), act_round=P.bf16_round if emulate else None).float()
    return _plain[key]


def runner_for(model_dir, name, dtype, max_tokens):
    from photon_infer_amd.engine.replay import make_runner
    return make_runner(model_dir, dtype, max(max_tokens, 64), TD.ALL[name][1]["block_size"])


def check(got, model_dir, reqs, dtype, what):
    assert got, "no logits came back"
    for rid, toks in reqs.items():
        ref = plain_logits(model_dir, toks)
        if dtype == "float32":
            tol = 1e-4 * max(1.0, float(ref.abs().max()))
        else:       # three times what rounding activations to bfloat16 does to the plain implementation itself
            tol = 3.0 * float((plain_logits(model_dir, toks, True) - ref).abs().max())
        for p in range(len(toks)):
            assert (rid, p) in got, f"{what}: logits of {rid} position {p} are missing"
            err = float((got[(rid, p)] - ref[p]).abs().max())
            assert err <= tol, f"{what}: {rid} position {p}: error {err:.3e} > {tol:.3e} (first wrong position)"


LENGTHS = {"A": [1, 26, 130], "B": [3, 100, 210], "C": [2, 30, 75], "D": [2, 45, 100]}


def requests_for(name, seed=0):
    vocab = TD.ALL[name][0]["vocab"]
    return {f"r{i}": random_tokens(n, vocab, seed * 100 + i) for i, n in enumerate(LENGTHS[name])}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(TD.ALL))
def test_whole_prompts_and_the_stream_after_every_layer(name, dtype, model_dirs, tmp_path):
    reqs = requests_for(name)
    steps = []
    for rid, toks in reqs.items():
        steps += cut_steps(rid, toks, [len(toks)], first_step=len(steps))
    runner = runner_for(model_dirs[name], name, dtype, live_token_need(steps))
    check(run_trace(runner, steps, str(tmp_path)), model_dirs[name], reqs, dtype, "whole")
    if dtype == "float32":
        from photon_infer_amd import ops
        from photon_infer_amd.engine.step import StepEntry
        toks = reqs["r2"]
        cfg, W = P.read_model_folder(model_dirs[name])
        want, got = [], []
        P.forward(cfg, W, toks, streams=want)
        for blk in runner.model.blocks:
            def wrapped(x, ctx, cache, f=blk.forward):
                f(x, ctx, cache)
                ops.materialize(x, ctx.workspace)
                got.append(x.detach().double().cpu())
            blk.forward = wrapped
        runner.admit("s")
        runner.step([StepEntry("s", toks, [])])
        assert len(got) == len(want) == len(cfg["layers"])
        for i, (g, w) in enumerate(zip(got, want)):
            close(g, w, f"stream after layer {i}", 1e-4)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(TD.ALL))
def test_prefill_then_token_by_token_and_all_token_by_token(name, dtype, model_dirs, tmp_path):
    """The last 50 tokens one by one (every chunk's edge of the tiny models is passed by single tokens), and a whole request
    token by token from its first."""
    reqs = requests_for(name, seed=1)
    steps = []
    for rid, toks in reqs.items():
        head = max(0, len(toks) - 50)
        sizes = ([head] if head else []) + [1] * (len(toks) - head)
        steps += cut_steps(rid, toks, sizes, first_step=len(steps))
    steps += cut_steps("all", reqs["r1"], [1], first_step=len(steps))
    runner = runner_for(model_dirs[name], name, dtype, live_token_need(steps))
    check(run_trace(runner, steps, str(tmp_path)), model_dirs[name], dict(reqs, all=reqs["r1"]), dtype, "decoding")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(TD.ALL))
@pytest.mark.parametrize("sizes", [[2], [7, 2, 31, 1, 3], [64, 5], [17]])
def test_portions_of_changing_size(name, dtype, sizes, model_dirs, tmp_path):
    reqs = {"r2": requests_for(name, seed=2)["r2"]}
    steps = cut_steps("r2", reqs["r2"], sizes)
    runner = runner_for(model_dirs[name], name, dtype, live_token_need(steps))
    check(run_trace(runner, steps, str(tmp_path)), model_dirs[name], reqs, dtype, f"portions {sizes}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(TD.ALL))
def test_mixed_batches_with_pages_and_slots_used_again(name, dtype, model_dirs, tmp_path):
    """Seven unequal requests through four slots: portions of some beside single tokens of others; a request may sit
    out a step; a finished request's pages and slot go to the next one.  Each must come out as it does alone."""
    vocab = TD.ALL[name][0]["vocab"]
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
    check(run_trace(runner, steps, str(tmp_path)), model_dirs[name], reqs, dtype, "mixed")
    assert all(g.pool.num_allocated == 0 for g in runner.cache.groups)


@pytest.mark.parametrize("name", ["A", "C"])
def test_long_decoding_over_many_chunks_gives_pages_back(name, model_dirs, tmp_path):
    """250 tokens one by one after a portion of three, over a pool of 256 tokens: the chunked layers' group hands pages back
    while the request runs, the latent layers' group keeps all."""
    vocab = TD.ALL[name][0]["vocab"]
    toks = random_tokens(250, vocab, 9)
    steps = cut_steps("long", toks, [3] + [1] * 247, end=False)
    runner = runner_for(model_dirs[name], name, "float32", 256)
    check(run_trace(runner, steps, str(tmp_path)), model_dirs[name], {"long": toks}, "float32", "long decoding")
    held = {g.window: g.pool.num_allocated for g in runner.cache.groups}
    page = TD.ALL[name][1]["block_size"]
    assert held[None] == -(-250 // page)
    assert all(n <= -(-w // page) + 1 for w, n in held.items() if w is not None), held


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", list(TD.ALL))
def test_greedy_generation_through_the_engine(name, dtype, model_dirs):
    """The engine's own entry point, scheduler, sampling and decode steps: unequal prompts at once, more requests than
    slots, prompts longer than a portion; every request must generate what the plain implementation generates alone."""
    from photon_infer_amd.engine import ContinuousBatchEngine, EngineOptions
    cfg, W = P.read_model_folder(model_dirs[name])
    vocab = cfg["vocab"]
    prompts = [random_tokens(n, vocab, 70 + i) for i, n in enumerate([5, 41, 18, 70, 2])]
    engine = ContinuousBatchEngine(model_dirs[name], EngineOptions(dtype=dtype, block_size=TD.ALL[name][1]["block_size"], max_batch=3,
                                                                   max_cache_tokens=1024, chunk_size=32, max_model_len=200))
    got = engine.generate(prompts, max_new_tokens=10)
    for prompt, out in zip(prompts, got):
        want = P.greedy(cfg, W, prompt, 10)
        if dtype == "float32":
            assert list(out) == want
        else:       # bfloat16: a near tie may fall the other way; everything before the first difference must agree and the
            # differing token must be a close second of the plain logits
            for i, (a, b) in enumerate(zip(out, want)):
                if a != b:
                    lg = P.forward(cfg, W, prompt + want[:i])[-1]
                    assert float(lg[b] - lg[a]) < 0.05 * float(lg.std()), f"token {i}: {a} instead of {b}"
                    break


def test_command_line_and_replayed_decode_steps(model_dirs, tmp_path):
    """The framework's commands serve the design as they serve its others (from a folder, and from a bare configuration
    with random weights); and decode steps replayed as HIP graphs give the tokens of eager steps, with new requests'
    prompts in between and pages that are used again."""
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
    assert "Architecture: Dokanex" in proc.stdout and f"Generated ids: {','.join(map(str, want))}" in proc.stdout
    (tmp_path / "cfg").mkdir()
    json.dump(TD.TINY_D, open(tmp_path / "cfg" / "config.json", "w"))
    proc = subprocess.run([os.path.join(root, "bin", "llama_infer"), str(tmp_path / "cfg"), "--random-weights", "--seed", "3",
                           "--prompt-ids", "5,6,7", "--max-new-tokens", "4", "--ignore-eos"], capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert "Generated ids:" in proc.stdout
    # the trace replay as a command, from the folder
    toks = random_tokens(12, cfg["vocab"], 82)
    lines = "\n".join(json.dumps(s) for s in cut_steps("x", toks, [5, 1, 6])) + "\n"
    proc = subprocess.run([os.path.join(root, "bin", "trace_run"), "--model", model_dirs["A"], "--dtype", "float32", "--out", str(tmp_path / "out"),
                           "--max-tokens", "64"], input=lines, capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [l for l in proc.stdout.split("\n") if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    last = torch.from_numpy(np.fromfile(tmp_path / "out" / "2.f32", dtype="<f4").reshape(6, cfg["vocab"]))
    close(last, plain_logits(model_dirs["A"], toks)[6:].double(), "trace_run", 1e-4)

    prompts = [random_tokens(n, cfg["vocab"], 90 + n) for n in (3, 40, 17, 9, 26)]

    def run(name, use_graphs):
        eng = ContinuousBatchEngine(model_dirs[name], EngineOptions(dtype="bfloat16", block_size=16, max_batch=3, max_cache_tokens=1024,
                                                                    chunk_size=8, max_step_tokens=24, max_model_len=200, use_graphs=use_graphs))
        assert eng.runner.graph_safe
        out = eng.generate(prompts, max_new_tokens=20, ignore_eos=True)
        return out, eng.runner.graphs_captured

    for name in ("A", "B"):
        graphs, captured = run(name, True)
        eager, none = run(name, False)
        assert captured > 0 and none == 0
        assert [list(o) for o in graphs] == [list(o) for o in eager]


def wide_config():
    att = dict(heads=16, kv_heads=4, dim=64, vdim=64, scale=0.12, softcap=15.0, mask={"size": 128})
    lat = dict(heads=8, dim=64, rot_dim=32, vdim=64, q_rank=384, kv_rank=160, scale=0.1,
               rot={"base": 10000.0, "dims": 32, "scaling": {"factor": 4.0, "original": 128, "fast": 16.0, "slow": 1.0}})
    ff = {"kind": "dense", "ff": 2048}
    return {"architecture": "Dokanex", "vocab": 1000, "width": 1024, "embedding": {"scale": 32.0}, "norm": {"eps": 1e-5}, "logit_softcap": 25.0,
            "layers": [{"type": "latent_attention", "mixer": lat, "mlp": ff}, {"type": "attention", "mixer": att, "mlp": ff},
                       {"type": "attention", "mixer": dict(att, kv_from=1), "mlp": ff}]}


def test_kernels_chosen_at_real_widths_against_the_general_kernels(tmp_path):
    """A model wide enough that the bfloat16 engine takes what it takes at real sizes (tile products for the prompt,
    weight-streaming products for single tokens, the matrix-core attention with chunks, a sink and a gate, and over the
    latent cache) against the same engine on the general kernels: a 300-token prompt, a mixed step and decode steps of a batch."""
    from photon_infer_amd import ops
    from photon_infer_amd.config import DokanexConfig
    from photon_infer_amd.engine.replay import make_runner
    from photon_infer_amd.engine.step import StepEntry
    from photon_infer_amd.weights import write_random_model
    d = write_random_model(DokanexConfig.from_dict(wide_config()), str(tmp_path / "wide"), seed=2, std=0.03, norm_init="uniform", dtype="bfloat16")
    prompts = {"a": random_tokens(300, 1000, 1), "b": random_tokens(70, 1000, 2), "c": random_tokens(5, 1000, 3)}
    outs = []
    for fast in (True, False):
        prev = ops.use_fast_kernels(fast)
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
            ops.use_fast_kernels(prev)
    err = float((outs[0] - outs[1]).abs().max())
    assert err <= 0.04 * float(outs[1].std()) + 0.02, (err, float(outs[1].std()))
