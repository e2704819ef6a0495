"""Dokanex without a GPU: configuration, tensor list, cache plan, the random-weights folder, the work lists of chunked
attention, and the plain implementation held to closed forms of its own."""
import json
import math

import pytest
import torch

import plain_dokanex as P
import tiny_dokanex as TD
from photon_infer_amd.config import DokanexConfig
from photon_infer_amd.errors import ConfigError, UnsupportedModelError
from photon_infer_amd.parts import plan_cache
from photon_infer_amd.registry import build_model_spec, config_from_dict, load_config, registered_architectures

F64 = torch.float64


def copy_of(raw):
    return json.loads(json.dumps(raw))


def test_the_architecture_is_registered_and_its_configuration_round_trips():
    assert "Dokanex" in registered_architectures()
    for name, (raw, _) in TD.ALL.items():
        cfg = config_from_dict(raw)
        assert isinstance(cfg, DokanexConfig) and cfg.vocab_size == raw["vocab"] and cfg.hidden_size == raw["width"]
        assert DokanexConfig.from_dict(cfg.to_dict()) == cfg
        assert cfg.to_dict() == raw, name


def test_configuration_errors_name_the_key():
    raw = copy_of(TD.TINY_A)
    raw["layers"][1]["mixer"]["kv_heads"] = 3
    with pytest.raises(ConfigError, match="kv_heads"):
        config_from_dict(raw)
    raw = copy_of(TD.TINY_A)
    raw["layers"][1]["type"] = "something"
    with pytest.raises(UnsupportedModelError, match="something"):
        config_from_dict(raw)
    raw = copy_of(TD.TINY_A)
    raw["layers"][0]["mixer"]["rot"]["dims"] = 6
    with pytest.raises(ConfigError, match="rot.dims"):
        config_from_dict(raw)
    raw = copy_of(TD.TINY_A)
    del raw["embedding"]
    with pytest.raises(ConfigError, match="embedding"):
        config_from_dict(raw)
    raw = copy_of(TD.TINY_A)
    raw["layers"][0]["mlp"]["kind"] = "other"
    with pytest.raises(UnsupportedModelError, match="other"):
        config_from_dict(raw)
    raw = copy_of(TD.TINY_A)
    raw["layers"][2]["mixer"]["kv_from"] = 0          # a latent layer holds no keys to read
    with pytest.raises(ConfigError, match="kv_from"):
        config_from_dict(raw)
    raw = copy_of(TD.TINY_A)
    raw["layers"][2]["mixer"]["kv_from"] = 2          # nor does the layer itself, nor a later one
    with pytest.raises(ConfigError, match="kv_from"):
        config_from_dict(raw)
    raw = copy_of(TD.TINY_A)
    raw["layers"][2]["mixer"]["dim"] = 32             # keys of another size than the owner's
    with pytest.raises(ConfigError, match="dim"):
        config_from_dict(raw)
    raw = copy_of(TD.TINY_A)
    del raw["layers"][0]["mixer"]["kv_rank"]
    with pytest.raises(ConfigError, match="kv_rank"):
        config_from_dict(raw)


def test_tensor_list_follows_the_layers():
    spec = build_model_spec(config_from_dict(TD.TINY_A))
    shapes = {s.name: tuple(s.shape) for s in spec.tensor_specs()}
    assert shapes["embed"] == (300, 64) and shapes["final.norm"] == (64,) and "head" not in shapes
    assert shapes["l0.mix.dq"] == (20, 64) and shapes["l0.mix.dq.norm"] == (20,) and shapes["l0.mix.uq"] == (2 * 24, 20)
    assert shapes["l0.mix.dkv"] == (24 + 8, 64) and shapes["l0.mix.dkv.norm"] == (24,)
    assert shapes["l0.mix.uk"] == (2 * 16, 24) and shapes["l0.mix.uv"] == (2 * 24, 24) and shapes["l0.mix.o"] == (64, 48)
    assert shapes["l1.mix.q"] == (64, 64) and shapes["l1.mix.k"] == (32, 64) and shapes["l1.mix.v"] == (64, 64)
    assert shapes["l1.mix.sink"] == (4,) and shapes["l1.mix.g"] == (4, 64) and shapes["l1.mix.o"] == (64, 128)
    assert "l2.mix.k" not in shapes and "l2.mix.v" not in shapes and shapes["l2.mix.q"] == (64, 64) and shapes["l2.mix.sink"] == (4,)
    assert not any(n.endswith("mix.q.norm") or n.endswith("mix.k.norm") for n in shapes)         # unit heads have no weights
    assert "l3.mlp.gate" not in shapes and "l3.norm2" not in shapes and shapes["l0.mlp.down"] == (64, 96)


def test_cache_plan_keeps_what_the_longest_reader_reaches():
    """Layers that see all earlier positions share one group; a chunked layer's pages are kept as far back as the longest
    chunk among itself and the layers that read its keys; a reader without chunks keeps everything."""
    plan = plan_cache(build_model_spec(config_from_dict(TD.TINY_A)))
    assert [(g.window, g.owners) for g in plan.groups] == [(None, ((0, 0), (3, 0))), (40, ((1, 0),))]
    assert plan.group_of[(2, 0)] == plan.group_of[(1, 0)] == 1 and plan.owner_of[(2, 0)] == (1, 0)
    latent = plan.groups[0].tensors[0]
    assert [(t.name, t.shape) for t in latent] == [("k", (1, -1, 32)), ("v", (1, 24, -1))]
    plan = plan_cache(build_model_spec(config_from_dict(TD.TINY_C)))
    assert sorted(g.window or 0 for g in plan.groups) == [0, 1, 7]
    plan = plan_cache(build_model_spec(config_from_dict(TD.TINY_D)))
    assert [g.window for g in plan.groups] == [None] and plan.group_of[(2, 0)] == 0


def test_random_weights_folder_loads_back(tmp_path):
    d = TD.make_model_dir(tmp_path, "C", seed=4)
    cfg = load_config(d)
    assert cfg == config_from_dict(TD.TINY_C)
    raw, W = P.read_model_folder(d)
    assert set(W) == {s.name for s in build_model_spec(cfg).tensor_specs()}
    logits = P.forward(raw, W, [3, 200, 17, 5])
    assert logits.shape == (4, 257) and bool(torch.isfinite(logits).all()) and float(logits.abs().max()) <= 30.0
    assert P.greedy(raw, W, [3, 200, 17, 5], 3) == P.greedy(raw, W, [3, 200, 17, 5], 3)


def test_work_lists_walk_a_chunk_not_the_context():
    """A tile's walk ends at its first token's chunk start: late in a long context a chunked layer's tiles walk one or two
    rounds of 128 keys where an unmasked layer's walk dozens."""
    from photon_infer_amd.ops.fast import AttentionPlanner
    full = AttentionPlanner(tile_rows=16, window=0, num_kv_heads=2, singles_apart=True, units=256)
    cut = AttentionPlanner(tile_rows=16, window=0, num_kv_heads=2, singles_apart=True, units=256, chunk=64)
    assert full != cut
    for planner, most in ((full, 33), (cut, 2)):
        arrays, _ = planner.plan([100, 1], [4100, 50])
        order = arrays["order"].reshape(-1)
        assert len(arrays["req"]) >= 7 and (order >= 0).sum() == len(arrays["req"])
        cuts = arrays["cut"] >> 8
        assert (cuts.max() > 1) == (most > 2)           # only the long walks are worth cutting into shares


# ----------------------------------------------------------------------------- the plain implementation, by closed forms
def test_chunk_mask_reaches_exactly_to_its_chunk_start():
    seen = P.chunk_mask(20, 6)
    for i in range(20):
        assert [j for j in range(20) if seen[i, j]] == list(range(i // 6 * 6, i + 1))
    assert bool((P.chunk_mask(5, None) == torch.ones(5, 5).tril().bool()).all())
    assert bool((P.chunk_mask(5, 1) == torch.eye(5).bool()).all())


def test_sink_takes_its_share_and_nothing_else():
    s = torch.tensor([[0.3, -1.0, 2.0]], dtype=F64)
    seen = torch.tensor([[True, True, False]])
    w = P.softmax_with_sink(s, seen, 0.5)
    den = math.exp(0.3) + math.exp(-1.0) + math.exp(0.5)
    assert torch.allclose(w, torch.tensor([[math.exp(0.3) / den, math.exp(-1.0) / den, 0.0]], dtype=F64), atol=1e-15)
    assert abs(float(P.softmax_with_sink(s, seen, None).sum()) - 1.0) < 1e-15
    big = P.softmax_with_sink(s, seen, 800.0)        # a huge sink takes everything, without overflow
    assert bool(torch.isfinite(big).all()) and float(big.sum()) < 1e-300


def test_capped_scores_stay_inside_the_cap():
    s = torch.tensor([-1e4, -3.0, 0.0, 0.01, 3.0, 1e4], dtype=F64)
    c = P.capped(s, 2.0)
    assert float(c.abs().max()) <= 2.0 and abs(float(c[3]) - 0.01) < 1e-6 and bool((P.capped(s, None) == s).all())


def test_rotation_keeps_lengths_up_to_its_factor_and_scores_depend_on_distance():
    freqs, mult = P.yarn_frequencies(8, 100.0, {"factor": 4.0, "original": 32, "fast": 8.0, "slow": 1.0})
    x, y = torch.randn(1, 8, dtype=F64), torch.randn(1, 8, dtype=F64)
    rx = lambda p: P.rotate_pairs(x, torch.tensor([p]), freqs, mult)
    ry = lambda p: P.rotate_pairs(y, torch.tensor([p]), freqs, mult)
    assert abs(float(rx(37).norm()) - mult * float(x.norm())) < 1e-12
    assert abs(float((rx(50) * ry(41)).sum()) - float((rx(109) * ry(100)).sum())) < 1e-9
    plain, one = P.yarn_frequencies(8, 100.0, None)
    assert one == 1.0 and plain == [100.0 ** (-2.0 * i / 8) for i in range(4)]


def test_latent_scores_equal_those_of_explicit_keys():
    """The mixer written out with explicit per-head keys [W_uk c | k_r] and values W_uv c, position by position."""
    torch.manual_seed(3)
    m = copy_of(TD._AL)
    H, d, dr, dv, rank, D, T = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], 64, 9
    W = {"dq": torch.randn(m["q_rank"], D, dtype=F64), "dq.norm": torch.rand(m["q_rank"], dtype=F64) + 0.5,
         "uq": torch.randn(H * (d + dr), m["q_rank"], dtype=F64), "dkv": torch.randn(rank + dr, D, dtype=F64),
         "dkv.norm": torch.rand(rank, dtype=F64) + 0.5, "uk": torch.randn(H * d, rank, dtype=F64),
         "uv": torch.randn(H * dv, rank, dtype=F64), "o": torch.eye(H * dv, dtype=F64)}
    h = torch.randn(T, D, dtype=F64)
    got = P.latent_attention(h, m, W, 1e-6, torch.arange(T))
    freqs, mult = P.yarn_frequencies(dr, m["rot"]["base"], m["rot"]["scaling"])
    for p in (0, 4, 8):
        cq = P.rms_norm(h[p] @ W["dq"].T, W["dq.norm"], 1e-6)
        q = (W["uq"] @ cq).reshape(H, d + dr)
        for n in range(H):
            scores, values = [], []
            for t in range(p + 1):
                down = W["dkv"] @ h[t]
                c = P.rms_norm(down[:rank], W["dkv.norm"], 1e-6)
                key = torch.cat([W["uk"][n * d:(n + 1) * d] @ c, P.rotate_pairs(down[rank:].unsqueeze(0), torch.tensor([t]), freqs, mult)[0]])
                qn = torch.cat([q[n, :d], P.rotate_pairs(q[n, d:].unsqueeze(0), torch.tensor([p]), freqs, mult)[0]])
                scores.append(float(qn @ key) * m["scale"])
                values.append(W["uv"][n * dv:(n + 1) * dv] @ c)
            w = torch.softmax(torch.tensor(scores, dtype=F64), dim=0)
            want = sum(wi * vi for wi, vi in zip(w, values))
            assert torch.allclose(got[p, n * dv:(n + 1) * dv], want, atol=1e-10)
