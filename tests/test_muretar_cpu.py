"""Muretar on the CPU: configuration, run order with shared tensors, tensor list, cache plan, random-weights folder, and the plain
implementation held to closed forms of its own."""
import copy
import math

import pytest
import torch

import plain_muretar as P
import tiny_muretar as TM
from photon_infer_amd.config import MuretarConfig
from photon_infer_amd.errors import ConfigError, UnsupportedModelError
from photon_infer_amd.parts import StateSpec
from photon_infer_amd.parts.model import plan_cache
from photon_infer_amd.registry import build_model_spec, config_from_dict, load_config

F64 = torch.float64


@pytest.mark.parametrize("name", list(TM.ALL))
def test_configuration_round_trip_and_registry(name):
    raw = TM.ALL[name][0]
    cfg = config_from_dict(raw)
    assert isinstance(cfg, MuretarConfig) and cfg.architecture == "Muretar"
    assert MuretarConfig.from_dict(cfg.to_dict()) == cfg
    assert cfg.vocab_size == raw["vocab"] and cfg.hidden_size == raw["width"] and len(cfg.layers) == len(raw["layers"])


def test_errors_name_their_key():
    def broken(edit):
        raw = copy.deepcopy(TM.TINY_A)
        edit(raw)
        return raw
    cases = [(lambda r: r["layers"][1]["mixer"].pop("diff"), "diff"), (lambda r: r["layers"][0]["mixer"].pop("tau"), "tau"),
             (lambda r: r["layers"][3]["mixer"]["left"].update(heads=3), "kv_heads"), (lambda r: r["layers"][3]["mixer"]["left"]["rot"].update(dims=7), "rot.dims"),
             (lambda r: r["layers"][1]["mlp"]["router"].update(top=9), "router.top"), (lambda r: r["layers"][4].update(weights_of=9), "weights_of"),
             (lambda r: r["layers"][4].update(weights_of=0), "cannot run the tensors"), (lambda r: r.pop("norm"), "norm"),
             (lambda r: r["layers"][3]["mixer"].pop("right"), "right")]
    for edit, word in cases:
        with pytest.raises(ConfigError, match=word):
            MuretarConfig.from_dict(broken(edit))
    with pytest.raises(UnsupportedModelError, match="layer type"):
        MuretarConfig.from_dict(broken(lambda r: r["layers"][0].update(type="conv")))
    with pytest.raises(UnsupportedModelError, match="feed-forward kind"):
        MuretarConfig.from_dict(broken(lambda r: r["layers"][0]["mlp"].update(kind="glu")))
    with pytest.raises(ConfigError, match="leads back"):
        MuretarConfig.from_dict(broken(lambda r: (r["layers"][0].update(weights_of=2))))


def test_layers_that_run_another_layers_tensors():
    cfg = MuretarConfig.from_dict(TM.TINY_A)
    assert [cfg.owner(i) for i in range(5)] == [0, 1, 0, 3, 1]
    spec = build_model_spec(cfg)
    assert [p for p, _ in spec.layers] == ["l0.", "l1.", "l3."]                       # layers 2 and 4 have no tensors
    assert [e.layer for e in spec.run_order] == [0, 1, 0, 2, 1]
    names = [s.name for s in spec.tensor_specs()]
    assert not any(n.startswith(("l2.", "l4.")) for n in names) and len(set(names)) == len(names)
    for want in ("embed", "head", "final.norm", "final.norm.b", "l0.norm1b.b", "l0.mix.a2.b", "l0.mlp.gate", "l1.mix.lq2", "l1.mix.q.b", "l1.mlp.e4.up",
                 "l1.mlp.correction", "l1.mlp.shared.down", "l3.mix.left.o.b", "l3.mix.left.out", "l3.mix.right.out", "l3.mix.right.q.conv",
                 "l3.mix.right.dt_bias", "l3.mix.right.A_log", "l3.mix.right.a", "l3.mix.right.g"):
        assert want in names, want
    assert "l1.mlp.e5.up" not in names and "l1.mlp.e0.gate" not in names              # identity experts and ungated experts have none
    shapes = {s.name: s.shape for s in spec.tensor_specs()}
    assert shapes["l1.mlp.router"] == (7, 64) and shapes["l1.mlp.correction"] == (7,)
    assert shapes["l1.mix.q"] == (4 * 2 * 16, 64) and shapes["l1.mix.k"] == (2 * 2 * 16, 64) and shapes["l1.mix.v"] == (2 * 24, 64)
    assert shapes["l3.mix.right.q"] == (2 * 16, 64) and shapes["l3.mix.right.v"] == (4 * 24, 64) and shapes["l3.mix.right.b"] == (4, 64)


def test_cache_plan_gives_every_run_a_memory_of_its_own():
    plan = plan_cache(build_model_spec(MuretarConfig.from_dict(TM.TINY_A)))
    assert len(plan.groups) == 1 and plan.groups[0].window is None
    assert plan.groups[0].owners == ((1, 0), (3, 0), (4, 0))                          # both runs of the attention layer, and the parallel layer's left
    assert [k for k, _ in plan.states] == [(0, 0), (2, 0), (3, 1)]                    # both runs of the gla layer, and the delta rule
    assert all(isinstance(s, StateSpec) and s.dtype == torch.float32 for _, s in plan.states)
    k, v = plan.groups[0].tensors[0]
    assert k.shape == (4, -1, 16) and v.shape == (4, 24, -1)                          # two maps per kv head, the values once per map
    plan = plan_cache(build_model_spec(MuretarConfig.from_dict(TM.TINY_C)))
    assert [k for k, _ in plan.states] == [(0, 1), (1, 1), (2, 0)] and plan.groups[0].owners == ((0, 0), (1, 0), (3, 0))


def test_folder_with_random_weights_and_a_size_taken_from_the_tensors(tmp_path):
    d = TM.make_model_dir(tmp_path, "A", seed=3, ranks_in_config=False)
    cfg = load_config(d)
    assert cfg.layers[0].mixer.decay_rank == 8 and cfg.layers[2].mixer.decay_rank == 8    # layer 2 reads layer 0's tensor
    raw, W = P.read_model_folder(d)
    assert set(W) == {s.name for s in build_model_spec(cfg).tensor_specs()}
    logits = P.forward(raw, W, [5, 6, 7, 8])
    assert logits.shape == (4, 300) and bool(torch.isfinite(logits).all())
    bare = copy.deepcopy(TM.TINY_A)
    bare["layers"][0]["mixer"].pop("decay_rank")
    with pytest.raises(UnsupportedModelError, match="decay_rank"):
        build_model_spec(MuretarConfig.from_dict(bare))


# ----------------------------------------------------------------------------- the plain implementation's own closed forms
def test_layer_norm_centres_and_scales():
    x = torch.randn(5, 33, dtype=F64) * 3 + 2
    y = P.layer_norm(x, torch.ones(33, dtype=F64), torch.zeros(33, dtype=F64), 0.0)
    assert float(y.mean(-1).abs().max()) < 1e-12 and float(((y * y).mean(-1) - 1).abs().max()) < 1e-12
    w, b = torch.rand(33, dtype=F64), torch.randn(33, dtype=F64)
    assert torch.allclose(P.layer_norm(x, w, b, 1e-6), y * w + b, atol=1e-6)


def test_two_equal_maps_leave_a_signed_unit_head():
    """With the second map's queries and keys equal to the first's, o = (1 - lam) a, so the head comes out as the map's own
    result at unit root mean square, signed by 1 - lam and scaled by 1 - diff: lam itself drops out."""
    D, H, G, d, dv, diff = 24, 2, 1, 8, 6, 0.3
    g = torch.Generator().manual_seed(0)
    rnd = lambda *s: torch.randn(*s, generator=g, dtype=F64)
    q1, k1 = rnd(H, d, D), rnd(G, d, D)
    W = {"q": torch.stack([q1, q1], 1).reshape(H * 2 * d, D), "k": torch.stack([k1, k1], 1).reshape(G * 2 * d, D), "v": rnd(G * dv, D),
         "q.b": torch.zeros(H * 2 * d, dtype=F64), "k.b": torch.zeros(G * 2 * d, dtype=F64), "v.b": rnd(G * dv), "o": torch.eye(H * dv, dtype=F64),
         "lq1": rnd(d) * 0.3, "lk1": rnd(d) * 0.3, "lq2": rnd(d) * 0.3, "lk2": rnd(d) * 0.3}
    m = {"heads": H, "kv_heads": G, "dim": d, "vdim": dv, "diff": diff, "scale": 0.4}
    h = rnd(9, D)
    lam = math.exp(float(W["lq1"] @ W["lk1"])) - math.exp(float(W["lq2"] @ W["lk2"])) + diff
    out = P.differential_attention(h, m, W, "", 0.0).view(9, H, dv)
    v = (h @ W["v"].T + W["v.b"]).view(9, G, dv)
    for n in range(H):
        a = P.causal_softmax_attention((h @ q1[n].T), (h @ k1[0].T), v[:, 0], 0.4)
        want = a / torch.sqrt((a * a).mean(-1, keepdim=True)) * math.copysign(1.0, 1.0 - lam) * (1 - diff)
        assert torch.allclose(out[:, n], want, atol=1e-9)
    assert torch.allclose(out[0, 0], v[0, 0] / torch.sqrt((v[0, 0] ** 2).mean()) * math.copysign(1.0, 1.0 - lam) * (1 - diff), atol=1e-9)   # the first token sees itself


def test_decayed_outer_walk_is_a_geometric_sum_per_channel():
    T, d, dv = 12, 3, 2
    alpha = torch.tensor([0.5, 0.9, 1.0], dtype=F64).expand(T, d)
    k, v = torch.ones(T, d, dtype=F64), torch.arange(1, T + 1, dtype=F64).unsqueeze(1) * torch.tensor([1.0, -2.0], dtype=F64)
    for c in range(d):
        q = torch.zeros(T, d, dtype=F64)
        q[:, c] = 1.0
        out = P.decayed_outer_walk(q, k, v, alpha)
        for t in range(T):
            want = sum(float(alpha[0, c]) ** (t - s) * v[s] for s in range(t + 1))
            assert torch.allclose(out[t], want, atol=1e-12)


def test_delta_rule_recalls_a_write_and_overwrites_it():
    d, dv = 4, 3
    e0, e1 = torch.eye(d, dtype=F64)[0], torch.eye(d, dtype=F64)[1]
    v = torch.tensor([[1.0, 2.0, 3.0], [5.0, 5.0, 5.0], [-1.0, 0.0, 1.0], [9.0, 9.0, 9.0]], dtype=F64)
    k = torch.stack([e0, e1, e0, e1])
    q = torch.stack([e0, e0, e0, e0])
    ones = torch.ones(4, dtype=F64)
    out = P.delta_rule_walk(q, k, v, ones, ones)
    assert torch.allclose(out, torch.stack([v[0], v[0], v[2], v[2]]))                # beta 1: a key's value is replaced, others stay
    half = P.delta_rule_walk(q, k, v, ones * 0.5, ones)
    assert torch.allclose(half[2], 0.5 * v[0] + 0.5 * (v[2] - 0.5 * v[0]))           # beta 1/2 moves half the way
    fade = P.delta_rule_walk(q, k, v, ones, ones * 0.5)
    assert torch.allclose(fade[1], 0.5 * v[0])                                        # the decay halves what was written


def test_routing_choice_by_corrected_scores_weights_by_the_scores():
    z = torch.log(torch.tensor([0.4, 0.3, 0.2, 0.1], dtype=F64))
    order, w = P.route(z, torch.zeros(4, dtype=F64), 2)
    assert order == [0, 1] and torch.allclose(w, torch.tensor([4 / 7, 3 / 7], dtype=F64))
    order, w = P.route(z, torch.tensor([0.0, 0.0, 0.0, 0.25], dtype=F64), 2)
    assert order == [0, 3] and torch.allclose(w, torch.tensor([0.8, 0.2], dtype=F64))  # chosen for 0.35, weighed as 0.1
    order, _ = P.route(torch.zeros(4, dtype=F64), torch.zeros(4, dtype=F64), 2)
    assert order == [0, 1]                                                              # equal scores: the lower index


def test_identity_experts_hand_the_input_through():
    D = 6
    h = torch.randn(3, D, dtype=F64)
    mlp = {"router": {"experts": 1, "identity": 2, "top": 2}, "expert": {"ff": 4}}
    W = {"router": torch.zeros(3, D, dtype=F64), "correction": torch.tensor([-1.0, 0.0, 0.0], dtype=F64), "e0.up": torch.randn(4, D, dtype=F64),
         "e0.down": torch.randn(D, 4, dtype=F64)}
    assert torch.allclose(P.routed_experts(h, mlp, W, ""), h)                           # two identities at half weight each
    W["correction"] = torch.tensor([1.0, 0.0, 0.0], dtype=F64)
    want = 0.5 * h + 0.5 * P.squared_relu_unit(h, W, "e0.")
    assert torch.allclose(P.routed_experts(h, mlp, W, ""), want)


def test_rotation_of_neighbouring_pairs_with_divided_frequencies():
    x = torch.randn(2, 8, dtype=F64)
    y = P.rotate_pairs(x, 5, 4, 10.0, 2.0)
    assert torch.equal(y[:, 4:], x[:, 4:])
    for i, f in enumerate([1.0 / 2.0, 10.0 ** -0.5 / 2.0]):
        c, s = math.cos(5 * f), math.sin(5 * f)
        assert torch.allclose(y[:, 2 * i], x[:, 2 * i] * c - x[:, 2 * i + 1] * s) and torch.allclose(y[:, 2 * i + 1], x[:, 2 * i + 1] * c + x[:, 2 * i] * s)
    assert torch.allclose((y * y).sum(-1), (x * x).sum(-1))
