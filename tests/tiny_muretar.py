"""Tiny Muretar configurations for tests; they differ from one another in every size, constant and layer order."""
from __future__ import annotations

import json
import os

from photon_infer_amd.config import MuretarConfig
from photon_infer_amd.weights import write_random_model


def _layer(kind, mixer, mlp, weights_of=None):
    d = {"type": kind, "mixer": mixer, "mlp": mlp}
    if weights_of is not None:
        d["weights_of"] = weights_of
    return d


def _moe(ff, experts, identity, top, shared=None):
    d = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "identity": identity, "top": top}}
    if shared is not None:
        d["shared"] = {"ff": shared}
    return d


def _dense(ff):
    return {"kind": "dense", "ff": ff}


# A: values wider than keys under two maps, two kv heads under four; a quarter of a head rotated with frequencies divided by
# three; a delta rule with two key heads under four and three taps; experts of which two of seven are identities, a shared
# expert; the attention layer's tensors run a second time at the end, the gla layer's in the middle
_AD = dict(heads=4, kv_heads=2, dim=16, vdim=24, scale=0.3, diff=0.35)
_AL = dict(heads=4, kv_heads=2, dim=16, vdim=32, scale=0.25, rot={"base": 100.0, "dims": 8, "scaling": {"factor": 3.0}})
_AR = dict(heads=4, kv_heads=2, dim=16, vdim=24, conv=3)
_AG = dict(heads=2, dim=24, vdim=16, tau=8.0, decay_rank=8)
_AM = _moe(40, 5, 2, 3, shared=56)
TINY_A = {"architecture": "Muretar", "vocab": 300, "width": 64, "norm": {"eps": 1e-6},
          "layers": [_layer("gla", _AG, _dense(96)), _layer("attention", _AD, _AM), _layer("gla", _AG, _dense(96), weights_of=0),
                     _layer("parallel", {"left": _AL, "right": _AR}, _AM), _layer("attention", _AD, _AM, weights_of=1)]}
TINY_A_INIT = dict(std=0.15, block_size=16)

# B: sizes the matrix-core kernels take: maps of 64 with values of 64, four heads on one kv head; the whole head of 64 rotated,
# no scaling of the frequencies; as many key heads as heads in the delta rule, four taps; eight experts, no identity, four
# chosen, expert widths that are multiples of 32
_BD = dict(heads=4, kv_heads=1, dim=64, vdim=64, scale=0.09, diff=0.8)
_BL = dict(heads=4, kv_heads=1, dim=64, vdim=64, scale=0.1, rot={"base": 10000.0, "dims": 64})
_BR = dict(heads=4, kv_heads=4, dim=32, vdim=32, conv=4)
_BG = dict(heads=4, dim=32, vdim=64, tau=16.0, decay_rank=16)
TINY_B = {"architecture": "Muretar", "vocab": 776, "width": 256, "norm": {"eps": 1e-5},
          "layers": [_layer("attention", _BD, _moe(128, 8, 0, 4, shared=64)), _layer("parallel", {"left": _BL, "right": _BR}, _dense(384)),
                     _layer("gla", _BG, _moe(96, 6, 2, 2))]}
TINY_B_INIT = dict(std=0.08, block_size=16)

# C: sizes that fit no fast kernel: a width that is no multiple of 8, an odd vocabulary, head sizes that are no multiples of
# 16 or 4, three kv heads, keys wider than values, no rotation at all, five taps, one key head under three, one expert per token,
# no shared expert, a layer without feed-forward, a parallel layer run twice in a row, pages of 8
_CD = dict(heads=6, kv_heads=3, dim=12, vdim=10, scale=0.4, diff=0.1)
_CL = dict(heads=6, kv_heads=3, dim=24, vdim=12, scale=0.25)
_CR = dict(heads=3, kv_heads=1, dim=20, vdim=28, conv=5)
_CG = dict(heads=3, dim=20, vdim=28, tau=3.5, decay_rank=5)
TINY_C = {"architecture": "Muretar", "vocab": 257, "width": 100, "norm": {"eps": 2e-6},
          "layers": [_layer("parallel", {"left": _CL, "right": _CR}, None), _layer("parallel", {"left": _CL, "right": _CR}, None, weights_of=0),
                     _layer("gla", _CG, _moe(36, 9, 3, 1)), _layer("attention", _CD, _dense(52))]}
TINY_C_INIT = dict(std=0.12, block_size=8)

# D: one head everywhere, values as wide as keys, one tap, a root of one, frequencies divided by one, half a head rotated; one
# real expert beside three identities with every router output chosen; diff zero
_DD = dict(heads=1, kv_heads=1, dim=48, vdim=48, scale=0.15, diff=0.0)
_DL = dict(heads=1, kv_heads=1, dim=32, vdim=32, scale=0.2, rot={"base": 50.0, "dims": 16, "scaling": {"factor": 1.0}})
_DR = dict(heads=1, kv_heads=1, dim=48, vdim=80, conv=1)
_DG = dict(heads=1, dim=40, vdim=40, tau=1.0, decay_rank=4)
TINY_D = {"architecture": "Muretar", "vocab": 512, "width": 128, "norm": {"eps": 1e-5},
          "layers": [_layer("parallel", {"left": _DL, "right": _DR}, _moe(48, 1, 3, 4)), _layer("gla", _DG, None), _layer("attention", _DD, _moe(32, 3, 1, 2, shared=16))]}
TINY_D_INIT = dict(std=0.1, block_size=16)

ALL = {"A": (TINY_A, TINY_A_INIT), "B": (TINY_B, TINY_B_INIT), "C": (TINY_C, TINY_C_INIT), "D": (TINY_D, TINY_D_INIT)}


def make_model_dir(tmp_path, name: str, seed: int = 0, ranks_in_config: bool = True) -> str:
    """A model folder with random weights.  ``ranks_in_config`` False: config.json does not name the decay projection's
    inner size, which a reader then takes from the tensors' shapes."""
    raw, init = ALL[name]
    d = os.path.join(str(tmp_path), f"muretar_{name}_{seed}")
    write_random_model(MuretarConfig.from_dict(raw), d, seed=seed, std=init["std"], norm_init="uniform", dtype="bfloat16")
    if not ranks_in_config:
        path = os.path.join(d, "config.json")
        cfg = json.load(open(path))
        for layer in cfg["layers"]:
            layer["mixer"].pop("decay_rank", None)
        json.dump(cfg, open(path, "w"))
    return d
