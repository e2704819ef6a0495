"""Tiny Dokanex configurations for tests; they differ from one another in every size, constant and layer order."""
from __future__ import annotations

import os

from photon_infer_amd.config import DokanexConfig
from photon_infer_amd.weights import write_random_model


def _att(mixer, mlp):
    return {"type": "attention", "mixer": mixer, "mlp": mlp}


def _lat(mixer, mlp):
    return {"type": "latent_attention", "mixer": mixer, "mlp": mlp}


def _ff(ff):
    return {"kind": "dense", "ff": ff}


def _rot(dims, base, scaling=None):
    r = {"base": base, "dims": dims}
    if scaling is not None:
        r["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    return r


# A: a chunk that is no multiple of the page; the layer that reads layer 1's keys has a longer chunk of its own (the cache
# keeps the longer reach); values wider than keys; a latent narrower than a head's value; the last layer has no feed-forward;
# frequencies scaled over an original length that the prompts pass
_AA = dict(heads=4, kv_heads=2, dim=16, vdim=32, scale=0.4, softcap=5.0, mask={"size": 24})
_AB = dict(_AA, kv_from=1, mask={"size": 40}, scale=0.3, softcap=3.0)
_AL = dict(heads=2, dim=16, rot_dim=8, vdim=24, q_rank=20, kv_rank=24, scale=0.2, rot=_rot(8, 100.0, (4.0, 32, 8.0, 1.0)))
TINY_A = {"architecture": "Dokanex", "vocab": 300, "width": 64, "embedding": {"scale": 8.0}, "norm": {"eps": 1e-6}, "logit_softcap": 8.0,
          "layers": [_lat(_AL, _ff(96)), _att(_AA, _ff(80)), _att(_AB, _ff(96)), _lat(_AL, None)]}
TINY_A_INIT = dict(std=0.15, block_size=16)

# B: sizes the matrix-core kernels take: heads of 64 on one kv head, values as wide as keys, a latent row of 64; one attention
# layer sees every earlier position and has no cap; the logits are not capped; no frequency scaling
_BA = dict(heads=4, kv_heads=1, dim=64, vdim=64, scale=0.12, softcap=10.0, mask={"size": 32})
_BB = dict(heads=2, kv_heads=2, dim=32, vdim=32, scale=0.2)
_BL = dict(heads=4, dim=32, rot_dim=16, vdim=32, q_rank=64, kv_rank=48, scale=0.15, rot=_rot(16, 10000.0))
TINY_B = {"architecture": "Dokanex", "vocab": 776, "width": 256, "embedding": {"scale": 16.0}, "norm": {"eps": 1e-5},
          "layers": [_att(_BA, _ff(512)), _lat(_BL, _ff(384)), _att(dict(_BA, kv_from=0), _ff(256)), _att(_BB, _ff(128))]}
TINY_B_INIT = dict(std=0.08, block_size=16)

# C: sizes that fit no fast kernel: a width that is no multiple of 8, an odd vocabulary, head sizes that are no multiples of 16,
# three kv heads, a chunk shorter than a page, a chunk of one position (a token sees itself and the sink), as many kv heads as
# heads, a rotated part of six, pages of 8; the embedding is not scaled
_CA = dict(heads=6, kv_heads=3, dim=24, vdim=12, scale=0.25, softcap=9.0, mask={"size": 7})
_CB = dict(heads=3, kv_heads=3, dim=40, vdim=40, scale=0.2, softcap=2.0, mask={"size": 1})
_CL = dict(heads=3, dim=20, rot_dim=6, vdim=28, q_rank=10, kv_rank=30, scale=0.3, rot=_rot(6, 50.0, (2.0, 16, 4.0, 0.5)))
TINY_C = {"architecture": "Dokanex", "vocab": 257, "width": 100, "embedding": {"scale": 1.0}, "norm": {"eps": 2e-6}, "logit_softcap": 30.0,
          "layers": [_att(_CA, None), _lat(_CL, _ff(36)), _att(_CB, _ff(52)), _att(dict(_CA, kv_from=0, mask={"size": 5}), _ff(44))]}
TINY_C_INIT = dict(std=0.12, block_size=8)

# D: one head everywhere; a latent row wider than 256 (the wide form of the general attention kernel); an attention layer whose
# reader has no chunks at all, so that the owner's cache keeps everything
_DA = dict(heads=1, kv_heads=1, dim=48, vdim=80, scale=0.15, softcap=4.0, mask={"size": 16})
_DL = dict(heads=1, dim=24, rot_dim=16, vdim=40, q_rank=32, kv_rank=272, scale=0.08, rot=_rot(16, 1000.0, (16.0, 64, 2.0, 1.0)))
TINY_D = {"architecture": "Dokanex", "vocab": 512, "width": 128, "embedding": {"scale": 11.3}, "norm": {"eps": 1e-5}, "logit_softcap": 4.0,
          "layers": [_att(_DA, _ff(160)), _lat(_DL, _ff(96)), _att({k: v for k, v in dict(_DA, kv_from=0).items() if k != "mask"}, None)]}
TINY_D_INIT = dict(std=0.1, block_size=16)

ALL = {"A": (TINY_A, TINY_A_INIT), "B": (TINY_B, TINY_B_INIT), "C": (TINY_C, TINY_C_INIT), "D": (TINY_D, TINY_D_INIT)}


def make_model_dir(tmp_path, name: str, seed: int = 0) -> str:
    """A model folder with random weights."""
    raw, init = ALL[name]
    d = os.path.join(str(tmp_path), f"dokanex_{name}_{seed}")
    return write_random_model(DokanexConfig.from_dict(raw), d, seed=seed, std=init["std"], norm_init="uniform", dtype="bfloat16")
