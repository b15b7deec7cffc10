"""Tiny Rorevik configurations for tests; they differ from one another in every size, constant, layer order and loop."""
from __future__ import annotations

import os

from photon_infer_amd.config import RorevikConfig
from photon_infer_amd.weights import write_random_model


def _par(left, right, ls, rs, mlp):
    return {"type": "parallel", "mixer": {"left": left, "right": right, "left_scale": ls, "right_scale": rs}, "mlp": mlp}


def _delta(mixer, mlp):
    return {"type": "channel_delta", "mixer": mixer, "mlp": mlp}


def _ff(ff, limit):
    return {"kind": "dense", "ff": ff, "limit": limit}


# A: two kv heads under four heads, values wider than keys, a quarter of a head rotated, one state-space group,
# a state narrower than its values, three taps; the delta rule with two key heads under four, two taps; the middle
# two layers run twice; the last layer has no feed-forward
_AL = dict(heads=4, kv_heads=2, dim=16, vdim=32, scale=0.3, softcap=4.0, rot={"base": 100.0, "dims": 8})
_AR = dict(heads=2, vdim=24, state=16, groups=1, norm_groups=2, conv=3)
_AD = dict(heads=4, kv_heads=2, dim=16, vdim=24, conv=2, decay_rank=8, gate_rank=12)
TINY_A = {"architecture": "Rorevik", "vocab": 300, "width": 64, "max_positions": 256, "embedding": {"scale": 8.0}, "norm": {"eps": 1e-6},
          "layers": [_par(_AL, _AR, 0.7, 1.3, _ff(96, 2.0)), _delta(_AD, _ff(80, 1.5)), _par(_AL, _AR, 1.1, 0.6, _ff(96, 0.8)), _delta(_AD, None)],
          "loop": {"start": 1, "stop": 3, "times": 2}}
TINY_A_INIT = dict(std=0.15, block_size=16)

# B: sizes the matrix-core kernels take: four heads on one kv head of 64, the whole head rotated, pages of 16; a state-space
# mixer with four norm parts and two groups; the delta rule with as many key heads as heads; no loop; a small cap
_BL = dict(heads=4, kv_heads=1, dim=64, vdim=64, scale=0.09, softcap=2.5, rot={"base": 10000.0, "dims": 64})
_BR = dict(heads=4, vdim=32, state=32, groups=2, norm_groups=4, conv=4)
_BD = dict(heads=4, kv_heads=4, dim=32, vdim=32, conv=4, decay_rank=16, gate_rank=16)
TINY_B = {"architecture": "Rorevik", "vocab": 776, "width": 256, "max_positions": 512, "embedding": {"scale": 16.0}, "norm": {"eps": 1e-5},
          "layers": [_delta(_BD, _ff(512, 7.0)), _par(_BL, _BR, 1.0, 1.0, _ff(384, 1.0))]}
TINY_B_INIT = dict(std=0.08, block_size=16)

# C: sizes that fit no fast kernel: a width that is no multiple of 8, an odd vocabulary, head sizes that are no multiples of
# 16, three kv heads, no rotation and no cap in one layer, keys wider than values, five taps, a state that is no power of
# two, three groups and three norm parts; the delta rule with one key head under three and odd ranks; one layer runs three
# times, beginning at layer 2; pages of 8
_CL = dict(heads=6, kv_heads=3, dim=24, vdim=12, scale=0.25, softcap=9.0, rot={"base": 50.0, "dims": 10})
_CL2 = dict(heads=3, kv_heads=3, dim=40, vdim=40, scale=0.2)
_CR = dict(heads=3, vdim=20, state=12, groups=3, norm_groups=3, conv=5)
_CD = dict(heads=3, kv_heads=1, dim=20, vdim=28, conv=3, decay_rank=5, gate_rank=7)
TINY_C = {"architecture": "Rorevik", "vocab": 257, "width": 100, "max_positions": 300, "embedding": {"scale": 1.0}, "norm": {"eps": 2e-6},
          "layers": [_par(_CL, _CR, 0.5, 2.0, None), _delta(_CD, _ff(36, 3.0)), _par(_CL2, _CR, 1.5, 0.25, _ff(52, 0.5))],
          "loop": {"start": 2, "stop": 3, "times": 3}}
TINY_C_INIT = dict(std=0.12, block_size=8)

# D: delta-rule layers only (no pages at all), one of them without feed-forward, the whole model run twice; one head
_DD = dict(heads=1, kv_heads=1, dim=48, vdim=80, conv=4, decay_rank=8, gate_rank=8)
_DD2 = dict(heads=5, kv_heads=5, dim=8, vdim=8, conv=1, decay_rank=8, gate_rank=16)
TINY_D = {"architecture": "Rorevik", "vocab": 512, "width": 128, "max_positions": 640, "embedding": {"scale": 11.3}, "norm": {"eps": 1e-5},
          "layers": [_delta(_DD, None), _delta(_DD2, _ff(160, 1.0))], "loop": {"start": 0, "stop": 2, "times": 2}}
TINY_D_INIT = dict(std=0.1, block_size=16)

ALL = {"A": (TINY_A, TINY_A_INIT), "B": (TINY_B, TINY_B_INIT), "C": (TINY_C, TINY_C_INIT), "D": (TINY_D, TINY_D_INIT)}


def make_model_dir(tmp_path, name: str, seed: int = 0, ranks_in_config: bool = True) -> str:
    """A model folder with random weights.  ``ranks_in_config`` False: config.json does not name the delta rule's
    low-rank sizes, which a reader then takes from the tensors' shapes."""
    import json
    raw, init = ALL[name]
    d = os.path.join(str(tmp_path), f"rorevik_{name}_{seed}")
    write_random_model(RorevikConfig.from_dict(raw), d, seed=seed, std=init["std"], norm_init="uniform", dtype="bfloat16")
    if not ranks_in_config:
        path = os.path.join(d, "config.json")
        cfg = json.load(open(path))
        for layer in cfg["layers"]:
            layer["mixer"].pop("decay_rank", None)
            layer["mixer"].pop("gate_rank", None)
        json.dump(cfg, open(path, "w"))
    return d
