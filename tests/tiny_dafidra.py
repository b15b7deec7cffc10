"""Tiny Dafidra configurations for tests; they differ from one another in every size and constant."""
from __future__ import annotations

import os

from photon_infer_amd.config import DafidraConfig
from photon_infer_amd.weights import write_random_model


def _layer(left, right, mlp):
    return {"type": "parallel", "mixer": {"left": left, "right": right}, "mlp": mlp}


def _moe(ff, experts, top, count, keep):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top, "groups": {"count": count, "keep": keep}}}


# P: values wider than keys, three expert groups of which two are kept, a window that is no multiple of a page
_PL = dict(heads=4, kv_heads=2, dim=16, vdim=32, scale=0.3, mask={"size": 24}, q_temp={"coef": 0.3, "every": 16})
_PR = dict(heads=2, dim=16, vdim=24, gate_cap=8.0)
TINY_P = {"architecture": "Dafidra", "vocab": 300, "width": 64, "norm": {"eps": 1e-6}, "residual_mult": 0.7,
          "layers": [_layer(_PL, _PR, {"kind": "dense", "ff": 96}), _layer(_PL, _PR, _moe(40, 6, 2, 3, 2))]}
TINY_P_INIT = dict(std=0.15, block_size=16)

# Q: as many kv heads as heads, one memory head, a layer without feed-forward, one expert per token in one group,
# keys wider than values, residual multiplier one, two different windows (two cache groups), a temperature period of 7
_QL = dict(heads=2, kv_heads=2, dim=32, vdim=16, scale=0.11, mask={"size": 40}, q_temp={"coef": 1.0, "every": 7})
_QL2 = dict(_QL, mask={"size": 9})
_QR = dict(heads=1, dim=40, vdim=48, gate_cap=15.0)
TINY_Q = {"architecture": "Dafidra", "vocab": 520, "width": 128, "norm": {"eps": 1e-5}, "residual_mult": 1.0,
          "layers": [_layer(_QL, _QR, None), _layer(_QL2, _QR, _moe(24, 4, 1, 1, 1)), _layer(_QL, _QR, {"kind": "dense", "ff": 200})]}
TINY_Q_INIT = dict(std=0.1, block_size=8)

# R: head sizes the matrix-core kernels take, four heads on one kv head, all groups kept, four of eight experts
_RL = dict(heads=4, kv_heads=1, dim=64, vdim=64, scale=0.09, mask={"size": 100}, q_temp={"coef": 0.45, "every": 50})
_RR = dict(heads=4, dim=32, vdim=32, gate_cap=10.0)
TINY_R = {"architecture": "Dafidra", "vocab": 776, "width": 256, "norm": {"eps": 1e-5}, "residual_mult": 0.25,
          "layers": [_layer(_RL, _RR, _moe(128, 8, 4, 4, 4)), _layer(_RL, _RR, {"kind": "dense", "ff": 512})]}
TINY_R_INIT = dict(std=0.08, block_size=16)

# S: sizes that fit no fast kernel: a width that is no multiple of 8, an odd vocabulary, head sizes that are no multiples
# of 16, three kv heads, three memory heads whose values fill two column groups unevenly, nine experts in three groups of
# which one is kept, a window shorter than a page, a temperature that changes with every position, no dense layer
_SL = dict(heads=6, kv_heads=3, dim=24, vdim=40, scale=0.25, mask={"size": 13}, q_temp={"coef": 0.2, "every": 1})
_SR = dict(heads=3, dim=20, vdim=28, gate_cap=5.0)
TINY_S = {"architecture": "Dafidra", "vocab": 257, "width": 100, "norm": {"eps": 2e-6}, "residual_mult": 0.4,
          "layers": [_layer(_SL, _SR, _moe(36, 9, 2, 3, 1)), _layer(_SL, _SR, None), _layer(_SL, _SR, _moe(20, 9, 3, 3, 1))]}
TINY_S_INIT = dict(std=0.12, block_size=16)

ALL = {"P": (TINY_P, TINY_P_INIT), "Q": (TINY_Q, TINY_Q_INIT), "R": (TINY_R, TINY_R_INIT), "S": (TINY_S, TINY_S_INIT)}


def make_model_dir(tmp_path, name: str, seed: int = 0) -> str:
    raw, init = ALL[name]
    d = os.path.join(str(tmp_path), f"dafidra_{name}_{seed}")
    write_random_model(DafidraConfig.from_dict(raw), d, seed=seed, std=init["std"], norm_init="uniform", dtype="bfloat16")
    return d
