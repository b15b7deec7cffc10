"""Dafidra without a GPU: its configuration and tensor list, what its cache must hold, the
random-weights folder, and the plain implementation's own invariants."""
import json
import os

import pytest
import torch

import plain_dafidra as P
import tiny_dafidra as TD
from photon_infer_amd.config import DafidraConfig
from photon_infer_amd.errors import ConfigError, UnsupportedModelError
from photon_infer_amd.parts import plan_cache
from photon_infer_amd.parts.base import StateSpec
from photon_infer_amd.registry import build_model_spec, config_from_dict, load_config


@pytest.mark.parametrize("name", list(TD.ALL))
def test_configuration_round_trip_and_registry(name):
    raw = TD.ALL[name][0]
    cfg = config_from_dict(raw)
    assert isinstance(cfg, DafidraConfig) and cfg.to_dict() == raw
    assert cfg.vocab_size == raw["vocab"] and len(cfg.layers) == len(raw["layers"])


def test_configuration_errors_name_the_key():
    raw = json.loads(json.dumps(TD.TINY_P))
    del raw["layers"][1]["mixer"]["left"]["scale"]
    with pytest.raises(ConfigError, match=r"layers\[1\].*scale"):
        config_from_dict(raw)
    raw = json.loads(json.dumps(TD.TINY_P))
    raw["layers"][0]["type"] = "serial"
    with pytest.raises(UnsupportedModelError, match="serial"):
        config_from_dict(raw)
    raw = json.loads(json.dumps(TD.TINY_P))
    raw["layers"][1]["mlp"]["router"]["top"] = 7
    with pytest.raises(ConfigError):
        config_from_dict(raw)


def test_tensor_list_cache_groups_and_states():
    spec = build_model_spec(config_from_dict(TD.TINY_Q))
    names = {s.name: s.shape for s in spec.tensor_specs()}
    assert names["embed"] == (520, 128) and names["head"] == (520, 128) and names["final.norm"] == (128,)
    assert names["l0.mix.left.q"] == (64, 128) and names["l0.mix.left.q.norm"] == (64,) and names["l0.mix.left.v"] == (32, 128)
    assert names["l0.mix.left.g"] == (2, 128) and names["l0.mix.left.sink"] == (2,) and names["l0.mix.left.out"] == (128,)
    assert names["l2.mix.right.i.b"] == (1,) and names["l1.mix.right.g"] == (48, 128) and names["l1.mlp.e3.down"] == (128, 24)
    assert "l0.norm2" not in names and "l0.mlp.gate" not in names and "l1.norm2" in names and names["l1.mlp.router"] == (4, 128)
    plan = plan_cache(spec)
    assert [g.window for g in plan.groups] == [9, 40]                   # two windows: two block tables
    assert [len(g.owners) for g in plan.groups] == [1, 2]
    assert len(plan.states) == 3 and all(isinstance(s, StateSpec) and s.dtype == torch.float32 for _, s in plan.states)
    # keys [kv heads, page, dim], values transposed [kv heads, vdim, page]
    k, v = plan.groups[1].tensors[0]
    assert k.page_shape(8) == (2, 8, 32) and v.page_shape(8) == (2, 16, 8)


def test_random_weights_folder_loads_back(tmp_path):
    d = TD.make_model_dir(tmp_path, "P", seed=1)
    cfg = load_config(d)
    assert cfg.to_dict() == TD.TINY_P
    raw, W = P.read_model_folder(d)
    assert set(W) == {s.name for s in build_model_spec(cfg).tensor_specs()}
    assert float(W["l0.norm1"].float().abs().max()) <= 0.5 and float(W["l0.mix.left.out"].float().min()) >= 0.5


def test_plain_recurrence_does_not_depend_on_the_running_maximum():
    """The cell with its running maximum equals the same recurrence in plain (unstabilised) arithmetic as long as the
    denominator's floor exp(-m) is expressed in the same units: a check of the plain implementation by itself."""
    torch.manual_seed(0)
    H, d, dv, T, D = 1, 6, 5, 30, 12
    W = {n: torch.randn(s, dtype=torch.float64) * 0.4 for n, s in
         dict(q=(d, D), k=(d, D), v=(dv, D), g=(dv, D), i=(H, D), f=(H, D), o=(D, dv)).items()}
    W.update({"i.b": torch.zeros(H, dtype=torch.float64), "f.b": torch.ones(H, dtype=torch.float64), "norm": torch.ones(dv, dtype=torch.float64)})
    h = torch.randn(T, D, dtype=torch.float64)
    c = dict(heads=H, dim=d, vdim=dv, gate_cap=5.0)
    got = P.matrix_memory(h, W, c, 1e-6)
    q, k, v = (h @ W["q"].T) * d ** -0.5, h @ W["k"].T, h @ W["v"].T
    S, n, out = torch.zeros(d, dv, dtype=torch.float64), torch.zeros(d, dtype=torch.float64), []
    import math
    m = 0.0
    for t in range(T):
        i_t = 5.0 * math.tanh(float(h[t] @ W["i"][0]) / 5.0)
        f_t = P.log_sigmoid(5.0 * math.tanh((float(h[t] @ W["f"][0]) + 1.0) / 5.0))
        m = max(f_t + m, i_t)
        S = math.exp(f_t) * S + math.exp(i_t) * torch.outer(k[t], v[t])       # true scale: S_true = exp(m) S_stabilised
        n = math.exp(f_t) * n + math.exp(i_t) * k[t]
        o = (S.T @ q[t]) / (max(abs(float(n @ q[t])), 1.0) + 1e-6 * math.exp(m))
        o = o / math.sqrt(float((o * o).sum()) / dv + 1e-6)
        out.append(o * torch.sigmoid(h[t] @ W["g"].T))
    want = torch.stack(out) @ W["o"].T
    assert float((got - want).abs().max()) < 1e-9


def test_plain_routing_examples():
    z = torch.tensor([0.0, 3.0, 2.9, 0.1, 2.0, 1.0], dtype=torch.float64)
    assert [e for e, _ in P.route(z, 2, 1, 1)] == [1, 2]
    assert [e for e, _ in P.route(z, 2, 3, 1)] == [1, 0]            # only the best group (experts 0, 1) may be chosen
    assert [e for e, _ in P.route(z, 3, 3, 2)] == [1, 2, 3]         # groups (0,1) and (2,3) are kept
    w = P.route(z, 2, 1, 1)
    s = torch.softmax(z, -1)
    assert abs(w[0][1] - float(s[1])) < 1e-12 and abs(sum(x for _, x in w) - float(s[1] + s[2])) < 1e-12   # not renormalised


def test_plain_attention_sees_exactly_its_window():
    """Moving a key that lies outside the window changes nothing; moving the oldest key inside it does."""
    torch.manual_seed(1)
    c = dict(heads=2, kv_heads=1, dim=4, vdim=3, scale=0.5, mask={"size": 5}, q_temp={"coef": 0.5, "every": 3})
    D = 8
    W = {n: torch.randn(s, dtype=torch.float64) for n, s in dict(q=(8, D), k=(4, D), v=(3, D), g=(2, D), o=(D, 6)).items()}
    W.update({"q.norm": torch.ones(8, dtype=torch.float64), "k.norm": torch.ones(4, dtype=torch.float64), "sink": torch.zeros(2, dtype=torch.float64)})
    h = torch.randn(12, D, dtype=torch.float64)
    base = P.sink_window_attention(h, W, c, 1e-6)[-1]
    far, edge = h.clone(), h.clone()
    far[11 - 5] += 1.0
    edge[11 - 4] += 1.0
    assert float((P.sink_window_attention(far, W, c, 1e-6)[-1] - base).abs().max()) == 0.0
    assert float((P.sink_window_attention(edge, W, c, 1e-6)[-1] - base).abs().max()) > 1e-6
