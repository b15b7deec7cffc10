"""Rorevik without a GPU: configuration, run order, tensor list, cache plan, the random-weights folder, sizes taken from
tensor shapes, and the plain implementation held to invariants of its own."""
import json
import math
import os

import pytest
import torch

import plain_rorevik as P
import tiny_rorevik as TR
from photon_infer_amd.config import RorevikConfig
from photon_infer_amd.errors import ConfigError, UnsupportedModelError
from photon_infer_amd.parts import StateSpec, plan_cache
from photon_infer_amd.registry import build_model_spec, config_from_dict, load_config, registered_architectures


def test_the_architecture_is_registered_and_its_configuration_round_trips():
    assert "Rorevik" in registered_architectures()
    for name, (raw, _) in TR.ALL.items():
        cfg = config_from_dict(raw)
        assert isinstance(cfg, RorevikConfig) and cfg.vocab_size == raw["vocab"] and cfg.hidden_size == raw["width"]
        assert RorevikConfig.from_dict(cfg.to_dict()) == cfg
        assert list(cfg.run_order()) == P.run_order(raw), name


def test_run_order_repeats_the_looped_span_in_a_row():
    raw = json.loads(json.dumps(TR.TINY_A))
    assert list(config_from_dict(raw).run_order()) == [0, 1, 2, 1, 2, 3]
    raw["loop"] = {"start": 0, "stop": 4, "times": 3}
    assert list(config_from_dict(raw).run_order()) == [0, 1, 2, 3] * 3
    raw["loop"] = {"start": 3, "stop": 4, "times": 1}
    assert list(config_from_dict(raw).run_order()) == [0, 1, 2, 3]
    del raw["loop"]
    assert list(config_from_dict(raw).run_order()) == [0, 1, 2, 3]
    raw["loop"] = {"start": 2, "stop": 5, "times": 2}
    with pytest.raises(ConfigError, match="loop"):
        config_from_dict(raw)


def test_configuration_errors_name_the_key():
    raw = json.loads(json.dumps(TR.TINY_A))
    raw["layers"][0]["mixer"]["left"]["kv_heads"] = 3
    with pytest.raises(ConfigError, match="kv_heads"):
        config_from_dict(raw)
    raw = json.loads(json.dumps(TR.TINY_A))
    raw["layers"][1]["type"] = "something"
    with pytest.raises(UnsupportedModelError, match="something"):
        config_from_dict(raw)
    raw = json.loads(json.dumps(TR.TINY_A))
    raw["layers"][0]["mixer"]["left"]["rot"]["dims"] = 7
    with pytest.raises(ConfigError, match="rot.dims"):
        config_from_dict(raw)
    raw = json.loads(json.dumps(TR.TINY_A))
    del raw["embedding"]
    with pytest.raises(ConfigError, match="embedding"):
        config_from_dict(raw)
    raw = json.loads(json.dumps(TR.TINY_A))
    raw["layers"][0]["mlp"]["kind"] = "other"
    with pytest.raises(UnsupportedModelError, match="other"):
        config_from_dict(raw)


def test_tensor_list_and_cache_plan():
    spec = build_model_spec(config_from_dict(TR.TINY_A))
    names = {s.name: s.shape for s in spec.tensor_specs()}
    assert names["embed"] == (300, 64) and names["pos"] == (256, 64) and names["embed.norm"] == (64,) and names["final.norm"] == (64,)
    assert names["l0.mix.left.q"] == (64, 64) and names["l0.mix.left.k"] == (32, 64) and names["l0.mix.left.v"] == (64, 64)
    assert names["l0.mix.left.o"] == (64, 128)
    assert names["l0.mix.right.in"] == (2 * 48 + 2 * 16 + 2, 64) and names["l0.mix.right.conv"] == (48 + 32, 3)
    assert names["l0.mix.right.conv.b"] == (80,) and names["l0.mix.right.norm"] == (48,) and names["l0.mix.right.A_log"] == (2,)
    assert names["l1.mix.q"] == (32, 64) and names["l1.mix.v"] == (96, 64) and names["l1.mix.k.conv"] == (32, 2)
    assert names["l1.mix.a1"] == (8, 64) and names["l1.mix.a2"] == (64, 8) and names["l1.mix.dt_bias"] == (64,)
    assert names["l1.mix.g1"] == (12, 64) and names["l1.mix.g2"] == (96, 12) and names["l1.mix.norm"] == (24,) and names["l1.mix.b"] == (4, 64)
    assert names["l1.mlp.gate.b"] == (80,) and names["l1.mlp.down.b"] == (64,)
    assert "l3.mlp.gate" not in names and "l3.norm2" not in names and "l3.norm2" in spec.ignorable
    # every pass of a looped layer has a cache or state of its own
    assert [e.layer for e in spec.run_order] == [0, 1, 2, 1, 2, 3]
    plan = plan_cache(spec)
    assert len(plan.groups) == 1 and plan.groups[0].window is None
    assert plan.groups[0].owners == ((0, 0), (2, 0), (4, 0))
    shapes = {key: s.shape for key, s in plan.states}
    # the convolution's inputs, then S in the walks' order: [head][slice of 16 columns][4 waves][rows per lane][64 lanes]
    ssm = ((3 - 1) * 80 + 2 * 2 * 4 * 1 * 64,)
    delta = ((2 - 1) * (32 + 32 + 96) + 4 * 2 * 4 * 1 * 64,)
    assert shapes == {(0, 1): ssm, (2, 1): ssm, (4, 1): ssm, (1, 0): delta, (3, 0): delta, (5, 0): delta}
    assert all(isinstance(s, StateSpec) and s.dtype == torch.float32 for _, s in plan.states)
    # a model of delta-rule layers only keeps no pages
    assert plan_cache(build_model_spec(config_from_dict(TR.TINY_D))).groups == ()


def test_sizes_that_only_the_tensors_give(tmp_path):
    d = TR.make_model_dir(tmp_path, "C", ranks_in_config=False)
    raw = json.load(open(os.path.join(d, "config.json")))
    assert "decay_rank" not in raw["layers"][1]["mixer"]
    with pytest.raises(UnsupportedModelError, match="low-rank"):
        build_model_spec(config_from_dict(raw))
    cfg = load_config(d)
    assert (cfg.layers[1].mixer.decay_rank, cfg.layers[1].mixer.gate_rank) == (5, 7)
    assert {s.name for s in build_model_spec(cfg).tensor_specs()} == set(P.read_model_folder(d)[1])
    os.remove(os.path.join(d, "model.safetensors"))
    with pytest.raises(ConfigError, match="l1.mix.a1"):
        load_config(d)


def test_random_weights_folder_holds_the_tensor_list(tmp_path):
    for name in TR.ALL:
        d = TR.make_model_dir(tmp_path, name)
        cfg, W = P.read_model_folder(d)
        spec = build_model_spec(load_config(d))
        assert {s.name: tuple(s.shape) for s in spec.tensor_specs()} == {n: tuple(t.shape) for n, t in W.items()}
        logits = P.forward(cfg, W, [1, 2, 3, 4, 5])
        assert logits.shape == (5, cfg["vocab"]) and bool(torch.isfinite(logits).all())


# ----------------------------------------------------------------------------- the plain implementation by itself
def test_plain_convolution_is_causal_and_its_last_column_is_the_current_token():
    u = torch.randn(9, 3, dtype=torch.float64)
    w = torch.tensor([[0.0, 0.0, 1.0], [0.0, 1.0, 0.0], [1.0, 0.0, 0.0]], dtype=torch.float64)
    out = P.causal_conv(u, w)
    assert torch.equal(out[:, 0], u[:, 0])
    assert torch.equal(out[1:, 1], u[:-1, 1]) and out[0, 1] == 0
    assert torch.equal(out[2:, 2], u[:-2, 2]) and out[0, 2] == 0 and out[1, 2] == 0


def test_plain_rotation_turns_neighbouring_pairs_and_leaves_the_rest():
    x = torch.randn(2, 12, dtype=torch.float64)
    y = P.rotate_interleaved(x, 7, 4, 100.0)
    assert torch.equal(y[:, 4:], x[:, 4:])
    for i in range(2):
        a = 7 * 100.0 ** (-2.0 * i / 4)
        assert torch.allclose(y[:, 2 * i], x[:, 2 * i] * math.cos(a) - x[:, 2 * i + 1] * math.sin(a))
        assert torch.allclose(y[:, 2 * i + 1], x[:, 2 * i + 1] * math.cos(a) + x[:, 2 * i] * math.sin(a))
    assert torch.allclose((y[:, :4] ** 2).sum(), (x[:, :4] ** 2).sum())
    assert torch.equal(P.rotate_interleaved(x, 0, 12, 5.0), x)


def test_plain_capped_scores_bound_a_keys_weight():
    # one key with an enormous score: its weight against n others with score 0 is e^cap / (e^cap + n), not 1
    T, cap = 50, 3.0
    q = torch.zeros(T, 1, 4, dtype=torch.float64); k = torch.zeros(T, 1, 4, dtype=torch.float64)
    q[:, 0, 0] = 1000.0; k[5, 0, 0] = 1000.0
    v = torch.zeros(T, 1, 2, dtype=torch.float64); v[5, 0, 0] = 1.0
    out = P.attend(q, k, v, 1.0, cap)
    want = math.exp(cap) / (math.exp(cap) + (T - 1))
    assert abs(float(out[T - 1, 0, 0]) - want) < 1e-12
    assert abs(float(P.attend(q, k, v, 1.0, None)[T - 1, 0, 0]) - 1.0) < 1e-12


def test_plain_delta_rule_recalls_a_write_and_decays_by_key_channel():
    d, dv, T = 4, 3, 6
    e = torch.eye(d, dtype=torch.float64)
    k = torch.stack([e[0], e[1], e[2], e[3], e[1], e[2]]).view(T, 1, d)
    q = e[0].repeat(T, 1).view(T, 1, d)
    v = torch.arange(T * dv, dtype=torch.float64).view(T, 1, dv) + 1.0
    beta = torch.ones(T, 1, dtype=torch.float64)
    decay = torch.ones(T, 1, d, dtype=torch.float64)
    o, S = P.delta_recurrence(q, k, v, beta, decay)
    assert torch.allclose(o[:, 0], v[0, 0].repeat(T, 1))            # the read-out sees the write of its own token, and keeps it
    decay[1:4, 0, 0] = 0.5                                           # channel 0 forgets, the others do not
    o, S = P.delta_recurrence(q, k, v, beta, decay)
    assert torch.allclose(o[5, 0], v[0, 0] / 8) and torch.allclose(S[0, 3], v[3, 0])
    # the same key again overwrites: u = beta (v - S^T k)
    assert torch.allclose(S[0, 1], v[4, 0])


def test_plain_state_space_recurrence_in_closed_form():
    T = 5
    x = torch.ones(T, 1, 1, dtype=torch.float64); B = torch.ones(T, 1, 1, dtype=torch.float64); C = torch.ones(T, 1, 1, dtype=torch.float64)
    dt = torch.full((T, 1), 0.5, dtype=torch.float64)
    A_log, D = torch.tensor([math.log(2.0)], dtype=torch.float64), torch.tensor([3.0], dtype=torch.float64)
    y, S = P.state_space_recurrence(x, B, C, dt, A_log, D)
    a = math.exp(-2.0 * 0.5)
    want = [0.5 * sum(a ** j for j in range(t + 1)) + 3.0 for t in range(T)]
    assert torch.allclose(y[:, 0, 0], torch.tensor(want, dtype=torch.float64))


def test_plain_clamped_unit_clamps_before_the_activation():
    W = {"gate": torch.eye(2, dtype=torch.float64), "up": torch.eye(2, dtype=torch.float64), "down": torch.eye(2, dtype=torch.float64),
         "gate.b": torch.zeros(2, dtype=torch.float64), "up.b": torch.zeros(2, dtype=torch.float64), "down.b": torch.tensor([10.0, 20.0], dtype=torch.float64)}
    out = P.clamped_glu(torch.tensor([[50.0, -50.0]], dtype=torch.float64), W, 2.0)
    g0, g1 = 2.0, -50.0                      # the gate is clamped from above only
    assert abs(float(out[0, 0]) - (g0 / (1 + math.exp(-1.702 * g0)) * 3.0 + 10.0)) < 1e-12
    assert abs(float(out[0, 1]) - (g1 / (1 + math.exp(-1.702 * g1)) * (-2.0 + 1.0) + 20.0)) < 1e-12
