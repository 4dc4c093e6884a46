"""Fedovik without a GPU: its configuration (keys, run order, tensors, errors) and the plain implementation's
mechanisms against cases whose answers are known."""
import copy
import math

import pytest
import torch

import plain_fedovik as pf
from fedovik_helpers import CONFIGS, attention_layer, make_weights, memory_layer, pair_layer
from vt_transformer_amd.config import ConfigError, config_from_dict
from vt_transformer_amd.weights.random_init import declared_tensors

DT = torch.float64


def test_run_order_re_entry_and_offsets():
    spec = config_from_dict(copy.deepcopy(CONFIGS["A"])).to_spec()
    assert [(e.layer, e.offset_row, e.inject) for e in spec.schedule] == [
        (0, 0, True), (1, None, False), (0, 1, True), (1, None, False), (0, 2, True), (1, None, False), (2, None, False),
        (3, None, False)]
    assert spec.stream_offsets == {"name": "loop.step", "rows": 3} and spec.stream_inject == {"name": "loop.in"}
    assert pf.layer_runs(CONFIGS["A"]) == [(e.layer, e.offset_row) for e in spec.schedule]
    spec = config_from_dict(copy.deepcopy(CONFIGS["B"])).to_spec()
    assert [(e.layer, e.offset_row, e.inject) for e in spec.schedule] == [(i, None, False) for i in range(5)]
    assert spec.stream_offsets is None and spec.stream_inject is None
    spec = config_from_dict(copy.deepcopy(CONFIGS["C"])).to_spec()
    assert [(e.layer, e.offset_row, e.inject) for e in spec.schedule] == [(0, None, False), (1, 0, True), (2, None, False)]


def test_parts_and_tensors_follow_the_configuration():
    cfg = config_from_dict(copy.deepcopy(CONFIGS["A"]))
    spec = cfg.to_spec()
    assert [ls.block.kind for ls in spec.layers] == ["parallel"] * 4
    assert [ls.mixer.kind for ls in spec.layers] == ["mixer_pair", "matrix_memory", "masked_attention", "matrix_memory"]
    assert [ls.feed_forward is not None for ls in spec.layers] == [True, True, True, False]
    assert spec.layers[0].feed_forward.params["activation"] == "relu"
    assert spec.layers[0].norms["input"].kind == "layernorm" and spec.final_norm.kind == "layernorm"
    assert spec.head.params["tied_to"] == "embed"
    pair = spec.layers[0].mixer.params
    left, right = pair["left"].params, pair["right"].params
    assert (pair["left_scale"], pair["right_scale"]) == (0.8, 1.3)
    assert (left["window"], left["qk_gain"], left["distance_log"], left["position"], left["unit_rms_eps"]) == (12, True, True, None, 1e-5)
    assert (right["decay"], right["decay_rank"], right["gate_rank"], right["gate_act"], right["conv_taps"]) == ("channel", 6, 5, "sigmoid", 3)
    att = spec.layers[2].mixer.params
    assert (att["weights"], att["score_shift"], att["out_gate"], att["o_bias"], att["rot_pairs"]) == ("sigmoid", True, True, True, "neighbours")
    assert att["position"].params == {"theta": 10000.0, "dim": 8, "scaling": None}
    mem = spec.layers[1].mixer.params
    assert (mem["num_heads"], mem["key_dim"], mem["value_dim"], mem["gate_cap"]) == (2, 16, 24, 12.0)
    t = declared_tensors(cfg)
    assert t["loop.step"].shape == (3, 96) and t["loop.in"].shape == (96, 192) and t["embed"].shape == (203, 96)
    assert t["final.norm.b"].shape == (96,) and t["l0.norm1.b"].shape == (96,) and "l0.norm2" not in t
    assert t["l0.mix.left.q.b"].shape == (4 * 16,) and t["l0.mix.left.q.norm"].shape == (16,) and t["l0.mix.left.r2"].shape == (4,)
    assert t["l0.mix.left.o"].shape == (96, 4 * 24) and "l0.mix.left.o.b" not in t and "l0.mix.left.g" not in t
    assert t["l0.mix.right.q.conv"].shape == (16, 3) and t["l0.mix.right.v.conv"].shape == (2 * 24, 3)
    assert t["l0.mix.right.b"].shape == (2, 96) and t["l0.mix.right.dt_bias"].shape == (2 * 16,)
    assert t["l0.mix.right.a1"].shape == (6, 96) and t["l0.mix.right.a2"].shape == (32, 6)
    assert t["l0.mix.right.g1"].shape == (5, 96) and t["l0.mix.right.g2"].shape == (48, 5) and t["l0.mix.right.norm"].shape == (24,)
    assert t["l1.mix.i"].shape == (2, 96) and t["l1.mix.f.b"].shape == (2,) and t["l1.mix.norm"].shape == (2 * 24,)
    assert t["l2.mix.pb"].shape == (4,) and t["l2.mix.g"].shape == (4 * 48, 96) and t["l2.mix.o.b"].shape == (96,)
    assert "l3.mlp.gate" not in t and t["l0.mlp.down"].shape == (96, 80)
    assert t["head"].optional and set(make_weights(CONFIGS["A"], 0)) == {k for k, d in t.items() if not d.optional}
    assert config_from_dict(cfg.to_dict()).to_dict() == cfg.to_dict()


def test_low_rank_sizes_come_from_the_tensors():
    raw = copy.deepcopy(CONFIGS["C"])
    for key in ("a_rank", "g_rank"):
        raw["layers"][1]["mixer"]["right"].pop(key)
    cfg = config_from_dict(raw)
    with pytest.raises(ConfigError, match="low-rank"):
        cfg.to_spec()
    cfg.take_tensor_shapes({"l1.mix.right.a1": (9, 64), "l1.mix.right.g1": (2, 64)})
    right = cfg.to_spec().layers[1].mixer.params["right"].params
    assert (right["decay_rank"], right["gate_rank"]) == (9, 2)
    said = config_from_dict(copy.deepcopy(CONFIGS["C"]))
    with pytest.raises(ConfigError, match="a_rank"):
        said.take_tensor_shapes({"l1.mix.right.a1": (9, 64)})


@pytest.mark.parametrize("change,text", [
    (lambda c: c["layers"][0].update(type="conv"), "mixer type"),
    (lambda c: c["layers"][2]["mixer"].update(kv_heads=3), "multiple"),
    (lambda c: c["layers"][2]["mixer"]["rot"].update(dims=34), "dims"),
    (lambda c: c["layers"][2]["mixer"].pop("scale"), "scale"),
    (lambda c: c["layers"][0]["mixer"].pop("right"), "right"),
    (lambda c: c["layers"][0]["mixer"]["left"]["mask"].update(size=0), "mask.size"),
    (lambda c: c["layers"][1]["mixer"].update(gate_cap=-1.0), "gate_cap"),
    (lambda c: c["loop"].update(stop=9), "loop"),
    (lambda c: c.pop("norm"), "norm"),
    (lambda c: c["layers"][0]["mlp"].update(kind="routed"), "kind"),
])
def test_configuration_errors(change, text):
    cfg = copy.deepcopy(CONFIGS["A"])
    change(cfg)
    with pytest.raises(ConfigError, match=text):
        config_from_dict(cfg)


# ---------------------------------------------------------------------------
# the plain mechanisms on cases with known answers
# ---------------------------------------------------------------------------
def test_layer_norm_known_values():
    x = torch.tensor([[1.0, 2.0, 3.0, 6.0]], dtype=DT)
    out = pf.layer_norm(x, torch.tensor([1.0, 1.0, 2.0, 1.0], dtype=DT), torch.tensor([0.0, 0.5, 0.0, 0.0], dtype=DT), 0.0)
    sd = math.sqrt((4 + 1 + 0 + 9) / 4)
    assert torch.allclose(out, torch.tensor([[-2 / sd, -1 / sd + 0.5, 0.0, 3 / sd]], dtype=DT))


def test_neighbouring_pairs_turn_together():
    x = torch.zeros(3, 1, 6, dtype=DT)
    x[:, 0, 0] = 1.0          # pair (0, 1) turns by position * 1
    x[:, 0, 3] = 1.0          # pair (2, 3) by position * base^(-1/2)
    x[:, 0, 4] = 7.0          # beyond the rotated part
    out = pf.rotate_neighbours(x, torch.arange(3), 4, 100.0)
    for p in range(3):
        assert torch.allclose(out[p, 0], torch.tensor([math.cos(p), math.sin(p), -math.sin(p * 0.1), math.cos(p * 0.1), 7.0, 0.0], dtype=DT))
    # a score depends on the distance only
    g = torch.Generator().manual_seed(0)
    q, k = torch.randn(1, 1, 8, generator=g, dtype=DT), torch.randn(1, 1, 8, generator=g, dtype=DT)
    def score(i, j):
        return float(pf.rotate_neighbours(q, torch.tensor([i]), 8, 50.0)[0, 0] @ pf.rotate_neighbours(k, torch.tensor([j]), 8, 50.0)[0, 0])
    assert abs(score(9, 4) - score(105, 100)) < 1e-9 and abs(score(9, 4) - score(9, 5)) > 1e-3


def test_sigmoid_weights_are_not_normalized():
    t = 5
    q, k = torch.zeros(t, 2, 4, dtype=DT), torch.zeros(t, 1, 4, dtype=DT)
    v = torch.arange(t, dtype=DT).reshape(t, 1, 1) + 1.0
    out = pf.sigmoid_attention(q, k, v, torch.arange(t), 1.0, torch.tensor([0.0, math.log(3.0)], dtype=DT))
    # every seen key weighs sigmoid(shift): 1/2 for head 0, 3/4 for head 1; position i sees values 1 .. i + 1
    for i in range(t):
        total = (i + 1) * (i + 2) / 2
        assert abs(float(out[i, 0, 0]) - 0.5 * total) < 1e-12 and abs(float(out[i, 1, 0]) - 0.75 * total) < 1e-12


def test_window_and_distance_bias():
    t = 9
    q, k = torch.zeros(t, 1, 2, dtype=DT), torch.zeros(t, 1, 2, dtype=DT)
    v = torch.arange(t, dtype=DT).reshape(t, 1, 1)
    # no bias: the mean of the last `window` values
    out = pf.window_attention(q, k, v, torch.arange(t), 1.0, 3, torch.zeros(1, dtype=DT), torch.ones(1, dtype=DT))
    assert abs(float(out[8, 0, 0]) - 7.0) < 1e-12 and abs(float(out[1, 0, 0]) - 0.5) < 1e-12
    # r1 = 1, r2 = 1: weights proportional to 1 / (1 + distance)
    out = pf.window_attention(q, k, v, torch.arange(t), 1.0, 3, torch.ones(1, dtype=DT), torch.ones(1, dtype=DT))
    w = [1.0, 1 / 2, 1 / 3]
    assert abs(float(out[8, 0, 0]) - (8 * w[0] + 7 * w[1] + 6 * w[2]) / sum(w)) < 1e-12
    # a window of one position returns the position's own value
    out = pf.window_attention(q, k, v, torch.arange(t), 1.0, 1, torch.ones(1, dtype=DT), torch.ones(1, dtype=DT))
    assert torch.allclose(out[:, 0, 0], torch.arange(t, dtype=DT))


def test_causal_convolution():
    x = torch.tensor([[1.0], [2.0], [3.0]], dtype=DT)
    out = pf.causal_conv(x, torch.tensor([[100.0, 10.0, 1.0]], dtype=DT))
    assert out[:, 0].tolist() == [1.0, 12.0, 123.0]


def test_delta_rule_with_channel_decay():
    # one head, keys along the axes: with beta 1 and no decay a written value is read back exactly, and written over
    e0, e1 = torch.tensor([1.0, 0.0], dtype=DT), torch.tensor([0.0, 1.0], dtype=DT)
    k = torch.stack([e0, e1, e0, e0]).reshape(4, 1, 2)
    q = torch.stack([e0, e0, e0, e1]).reshape(4, 1, 2)
    v = torch.tensor([[5.0], [7.0], [9.0], [11.0]], dtype=DT).reshape(4, 1, 1)
    ones = torch.ones(4, 1, 2, dtype=DT)
    out = pf.channel_delta_rule(q, k, v, torch.ones(4, 1, dtype=DT), ones)
    assert out[:, 0, 0].tolist() == [5.0, 5.0, 9.0, 7.0]
    # a decay on channel 0 alone shrinks what lies under key e0 and leaves key e1's
    g = ones.clone()
    g[:, 0, 0] = 0.5
    out = pf.channel_delta_rule(q, k, v, torch.zeros(4, 1, dtype=DT).fill_(1.0), g)
    assert out[1, 0, 0] == 2.5 and out[3, 0, 0] == 7.0
    # beta 1/2 moves the stored value half of the way
    out = pf.channel_delta_rule(q[:3], torch.stack([e0, e0, e0]).reshape(3, 1, 2), v[:3], torch.full((3, 1), 0.5, dtype=DT), ones[:3])
    assert out[:, 0, 0].tolist() == [2.5, 2.5 + 0.5 * (7 - 2.5), 4.75 + 0.5 * (9 - 4.75)]


def test_matrix_memory_known_values():
    # forget gate fully open (f = 0), input gate i = 0: m stays 0, S and n add up, o = sum(k.q v) / max(|sum k.q|, 1)
    k = torch.tensor([[1.0, 0.0], [1.0, 0.0], [0.0, 1.0]], dtype=DT).reshape(3, 1, 2)
    q = torch.tensor([[1.0, 0.0]] * 3, dtype=DT).reshape(3, 1, 2)
    v = torch.tensor([[2.0], [4.0], [8.0]], dtype=DT).reshape(3, 1, 1)
    zero = torch.zeros(3, 1, dtype=DT)
    out = pf.matrix_memory(q, k, v, zero, zero)
    assert torch.allclose(out[:, 0, 0], torch.tensor([2.0, 3.0, 3.0], dtype=DT), atol=1e-5)
    # a large input gate takes the maximum along: the state is scaled, the result is not
    big = torch.full((3, 1), 9.0, dtype=DT)
    out_big = pf.matrix_memory(q, k, v, big, zero)
    assert torch.allclose(out_big[0], out[0], atol=1e-5)
    # a closed forget gate (f very negative) leaves only the newest token
    out = pf.matrix_memory(q, torch.tensor([[1.0, 0.0]] * 3, dtype=DT).reshape(3, 1, 2), v, zero, torch.full((3, 1), -40.0, dtype=DT))
    assert torch.allclose(out[:, 0, 0], torch.tensor([2.0, 4.0, 8.0], dtype=DT), atol=1e-4)
    # the maximum starts at 0, not at minus infinity: a first token with i = -5 is divided by max(|n.q|, e^0) = 1
    out = pf.matrix_memory(q[:1], k[:1], v[:1], torch.full((1, 1), -5.0, dtype=DT), zero[:1])
    assert abs(float(out[0, 0, 0]) - 2.0 * math.exp(-5.0)) < 1e-6


def test_whole_model_prefix_property_and_layers():
    """Logits at a position depend on the tokens up to it only, every mechanism has an effect, and the stream after
    every layer run is handed out."""
    cfg = copy.deepcopy(CONFIGS["A"])
    w = {k: v.float() for k, v in make_weights(cfg, 3).items()}
    ids = torch.randint(0, cfg["vocab"], (40,), generator=torch.Generator().manual_seed(1)).tolist()
    streams = []
    full = pf.forward(cfg, w, ids, streams)
    assert len(streams) == len(pf.layer_runs(cfg)) == 8 and streams[0].shape == (40, 96)
    assert torch.allclose(pf.forward(cfg, w, ids[:17]), full[:17], atol=1e-9)
    for name in ("l0.mix.left.r1", "l0.mix.right.dt_bias", "l2.mix.pb", "l1.mix.f.b", "loop.in", "loop.step", "l0.norm1.b",
                 "l0.mix.right.g2", "l0.mix.left.k.norm", "l2.mix.o.b", "final.norm.b"):
        changed = dict(w)
        # (a ramp, not a constant: the norms take a constant over the channels off again)
        changed[name] = w[name] + 0.25 * torch.linspace(-1.0, 1.0, w[name].numel()).reshape(w[name].shape)
        assert float((pf.forward(cfg, changed, ids) - full).abs().max()) > 1e-4, name
    assert pf.greedy(cfg, w, ids[:5], 3) == pf.greedy(cfg, w, ids[:5], 3)


def test_random_model_from_the_command_line(tmp_path):
    """`--write-random-model` on a Fedovik config.json that says its low-rank sizes: every declared tensor is written,
    the folder loads back into the same configuration, and the distance factor r2 is drawn around 1 (positive, as the
    logarithm wants it)."""
    import json
    import os
    import subprocess
    import sys
    from vt_transformer_amd.config import load_config
    from vt_transformer_amd.weights import WeightStore
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    cfg_path = tmp_path / "c.json"
    cfg_path.write_text(json.dumps(CONFIGS["C"]))
    out = tmp_path / "m"
    r = subprocess.run([sys.executable, "-m", "vt_transformer_amd", "--write-random-model", str(out), "--config", str(cfg_path),
                        "--seed", "4"], capture_output=True, text=True, env=dict(os.environ, PYTHONPATH=root), timeout=300)
    assert r.returncode == 0, r.stderr
    cfg = load_config(str(out))
    assert cfg.to_dict() == config_from_dict(copy.deepcopy(CONFIGS["C"])).to_dict()
    store = WeightStore(str(out))
    want = {k for k, d in declared_tensors(cfg).items() if not d.optional}
    assert set(store.names()) == want
    _, w = pf.read_folder(str(out))
    assert float(w["l1.mix.left.r2"].min()) > 0.5
    assert torch.isfinite(pf.forward(cfg.to_dict(), w, [3, 1, 4, 1, 5, 9, 2, 6])).all()
