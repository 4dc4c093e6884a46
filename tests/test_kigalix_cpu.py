"""Kigalix without a GPU: the configuration (keys, parts, tensors, errors) and the plain implementation's mechanisms on
cases with known answers."""
import copy
import math

import pytest
import torch

import plain_kigalix as pk
from kigalix_helpers import CFG_A, CFG_B, CFG_C, CFG_D, delta_layer, dense, latent_layer, make_weights, moe, write_model


def spec_of(cfg):
    from vt_transformer_amd.config import config_from_dict
    return config_from_dict(copy.deepcopy(cfg)).to_spec()


def test_configuration_becomes_parts():
    from vt_transformer_amd.config import KigalixConfig, architectures, config_from_dict
    assert "Kigalix" in architectures()
    cfg = config_from_dict(copy.deepcopy(CFG_A))
    assert isinstance(cfg, KigalixConfig) and cfg.vocab_size == 211
    spec = cfg.to_spec()
    assert spec.streams == 3 and [e.layer for e in spec.schedule] == list(range(5))
    assert [ls.mixer.kind for ls in spec.layers] == ["general_delta", "latent_attention", "latent_attention", "general_delta",
                                                     "latent_attention"]
    assert all(ls.block.kind == "hyper" and ls.block.params == {"streams": 3, "learned_streams": True, "token_shift": True,
                                                                "residual_gate": True} for ls in spec.layers)
    d = spec.layers[0].mixer.params
    assert (d["num_heads"], d["key_dim"], d["decay_rank"]) == (3, 20, 12)
    assert d["decay_scale"] == math.exp(-0.5) and d["key_eps"] == 1e-6
    lat = spec.layers[1].mixer.params
    assert (lat["num_heads"], lat["plain_dim"], lat["rot_dim"], lat["value_dim"], lat["rank"]) == (4, 16, 16, 24, 32)
    assert lat["rot_pairs"] == "neighbours" and not lat["out_gate"] and not lat["sink"] and lat["window"] == 0
    assert lat["position"].params == {"theta": 10000.0, "dim": 16, "scaling": None}
    two = spec.layers[2].mixer.params
    assert two["out_gate"] and two["position"].params["scaling"] == {"factor": 4.0, "original": 64.0, "fast": 16.0, "slow": 2.0}
    ex = spec.layers[0].feed_forward
    assert ex.kind == "expert_mixture" and (ex.params["num_experts"], ex.params["top"], ex.params["intermediate_size"]) == (5, 2, 40)
    assert ex.params["score"] == "sigmoid" and ex.params["weight_on"] == "input" and not ex.params["renormalize"]
    ff = spec.layers[1].feed_forward
    assert ff.kind == "gated_mlp" and ff.params["activation"] == "gelu_tanh" and ff.params["intermediate_size"] == 80
    assert spec.layers[2].feed_forward is None and "post_mixer" not in spec.layers[2].norms
    assert all(n.params["unit_offset"] for ls in spec.layers for n in ls.norms.values()) and spec.final_norm.params["unit_offset"]
    assert config_from_dict(cfg.to_dict()).to_spec() == spec
    # no 'streams': one stream without learned numbers
    c = spec_of(CFG_C)
    assert c.streams == 1 and c.layers[0].block.params["learned_streams"] is False
    assert spec_of(CFG_B).layers[2].mixer.params["position"] is None        # nothing to rotate


def test_declared_tensors():
    from vt_transformer_amd.config import config_from_dict
    from vt_transformer_amd.weights.random_init import declared_tensors
    t = declared_tensors(config_from_dict(copy.deepcopy(CFG_A)))
    assert t["embed"].shape == (211, 96) and t["head"].shape == (211, 96) and t["final.norm"].shape == (96,)
    assert t["l0.mix.r"].shape == (60, 96) and t["l0.mix.w1"].shape == (12, 96) and t["l0.mix.w2"].shape == (60, 12)
    assert t["l0.mix.w0"].shape == (60,) and t["l0.mix.a.b"].shape == (60,) and t["l0.mix.norm"].shape == (60,)
    assert t["l0.mix.o"].shape == (96, 60) and t["l0.mix.g"].shape == (60, 96)
    assert t["l0.mlp.router"].shape == (5, 96) and t["l0.mlp.router"].role == "matrix32"
    assert t["l0.mlp.e4.gate"].shape == (40, 96) and t["l0.mlp.e0.down"].shape == (96, 40) and "l0.mlp.e5.up" not in t
    assert t["l1.mix.q"].shape == (4 * 32, 96) and t["l1.mix.dkv"].shape == (48, 96) and t["l1.mix.dkv.norm"].shape == (32,)
    assert t["l1.mix.uk"].shape == (64, 32) and t["l1.mix.uv"].shape == (96, 32) and "l1.mix.g" not in t
    # a layer without a feed-forward: the second sublayer's tensors are tolerated in a checkpoint, never required
    assert t["l2.mix.g"].shape == (30, 96) and all(t[n].optional for n in ("l2.norm2", "l2.hc2.in", "l2.hc2.mix", "l2.rg2", "l2.rg2.b"))
    assert not t["l2.hc1.in"].optional and not t["l1.hc2.in"].optional and not t["l1.norm2"].optional
    from vt_transformer_amd.weights.loader import check_tensors
    for idle in (False, True):
        held = {n: (w.dtype, tuple(w.shape)) for n, w in make_weights(CFG_A, 1, idle=idle).items()}
        assert ("l2.norm2" in held) == idle
        check_tensors(t, held, "here")
    assert t["l1.hc1.in"].shape == (3,) and t["l1.hc2.out"].shape == (3,) and t["l1.hc1.mix"].shape == (3, 3)
    assert t["l1.shift"].shape == (96,) and t["l1.rg1"].shape == (96, 96) and t["l1.rg2.b"].shape == (96,)
    c = declared_tensors(config_from_dict(copy.deepcopy(CFG_C)))
    assert not any(".hc" in n for n in c) and "l0.rg1" in c and "l0.shift" in c


def test_the_decay_projections_size_comes_from_its_tensor(tmp_path):
    from vt_transformer_amd.config import ConfigError, load_config
    from vt_transformer_amd.weights.safetensors_io import WeightStore
    folder = write_model(copy.deepcopy(CFG_A), str(tmp_path / "m"), seed=1)
    cfg = load_config(folder)
    assert "decay_rank" not in cfg.layers[0]["mixer"]
    store = WeightStore(folder)
    shapes = {n: tuple(store.info(n)[1]) for n in store.names()}
    store.close()
    cfg.take_tensor_shapes(shapes)
    assert cfg.layers[0]["mixer"]["decay_rank"] == 12 and cfg.layers[3]["mixer"]["decay_rank"] == 4
    assert cfg.to_spec().layers[3].mixer.params["decay_rank"] == 4
    said = load_config(write_model(copy.deepcopy(CFG_A), str(tmp_path / "k"), seed=1, keep_rank=True))
    said.layers[0]["mixer"]["decay_rank"] = 13
    with pytest.raises(ConfigError, match="decay_rank"):
        said.take_tensor_shapes(shapes)


def test_configuration_errors():
    from vt_transformer_amd.config import ConfigError, config_from_dict

    def broken(change):
        cfg = copy.deepcopy(CFG_A)
        change(cfg)
        return cfg
    cases = [
        (lambda c: c["layers"][0].update(type="attention"), "not known"),
        (lambda c: c["layers"][1]["mixer"].pop("kv_rank"), "kv_rank"),
        (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=7), "dims"),
        (lambda c: c["layers"][0]["mlp"]["router"].update(top=6), "top 6 of 5"),
        (lambda c: c["layers"][1]["mlp"].update(kind="sparse"), "not known"),
        (lambda c: c.update(streams=0), "streams"),
        (lambda c: c.pop("norm"), "norm"),
        (lambda c: c["layers"][2]["mixer"]["rot"]["scaling"].pop("slow"), "slow"),
    ]
    for change, text in cases:
        with pytest.raises(ConfigError, match=text):
            config_from_dict(broken(change))


def test_random_weights_of_a_kigalix_configuration(tmp_path):
    """The framework's own random model: stream mixing around the identity, routers in float32 roles, readable again."""
    from vt_transformer_amd.config import config_from_dict, load_config
    from vt_transformer_amd.weights import write_random_model
    folder = write_random_model(config_from_dict(copy.deepcopy(CFG_D)), str(tmp_path / "r"), seed=3)
    cfg, w = pk.read_folder(folder)
    assert load_config(folder).to_dict() == config_from_dict(copy.deepcopy(CFG_D)).to_dict()
    mix = w["l0.hc1.mix"].double()
    assert mix.shape == (4, 4) and float((mix - torch.eye(4, dtype=torch.float64)).abs().max()) < 0.2
    assert abs(float(w["l0.norm1"].double().mean())) < 0.05          # the gain less one
    logits = pk.forward(cfg, w, [1, 2, 3, 4, 5])
    assert logits.shape == (5, 150) and bool(torch.isfinite(logits).all())


# ---------------------------------------------------------------------------
# the plain mechanisms on cases with known answers
# ---------------------------------------------------------------------------
def test_token_shift_blends_with_the_token_before():
    h = torch.tensor([[1.0, 2.0], [3.0, 6.0], [5.0, 10.0]], dtype=torch.float64)
    out = pk.token_shift(h, torch.tensor([0.0, 0.5], dtype=torch.float64))
    assert torch.equal(out, torch.tensor([[1.0, 1.0], [3.0, 4.0], [5.0, 8.0]], dtype=torch.float64))
    assert torch.equal(pk.token_shift(h, torch.ones(2, dtype=torch.float64))[1:], h[:-1])


def test_gelu_in_its_sigmoid_form():
    z = torch.linspace(-6, 6, 101, dtype=torch.float64)
    alpha = 2.0 * math.sqrt(2.0 / math.pi)
    assert torch.allclose(pk.gelu_tanh(z), z * torch.sigmoid(alpha * z * (1.0 + 0.044715 * z * z)), atol=1e-14)
    assert abs(float(pk.gelu_tanh(torch.tensor(1.0, dtype=torch.float64))) - 0.8411919906082768) < 1e-12


def test_rotation_of_neighbours_and_stretched_frequencies():
    x = torch.zeros(3, 6, dtype=torch.float64)
    x[:, 0] = 1.0
    x[:, 5] = 7.0
    out = pk.rotate_neighbours(x, torch.arange(3), 4, 100.0, None)
    assert torch.allclose(out[:, 0], torch.cos(torch.arange(3, dtype=torch.float64)))
    assert torch.allclose(out[:, 1], torch.sin(torch.arange(3, dtype=torch.float64)))
    assert torch.equal(out[:, 2:], x[:, 2:])                  # a pair of zeros stays, what lies behind `dims` passes
    # with scaling: the fastest pair keeps its frequency, the slowest is divided by the factor, both get the magnitude
    f, mag = pk.pair_frequencies(16, 10000.0, {"factor": 8.0, "original": 64, "fast": 8.0, "slow": 0.5})
    plain, one = pk.pair_frequencies(16, 10000.0, None)
    assert one == 1.0 and abs(mag - (0.1 * math.log(8.0) + 1.0)) < 1e-15
    assert float(f[0]) == float(plain[0]) and abs(float(f[-1]) - float(plain[-1]) / 8.0) < 1e-18
    assert all(float(plain[i]) / 8.0 - 1e-18 <= float(f[i]) <= float(plain[i]) for i in range(8))
    # the engine's table of the same constants, in the half-split order of its kernels
    from vt_transformer_amd.parts.rotary import rotary_table
    cos, sin = rotary_table(50, 16, 10000.0, {"factor": 8.0, "original": 64, "fast": 8.0, "slow": 0.5})
    ang = torch.arange(50, dtype=torch.float64)[:, None] * f[None, :]
    assert torch.allclose(torch.from_numpy(cos).double(), torch.cos(ang) * mag, atol=1e-6)
    assert torch.allclose(torch.from_numpy(sin).double(), torch.sin(ang) * mag, atol=1e-6)


def test_delta_rule_by_hand():
    """One head of two channels.  With no decay and full removal along the unit key, a key written twice holds the
    second value only; an orthogonal key is untouched."""
    width = 2
    eye = torch.eye(2, dtype=torch.float64)
    big = 40.0
    w = {"r": eye, "k": eye, "v": eye, "g": torch.zeros(2, 2, dtype=torch.float64), "a": torch.zeros(2, 2, dtype=torch.float64),
         "a.b": torch.full((2,), big, dtype=torch.float64), "w1": torch.zeros(1, 2, dtype=torch.float64),
         "w2": torch.zeros(2, 1, dtype=torch.float64), "w0": torch.full((2,), -big, dtype=torch.float64),
         "norm": torch.ones(2, dtype=torch.float64), "o": eye}
    h = torch.tensor([[1.0, 0.0], [1.0, 0.0], [0.0, 1.0]], dtype=torch.float64)
    out = pk.general_delta_mixer(h, w, "", {"heads": 1, "dim": 2}, 0.0)
    # token 0: S = e0 e0^T, o = e0.  token 1: the old e0 row is removed, written again: the same.  token 2: S gains e1 e1^T.
    # behind the per-head norm (over two channels) and a gate of one half: e * sqrt(2) / 2
    s = math.sqrt(2.0) / 2.0
    assert torch.allclose(out, torch.tensor([[s, 0.0], [s, 0.0], [0.0, s]], dtype=torch.float64), atol=1e-6)
    # no removal (a = 0): the same key twice adds up, o = 2 e0, which the norm hides; a read-out along e0 + e1 shows it
    w2 = dict(w)
    w2["a.b"] = torch.full((2,), -big, dtype=torch.float64)
    w2["r"] = torch.ones(2, 2, dtype=torch.float64)
    out2 = pk.general_delta_mixer(h, w2, "", {"heads": 1, "dim": 2}, 0.0)
    assert abs(float(out2[2, 0] / out2[2, 1]) - 2.0) < 1e-6
    # a decay of exp(-exp(-1/2)) per step where the logit is large
    w3 = dict(w2)
    w3["w0"] = torch.full((2,), big, dtype=torch.float64)
    out3 = pk.general_delta_mixer(h, w3, "", {"heads": 1, "dim": 2}, 0.0)
    d = math.exp(-math.exp(-0.5))
    assert abs(float(out3[2, 0] / out3[2, 1]) - (d * d + d)) < 1e-6


def test_experts_scale_their_input_by_the_score():
    g = torch.Generator().manual_seed(0)
    width, ff, n = 6, 5, 4
    w = {"router": torch.randn(3, width, generator=g, dtype=torch.float64)}
    for e in range(3):
        for name, shape in (("gate", (ff, width)), ("up", (ff, width)), ("down", (width, ff))):
            w[f"e{e}.{name}"] = torch.randn(shape, generator=g, dtype=torch.float64)
    x = torch.randn(n, width, generator=g, dtype=torch.float64)
    out = pk.expert_mixture(x, w, "", 3, 2)
    s = torch.sigmoid(x @ w["router"].T)
    for t in range(n):
        want = torch.zeros(width, dtype=torch.float64)
        for e in sorted(range(3), key=lambda e: -float(s[t, e]))[:2]:
            xe = s[t, e] * x[t]
            a = xe @ w[f"e{e}.gate"].T
            want += (a * torch.sigmoid(a) * (xe @ w[f"e{e}.up"].T)) @ w[f"e{e}.down"].T
        assert torch.allclose(out[t], want, atol=1e-12)
    # all three chosen is not the same as two
    assert not torch.allclose(pk.expert_mixture(x, w, "", 3, 3), out)


def test_streams_with_identity_numbers_are_the_plain_residual_sum():
    """in = (1, 0), out = (1, 1) and the identity as mix: stream 0 is an ordinary pre-norm model's stream."""
    cfg = {"architecture": "Kigalix", "vocab": 17, "width": 8, "streams": 2, "norm": {"eps": 1e-5},
           "layers": [latent_layer(heads=1, dim=4, rot_dim=4, vdim=4, rank=4, mlp=dense(8))]}
    w = {k: v.double() for k, v in make_weights(cfg, 2).items()}
    for q in (1, 2):
        w[f"l0.hc{q}.in"] = torch.tensor([1.0, 0.0], dtype=torch.float64)
        w[f"l0.hc{q}.out"] = torch.tensor([1.0, 1.0], dtype=torch.float64)
        w[f"l0.hc{q}.mix"] = torch.eye(2, dtype=torch.float64)
    single = copy.deepcopy(cfg)
    single["streams"] = 1
    w1 = dict(w)
    for q in (1, 2):
        w1[f"l0.hc{q}.in"] = w1[f"l0.hc{q}.out"] = torch.ones(1, dtype=torch.float64)
        w1[f"l0.hc{q}.mix"] = torch.ones(1, 1, dtype=torch.float64)
    ids = [3, 1, 4, 1, 5]
    s2, s1 = [], []
    pk.forward(cfg, w, ids, s2)
    pk.forward(single, w1, ids, s1)
    # both streams started equal and got the same additions: their sum is twice the single stream
    assert torch.allclose(s2[0], 2.0 * s1[0], atol=1e-12)
