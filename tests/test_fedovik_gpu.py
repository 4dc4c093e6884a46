"""Fedovik on the GPU against the plain implementation (plain_fedovik.py): each mechanism alone, prompts against
token-by-token decoding, portions down to two tokens, unequal batches, pages and slots used again, window edges and
far keys, the first tokens of a sequence, long decoding, generation through the engine and through bin/trace_run."""
import copy

import numpy as np
import pytest
import torch

import plain_fedovik as pf
import replay_helpers as rh
from fedovik_helpers import CONFIGS, TOL, attention_layer, check_logits, memory_layer, pair_layer, row_error, write_model
from test_lisunex_gpu import step_part, weights_for
from test_parts_gpu import DEV, OneMixer, rel, runtime
from vt_transformer_amd.config.base import PartSpec

pytestmark = pytest.mark.gpu
PART_TOL = {torch.float32: 2e-5, torch.bfloat16: 2.5e-2}
CUTS = [(0, 20), (20, 21), (21, 23), (23, 70), (70, 71), (71, 83)]


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    root = tmp_path_factory.mktemp("fedovik")
    return {k: write_model(copy.deepcopy(cfg), str(root / k), seed=11 + i) for i, (k, cfg) in enumerate(CONFIGS.items())}


def make_runner(folder, dtype, pool_tokens, max_requests=4, page_size=16, max_seq_len=None):
    from vt_transformer_amd.engine import load_model, make_runner as mk
    model = load_model(folder, dtype, page_size=page_size)
    return mk(model, pool_tokens=pool_tokens, page_size=page_size, max_requests=max_requests,
              max_seq_len=max_seq_len or pool_tokens)


def strip(w, prefix):
    return {k[len(prefix):]: v.double() for k, v in w.items()}


# ---------------------------------------------------------------------------
# each mechanism alone
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width", [40, 272, 700, 5000])
def test_layer_norm_part(dtype, width):
    """Gain and bias, one and two addends in front (the sum goes back into the stream), chosen rows."""
    from vt_transformer_amd.parts import NORMS
    rt = runtime(dtype)
    norm = NORMS.build(PartSpec("layernorm", {"eps": 1e-5, "name": "n", "bias_name": "n.b"}), rt=rt, width=width, prefix="x.")
    g = torch.Generator().manual_seed(width)
    w = {"x.n": (1 + 0.3 * torch.randn(width, generator=g)).to(torch.bfloat16).float(),
         "x.n.b": (0.3 * torch.randn(width, generator=g)).to(torch.bfloat16).float()}
    norm.load(w.__getitem__, rt)
    h = torch.randn(9, width, generator=g) * 3 + 1.5
    d1, d2 = (torch.randn(9, width, generator=g).to(dtype) for _ in range(2))
    tol = 1e-5 if dtype == torch.float32 else 1e-2
    for deltas in ((), (d1,), (d1, d2)):
        hd = h.clone().to(DEV)
        x = h.double() + sum(d.double() for d in deltas)
        ref = pf.layer_norm(x, w["x.n"].double(), w["x.n.b"].double(), 1e-5)
        got = norm.forward(hd, *(d.to(DEV) for d in deltas[:1]), **({"delta2": deltas[1].to(DEV)} if len(deltas) > 1 else {}))
        assert rel(got.float(), ref) < tol
        assert rel(hd, x) < 1e-6                     # the sum is the new stream
    rows = torch.tensor([7, 0, 3], dtype=torch.int32, device=DEV)
    hd = h.clone().to(DEV)
    got = norm.forward(hd, d1.to(DEV), rows=rows, delta2=d2.to(DEV))
    ref = pf.layer_norm((h.double() + d1.double() + d2.double())[[7, 0, 3]], w["x.n"].double(), w["x.n.b"].double(), 1e-5)
    assert rel(got.float(), ref) < tol and torch.equal(hd.cpu(), h)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows", [1, 5, 40, 200])
def test_relu_feed_forward(dtype, rows):
    from vt_transformer_amd.parts import FEED_FORWARDS
    rt = runtime(dtype)
    ff = FEED_FORWARDS.build(PartSpec("gated_mlp", {"intermediate_size": 88, "activation": "relu", "weight_suffix": "",
                                                    "names": {"gate": "gate", "up": "up", "down": "down"}}),
                             rt=rt, width=72, prefix="m.")
    w = weights_for(ff, 3, 0.2)
    ff.load(w.__getitem__, rt)
    x = torch.randn(rows, 72, generator=torch.Generator().manual_seed(rows)).to(dtype)
    ref = pf.relu_mlp(x.double(), strip(w, "m."), "")
    assert rel(ff.forward(x.to(DEV)).float(), ref) < PART_TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nh,kvh,d,dv,rot", [
    (4, 2, 32, 48, 8),       # grouped heads, part of the head rotated (the matrix-core kernels in bfloat16)
    (3, 3, 16, 16, 16),      # as many key heads as query heads, the whole head rotated
    (6, 1, 40, 24, 2),       # sizes that are no multiples of 16: the kernel with a block per token and head
    (8, 2, 64, 32, 64),      # four query heads to a key/value head: a block's waves share keys
    (2, 1, 24, 300, 0),      # no rotation, values wider than a block
])
def test_sigmoid_attention_part(dtype, nh, kvh, d, dv, rot):
    """Neighbouring pairs, biases on every projection, a shift per head, weights that are sigmoids, an elementwise
    gate, in portions that cut pages and in single tokens."""
    from vt_transformer_amd.engine.step import ModelRunner
    from vt_transformer_amd.parts import MIXERS
    rt = runtime(dtype)
    width, t = 72, 83
    pos_spec = PartSpec("rotary", {"theta": 300.0, "dim": rot, "scaling": None}) if rot else None
    names = {"q": "q", "k": "k", "v": "v", "o": "o", "g": "g", "q_bias": "q.b", "k_bias": "k.b", "v_bias": "v.b", "o_bias": "o.b",
             "shift": "pb"}
    mixer = MIXERS.build(PartSpec("masked_attention", dict(
        num_heads=nh, num_kv_heads=kvh, key_dim=d, value_dim=dv, qkv_bias=True, o_bias=True, position=pos_spec,
        rot_pairs="neighbours", scale=0.4, weights="sigmoid", score_shift=True, out_gate=True, names=names)),
        rt=rt, width=width, prefix="a.", shared={})
    w = weights_for(mixer, 3, 0.3)
    w["a.pb"] = torch.linspace(-3.0, -0.5, nh).to(torch.bfloat16).float()
    mixer.load(w.__getitem__, rt)
    runner = ModelRunner(OneMixer(mixer), rt, 16, 256, 4, 256)
    x = (torch.randn(t, width, generator=torch.Generator().manual_seed(4)) * 0.7).to(dtype)
    m = {"heads": nh, "kv_heads": kvh, "dim": d, "vdim": dv, "scale": 0.4}
    if rot:
        m["rot"] = {"dims": rot, "base": 300.0}
    ref = pf.attention_mixer(x.double(), strip(w, "a."), "", m, torch.arange(t))
    assert rel(step_part(runner, mixer, x, CUTS), ref) < PART_TOL[dtype]
    assert rel(step_part(runner, mixer, x, [(0, 60)] + [(i, i + 1) for i in range(60, t)]), ref) < PART_TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nh,kvh,d,dv,window", [
    (4, 2, 16, 32, 12),      # a window that is no multiple of a page
    (3, 3, 8, 40, 1),        # a window of one position
    (8, 2, 32, 16, 33),      # four heads to a key/value head, a window that passes page borders
    (2, 1, 64, 16, 500),     # a window longer than the sequence
    (5, 1, 24, 20, 16),      # sizes that are no multiples of 16
])
def test_window_attention_part(dtype, nh, kvh, d, dv, window):
    """No rotation, queries and keys over their root mean square times a gain, a bias that grows with the logarithm of
    the distance, a window; in portions and single tokens."""
    from vt_transformer_amd.engine.step import ModelRunner
    from vt_transformer_amd.parts import MIXERS
    rt = runtime(dtype)
    width, t = 56, 83
    names = {"q": "q", "k": "k", "v": "v", "o": "o", "q_bias": "q.b", "k_bias": "k.b", "v_bias": "v.b", "q_norm": "q.norm",
             "k_norm": "k.norm", "r1": "r1", "r2": "r2"}
    mixer = MIXERS.build(PartSpec("masked_attention", dict(
        num_heads=nh, num_kv_heads=kvh, key_dim=d, value_dim=dv, qkv_bias=True, scale=0.3, window=window, unit_rms_eps=1e-5,
        qk_gain=True, distance_log=True, names=names)), rt=rt, width=width, prefix="a.", shared={})
    w = weights_for(mixer, 5, 0.3)
    w["a.r1"] = torch.linspace(0.0, 2.5, nh).to(torch.bfloat16).float()
    w["a.r2"] = torch.linspace(0.05, 0.7, nh).to(torch.bfloat16).float()
    mixer.load(w.__getitem__, rt)
    assert mixer.cache_need().window == window
    runner = ModelRunner(OneMixer(mixer), rt, 16, 256, 4, 256)
    x = (torch.randn(t, width, generator=torch.Generator().manual_seed(6)) * 0.7).to(dtype)
    m = {"heads": nh, "kv_heads": kvh, "dim": d, "vdim": dv, "scale": 0.3, "mask": {"size": window}}
    ref = pf.left_mixer(x.double(), strip(w, "a."), "", m, 1e-5, torch.arange(t))
    assert rel(step_part(runner, mixer, x, CUTS), ref) < PART_TOL[dtype]
    assert rel(step_part(runner, mixer, x, [(0, 60)] + [(i, i + 1) for i in range(60, t)]), ref) < PART_TOL[dtype]


@pytest.mark.parametrize("dtype,kernel", [(torch.float32, "plain"), (torch.bfloat16, "plain"), (torch.bfloat16, "cores")])
@pytest.mark.parametrize("form", ["sigmoid", "window"])
def test_one_key_that_stands_out(dtype, kernel, form):
    """Queries and keys are made so that one key takes nearly all the weight from whoever sees it.  Sigmoid weights:
    the key lies hundreds of positions back at the last slot of a page, every other key weighs next to nothing, and
    every later position must return its value, in a prompt's portion and decoded alone.  Window: the positions up
    to the last one whose window holds the key return its value, the next one does not."""
    from vt_transformer_amd.engine.step import ModelRunner, StepEntry
    from vt_transformer_amd.kernels import ops
    from vt_transformer_amd.parts import MIXERS
    from vt_transformer_amd.parts.masked_attention import run_masked_attention
    rt = runtime(dtype)
    cores = kernel == "cores"
    nh, kvh, d, dv = (4 if cores else 2), 1, (16 if cores else 12), 16
    window = 0 if form == "sigmoid" else 150
    mixer = MIXERS.build(PartSpec("masked_attention", dict(num_heads=nh, num_kv_heads=kvh, key_dim=d, value_dim=dv, scale=1.0,
                                                           window=window)), rt=rt, width=8, prefix="a.", shared={})
    runner = ModelRunner(OneMixer(mixer), rt, 16, 1024, 2, 1024)
    t, star = 700, 31                      # the key that stands out: the last slot of the second page
    g = torch.Generator().manual_seed(5)
    y = torch.randn(t, (nh + kvh) * d + kvh * dv, generator=g) * 0.1
    y[:, :nh * d] = 0
    for hh in range(nh):
        y[:, hh * d] = 6.0                 # every query points along element 0 ...
    y[star, nh * d] = 6.0                  # ... and so does the one key: score 36 against about 0
    y[star, (nh + kvh) * d:] = 50.0
    far = star + window - 1 if window else t - 1          # the last position that sees it
    shift = torch.full((nh,), -18.0, device=DEV)          # sigmoid(36 - 18) = 1, sigmoid(0 - 18) = 1.5e-8
    r1 = torch.full((nh,), 0.5, device=DEV)
    r2 = torch.full((nh,), 0.1, device=DEV)
    kw = dict(score_shift=shift, sigmoid_weights=True) if form == "sigmoid" else dict(dist_log=(r1, r2))
    for cuts in ([(0, t)], [(0, 100), (100, far), (far, far + 1)] + [(i, i + 1) for i in range(far + 1, min(t, far + 3))]
                 + ([(far + 3, t)] if far + 3 < t else [])):
        runner.admit("r")
        outs = []
        for a, b in cuts:
            assert runner.cache.reserve([("r", b)])
            ctx = runner.build_context([StepEntry("r", [0] * (b - a), [])])
            cache = runner.storage.layer_caches(ctx.block_tables)[0]
            yy = y[a:b].to(DEV).to(dtype).contiguous()
            q = torch.empty(b - a, nh * d, dtype=dtype, device=DEV)
            out = torch.empty(b - a, nh * dv, dtype=dtype, device=DEV)
            ops.qk_prepare(yy, None, None, ctx.positions, ctx.tok_entry, cache.block_table, q, cache["k"], cache["v"], nh, kvh,
                           d, dv, None)
            # (the product's own choice among its three kernels: with heads of 16 in bfloat16 the matrix-core ones)
            run_masked_attention(rt, ctx, cache, q, out, nh, kvh, d, dv, 1.0, window=window, **kw)
            outs.append(out.float().cpu())
            runner.cache.commit("r", b)
        runner.release("r")
        got = torch.cat(outs)
        assert float(got[star:far + 1].min()) > 49.0, "a position that should see the key that stands out lost it"
        assert float(got[far + 1:].abs().max() if far + 1 < t else 0.0) < 1.0, "a position behind the window saw the key"
        assert float(got[:star].abs().max()) < 1.0
        yd = y.to(dtype).double()
        qd, kd = yd[:, :nh * d].reshape(t, nh, d), yd[:, nh * d:(nh + kvh) * d].reshape(t, kvh, d)
        vd = yd[:, (nh + kvh) * d:].reshape(t, kvh, dv)
        if form == "sigmoid":
            ref = pf.sigmoid_attention(qd, kd, vd, torch.arange(t), 1.0, shift.cpu().double())
        else:
            ref = pf.window_attention(qd, kd, vd, torch.arange(t), 1.0, window, r1.cpu().double(), r2.cpu().double())
        assert rel(got, ref.reshape(t, nh * dv)) < PART_TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nh,kvh,d,dv,taps,ar,gr", [(4, 2, 16, 24, 3, 6, 5), (2, 2, 20, 72, 5, 1, 9), (3, 1, 64, 16, 2, 20, 1),
                                                    (1, 1, 8, 130, 4, 3, 3), (2, 1, 12, 8, 1, 2, 2), (2, 2, 256, 16, 4, 8, 8)])
def test_channel_decay_delta_part(dtype, nh, kvh, d, dv, taps, ar, gr):
    """Prompt in one step, in portions (down to one and two tokens, shorter than the convolution), and token by token,
    all against the plain recurrence."""
    from vt_transformer_amd.engine.step import ModelRunner
    from vt_transformer_amd.parts import MIXERS
    rt = runtime(dtype)
    width, t = 56, 70
    names = {"q": "q", "k": "k", "v": "v", "o": "o", "q_conv": "q.conv", "k_conv": "k.conv", "v_conv": "v.conv", "b": "b",
             "A_log": "A_log", "dt_bias": "dt_bias", "norm": "norm"}
    mixer = MIXERS.build(PartSpec("gated_delta", dict(
        num_heads=nh, num_kv_heads=kvh, key_dim=d, value_dim=dv, conv_taps=taps, norm_eps=1e-5, decay="channel", decay_rank=ar,
        gate_rank=gr, gate_act="sigmoid", names=names)), rt=rt, width=width, prefix="m.", shared={})
    w = weights_for(mixer, 7, 0.25)
    w["m.A_log"] = torch.log(torch.linspace(0.02, 1.5, nh)).to(torch.bfloat16).float()
    w["m.a2"] = (w["m.a2"] * 4).to(torch.bfloat16).float()             # decays that differ from channel to channel
    mixer.load(w.__getitem__, rt)
    runner = ModelRunner(OneMixer(mixer), rt, 16, 256, 3, 256)
    assert runner.storage.state[0].shape == (3 + 1, (taps - 1) * (2 * kvh * d + nh * dv) + nh * d * dv)
    x = (torch.randn(t, width, generator=torch.Generator().manual_seed(8)) * 0.8).to(dtype)
    ref = pf.right_mixer(x.double(), strip(w, "m."), "", dict(heads=nh, kv_heads=kvh, dim=d, vdim=dv), 1e-5)
    whole = step_part(runner, mixer, x, [(0, t)])
    assert rel(whole, ref) < PART_TOL[dtype]
    cut = step_part(runner, mixer, x, [(0, 1), (1, 3), (3, 4), (4, 6), (6, 37), (37, 38), (38, 40), (40, 57), (57, t)])
    steps = step_part(runner, mixer, x, [(i, i + 1) for i in range(t)])
    assert rel(cut, ref) < PART_TOL[dtype] and rel(steps, ref) < PART_TOL[dtype]
    if dtype == torch.float32:
        assert torch.equal(whole, cut) and torch.equal(whole, steps)      # the same operations whatever the cut


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nh,d,dv,cap", [(2, 16, 24, 12.0), (4, 32, 48, 14.0), (3, 20, 8, 3.0), (1, 8, 130, 0.5), (2, 256, 16, 8.0),
                                         (1, 12, 16, 0.0)])
def test_matrix_memory_part(dtype, nh, d, dv, cap):
    """The memory over a prompt in one step, in portions down to one and two tokens, and token by token (the running
    maximum, the normalizer and the matrices travel in the request's state), against the plain recurrence; gates that
    open and close within the sequence."""
    from vt_transformer_amd.engine.step import ModelRunner
    from vt_transformer_amd.kernels import ops
    from vt_transformer_amd.parts import MIXERS
    rt = runtime(dtype)
    width, t = 56, 70
    mixer = MIXERS.build(PartSpec("matrix_memory", dict(num_heads=nh, key_dim=d, value_dim=dv, gate_cap=cap, norm_eps=1e-5)),
                         rt=rt, width=width, prefix="m.", shared={})
    w = weights_for(mixer, 9, 0.25)
    # (gates that open and close all the way in float32; in bfloat16, where a long portion's logits are rounded to
    # eight bits, gates whose exponentials that rounding does not move by more than the tolerance)
    steep = 8 if dtype == torch.float32 else 1.5
    w["m.i"], w["m.f"] = (w["m.i"] * steep).to(torch.bfloat16).float(), (w["m.f"] * steep).to(torch.bfloat16).float()
    w["m.f.b"] = torch.linspace(0.5, 4.0, nh).to(torch.bfloat16).float()
    mixer.load(w.__getitem__, rt)
    runner = ModelRunner(OneMixer(mixer), rt, 16, 256, 3, 256)
    assert runner.storage.state[0].shape == (3 + 1, ops.matrix_memory_state_floats(nh, d, dv))
    x = (torch.randn(t, width, generator=torch.Generator().manual_seed(10)) * 0.8).to(dtype)
    if cap > 0:
        ref = pf.mlstm_mixer(x.double(), strip(w, "m."), "", dict(heads=nh, dim=d, vdim=dv, gate_cap=cap), 1e-5)
    else:
        # (no cap: the plain mixer with a cap so large that the tanh is the identity)
        ref = pf.mlstm_mixer(x.double(), strip(w, "m."), "", dict(heads=nh, dim=d, vdim=dv, gate_cap=1e6), 1e-5)
    # (steep gates make the normalizer's product n . q cancel now and then: where it loses four digits, float32 leaves
    # 1e-4 of a head's read-out uncertain, and the norm behind takes only part of that out again)
    # In bfloat16 a token whose normalizer cancels is moved a long way by the rounding of q and k alone, while a lost
    # state or a wrong gate moves every token behind it: nine tokens in ten within the tolerance, none wildly off.
    def close(got):
        if dtype == torch.float32:
            return rel(got, ref) < 5e-4
        rows = (got.double() - ref).abs().amax(dim=1) / ref.abs().amax()
        return float((rows < PART_TOL[dtype]).double().mean()) >= 0.9 and float(rows.max()) < 1.0
    whole = step_part(runner, mixer, x, [(0, t)])
    assert close(whole)
    cut = step_part(runner, mixer, x, [(0, 1), (1, 3), (3, 4), (4, 6), (6, 37), (37, 38), (38, 40), (40, 57), (57, t)])
    steps = step_part(runner, mixer, x, [(i, i + 1) for i in range(t)])
    assert close(cut) and close(steps)
    if dtype == torch.float32:
        assert torch.equal(whole, cut) and torch.equal(whole, steps)      # the same operations whatever the cut


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_pair_of_mixers(dtype):
    """Two mixers side by side with their factors: pages for the one, state for the other, both through one layer."""
    from vt_transformer_amd.engine.step import ModelRunner
    from vt_transformer_amd.parts import MIXERS
    rt = runtime(dtype)
    width, t = 48, 83
    left = PartSpec("masked_attention", dict(num_heads=2, num_kv_heads=1, key_dim=16, value_dim=16, scale=0.3, window=9,
                                             names={"q": "q", "k": "k", "v": "v", "o": "o"}, prefix="left."))
    right = PartSpec("matrix_memory", dict(num_heads=2, key_dim=8, value_dim=12, gate_cap=10.0, norm_eps=1e-5, prefix="right."))
    pair = MIXERS.build(PartSpec("mixer_pair", dict(left=left, right=right, left_scale=0.75, right_scale=-1.5)), rt=rt,
                        width=width, prefix="p.", shared={})
    assert pair.cache_need().window == 9 and pair.state_need().shape == pair.members[1].state_need().shape and pair.replayable
    w = weights_for(pair, 13, 0.3)
    w["p.right.f.b"] = torch.tensor([2.0, 3.0])
    pair.load(w.__getitem__, rt)
    runner = ModelRunner(OneMixer(pair), rt, 16, 256, 3, 256)
    x = (torch.randn(t, width, generator=torch.Generator().manual_seed(14)) * 0.8).to(dtype)
    xd, pos = x.double(), torch.arange(t)
    lw = strip({k: v for k, v in w.items() if k.startswith("p.left.")}, "p.left.")
    q, k, v = ((xd @ lw[n].t()).reshape(t, -1, 16) for n in ("q", "k", "v"))
    lo = pf.window_attention(q, k, v, pos, 0.3, 9, torch.zeros(2, dtype=torch.float64), torch.ones(2, dtype=torch.float64))
    ref = 0.75 * (lo.reshape(t, 32) @ lw["o"].t()) - 1.5 * pf.mlstm_mixer(
        xd, strip({k: v for k, v in w.items() if k.startswith("p.right.")}, "p.right."), "",
        dict(heads=2, dim=8, vdim=12, gate_cap=10.0), 1e-5)
    assert rel(step_part(runner, pair, x, CUTS), ref) < PART_TOL[dtype]
    with pytest.raises(ValueError, match="one kind"):
        MIXERS.build(PartSpec("mixer_pair", dict(left=left, right=left)), rt=rt, width=width, prefix="p.", shared={})


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_stream_after_every_layer_run(folders, dtype):
    """The residual stream behind every layer run (re-entry, offsets and both sublayers included) against the plain
    implementation's, for a prompt in one step."""
    from vt_transformer_amd.engine.step import StepEntry
    folder = folders["A"]
    cfg, w = pf.read_folder(folder)
    toks = rh.random_requests(cfg["vocab"], [29], seed=1)["r0"]
    streams = []
    pf.forward(cfg, w, toks, streams)
    runner = make_runner(folder, dtype, pool_tokens=64, max_requests=1)
    seen = []
    model = runner.model
    for block in model.layers:
        inner = block.forward

        def wrapped(h, delta, ctx, cache, state, inner=inner):
            from vt_transformer_amd.models.model import settle
            h, d = inner(h, delta, ctx, cache, state)
            seen.append(settle(h.clone(), d).cpu().double())
            return h, d
        block.forward = wrapped
    runner.admit("r")
    runner.step([StepEntry("r", toks, [len(toks) - 1])])
    assert len(seen) == len(streams)
    for i, (a, b) in enumerate(zip(seen, streams)):
        assert rel(a, b) < (2e-5 if dtype == "float32" else 5e-2), f"layer run {i}"


# ---------------------------------------------------------------------------
# whole models: schedules against the plain implementation
# ---------------------------------------------------------------------------
LENGTHS = [61, 1, 23, 90, 2, 47]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_schedules(folders, name, dtype):
    """Whole prompts; most of a prompt and then its last tokens one by one; portions of changing sizes down to two
    tokens; unequal requests side by side with three slots and few pages, so that both are used again."""
    folder, vocab = folders[name], CONFIGS[name]["vocab"]
    reqs = rh.random_requests(vocab, LENGTHS, seed=3)
    cache = {}
    runner = make_runner(folder, dtype, pool_tokens=256, max_requests=3)
    whole = rh.trace_alone(reqs, {r: [(0, len(t))] for r, t in reqs.items()})
    got_whole = rh.run_in_process(runner, whole)
    check_logits(folder, reqs, whole, got_whole, dtype, cache)
    decode = rh.trace_alone(reqs, {r: ([(0, max(1, len(t) - 30))] + [(i, i + 1) for i in range(max(1, len(t) - 30), len(t))])
                                   for r, t in reqs.items()})
    got_decode = rh.run_in_process(runner, decode)
    check_logits(folder, reqs, decode, got_decode, dtype, cache)
    portions = {r: rh.cut(t, [7, 2, 16, 3, 2, 33, 1, 5]) for r, t in reqs.items()}
    chunked = rh.trace_alone(reqs, portions)
    got_chunked = rh.run_in_process(runner, chunked)
    check_logits(folder, reqs, chunked, got_chunked, dtype, cache)
    mixed = rh.trace_mixed(reqs, {r: rh.cut(t, [9, 2, 1, 1, 20, 1, 1, 1, 4]) for r, t in reqs.items()}, max_live=3, seed=5)
    assert rh.max_live_tokens(mixed) <= 256
    got_mixed = rh.run_in_process(runner, mixed)
    check_logits(folder, reqs, mixed, got_mixed, dtype, cache)
    if dtype == "float32":
        # a position's logits do not depend on the cut, the batch, the pages or the slots, beyond rounding
        flat = {}
        for steps, got in ((whole, got_whole), (decode, got_decode), (chunked, got_chunked), (mixed, got_mixed)):
            pos = {r: 0 for r in reqs}
            for s in steps:
                row = 0
                for e in s["entries"]:
                    for wi in e["want"]:
                        flat.setdefault((e["id"], pos[e["id"]] + wi), []).append(got[s["step"]][row])
                        row += 1
                    pos[e["id"]] += len(e["tokens"])
        for key, rows in flat.items():
            assert len(rows) == 4
            for r in rows[1:]:
                assert row_error(r, rows[0].astype(np.float64)) < 2e-6, f"{key} depends on the schedule"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_across_windows_and_pages(folders, dtype):
    folder, vocab = folders["A"], CONFIGS["A"]["vocab"]
    reqs = rh.random_requests(vocab, [150], seed=9)
    steps = rh.trace_alone(reqs, {"r0": [(0, 5)] + [(i, i + 1) for i in range(5, 150)]})
    runner = make_runner(folder, dtype, pool_tokens=192, max_requests=1)
    check_logits(folder, reqs, steps, rh.run_in_process(runner, steps), dtype)
    assert sum(runner.cache.available_pages()) == sum(p.num_pages for p in runner.cache.pools)


def test_pages_behind_a_window_are_given_back():
    """A model whose only pages are a window's: a request longer than the pool runs, because keys that no later
    position can see are dead; the plain logits still come out."""
    import tempfile
    cfg = {"architecture": "Fedovik", "vocab": 61, "width": 48, "embedding": {"scale": 2.0}, "norm": {"eps": 1e-5},
           "layers": [pair_layer(window=20, ff=40), memory_layer()], "loop": {"start": 0, "stop": 1, "times": 2}}
    with tempfile.TemporaryDirectory() as tmp:
        folder = write_model(cfg, tmp, seed=77)
        reqs = rh.random_requests(61, [140], seed=13)
        steps = rh.trace_alone(reqs, {"r0": rh.cut(reqs["r0"], [10])})
        runner = make_runner(folder, "float32", pool_tokens=96, max_requests=1, max_seq_len=160)
        check_logits(folder, reqs, steps, rh.run_in_process(runner, steps), "float32")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_generation_through_the_engine(folders, dtype):
    """Greedy tokens through Engine.generate (scheduler with short portions, two slots for three requests)."""
    from vt_transformer_amd.engine import Engine
    from vt_transformer_amd.sampling import SamplingParams
    folder = folders["C"]
    cfg, w = pf.read_folder(folder)
    prompts = [r for r in rh.random_requests(cfg["vocab"], [19, 3, 41], seed=21).values()]
    eng = Engine(folder, dtype=dtype, num_pages=16, max_running_reqs=2, max_seq_len=128, chunk_size=16, max_extend_tokens=24)
    got = eng.generate(prompts, SamplingParams(max_tokens=8, ignore_eos=True))
    for p, g in zip(prompts, got):
        assert len(g) == 8
        if dtype == "float32":
            assert g == pf.greedy(cfg, w, p, 8)
        else:
            logits = pf.forward(cfg, w, p + g)
            for i, tok in enumerate(g):
                row = logits[len(p) - 1 + i]
                assert float(row.max() - row[tok]) <= 3e-2 * float(row.abs().max())


def test_trace_run_with_a_fedovik_folder(folders, tmp_path):
    folder, vocab = folders["C"], CONFIGS["C"]["vocab"]
    reqs = rh.random_requests(vocab, [40, 9, 27], seed=17)
    steps = rh.trace_mixed(reqs, {r: rh.cut(t, [6, 2, 11, 1]) for r, t in reqs.items()}, max_live=2, seed=2)
    got = rh.run_trace_run(folder, "float32", steps, str(tmp_path / "out"), rh.max_live_tokens(steps), vocab,
                           extra_args=("--max-requests", "2"))
    check_logits(folder, reqs, steps, got, "float32")


def test_captured_decoding_steps_move_the_state_once(folders):
    """Decoding through captured steps (bfloat16): the launch-by-launch run in front of a capture is the step itself,
    later steps are replays, padding entries use the state row that nobody owns; the logits are those of the same
    schedule launched step by step, bit for bit, and the plain implementation's within rounding."""
    folder, vocab = folders["A"], CONFIGS["A"]["vocab"]
    reqs = rh.random_requests(vocab, [30, 12, 21], seed=31)
    steps, nxt = [], {r: 6 for r in reqs}
    steps.append({"step": 0, "entries": [{"id": r, "tokens": t[:6], "want": [5]} for r, t in reqs.items()], "end": []})
    while nxt:
        live = list(nxt)
        entries = [{"id": r, "tokens": reqs[r][nxt[r]:nxt[r] + 1], "want": [0]} for r in live]
        end = []
        for r in live:
            nxt[r] += 1
            if nxt[r] == len(reqs[r]):
                end.append(r)
                del nxt[r]
        steps.append({"step": len(steps), "entries": entries, "end": end})
    plain = make_runner(folder, "bfloat16", pool_tokens=192, max_requests=3)
    got_plain = rh.run_in_process(plain, steps)
    graphs = make_runner(folder, "bfloat16", pool_tokens=192, max_requests=3)
    graphs.decode_graphs = True
    assert graphs.replays(3) and not graphs._stateless
    got = rh.run_in_process(graphs, steps)
    assert graphs._graphs, "no decoding step was captured"
    for k in got_plain:
        assert np.array_equal(got[k], got_plain[k]), f"step {k} differs between replayed and launched steps"
    check_logits(folder, reqs, steps, got, "bfloat16")


def random_fedovik_config(seed: int) -> dict:
    """Sizes, orders and constants drawn at random, odd ones on purpose."""
    rs = np.random.RandomState(seed)
    pick = lambda xs: xs[rs.randint(len(xs))]
    width = int(pick([40, 72, 100, 136, 200]))
    layers = []
    for _ in range(rs.randint(2, 6)):
        heads = int(pick([1, 2, 3, 4, 6, 8]))
        kv = int(pick([k for k in (1, 2, 3, 4) if heads % k == 0]))
        ff = int(pick([0, 24, 100, 136])) or None
        kind = rs.randint(3)
        if kind == 0:
            dim = int(pick([8, 16, 24, 40, 64]))
            layers.append(attention_layer(heads=heads, kv_heads=kv, dim=dim, vdim=int(pick([8, 16, 32, 40, 80, 144])),
                                          scale=float(pick([0.05, 0.3, 1.0])),
                                          rot_dims=int(pick([d for d in (2, 4, 8, 16, 24, 40, 64) if d <= dim])),
                                          base=float(pick([100.0, 1e4, 1e6])), ff=ff))
        elif kind == 1:
            r_heads = int(pick([1, 2, 4, 6]))
            layers.append(pair_layer(heads=heads, kv_heads=kv, dim=int(pick([8, 16, 24, 64])), vdim=int(pick([8, 16, 48, 80])),
                                     scale=float(pick([0.1, 0.3, 1.0])), window=int(pick([1, 3, 16, 50, 1000])),
                                     r_heads=r_heads, r_kv=int(pick([k for k in (1, 2, 3) if r_heads % k == 0])),
                                     r_dim=int(pick([8, 12, 32, 72, 128])), r_vdim=int(pick([8, 20, 64])),
                                     conv=int(pick([2, 3, 4, 6])), a_rank=int(pick([1, 4, 20])), g_rank=int(pick([1, 7, 16])),
                                     left_scale=float(pick([1.0, 0.5, 1.7])), right_scale=float(pick([1.0, 0.9, 2.0])), ff=ff))
        else:
            layers.append(memory_layer(heads=heads, dim=int(pick([8, 12, 32, 72])), vdim=int(pick([8, 20, 64, 80])),
                                       gate_cap=float(pick([2.0, 16.0, 30.0])), ff=ff))
    n = len(layers)
    loop = None
    if rs.rand() < 0.6:
        a = int(rs.randint(0, n))
        loop = {"start": a, "stop": int(rs.randint(a + 1, n + 1)), "times": int(rs.randint(1, 4))}
    return {"architecture": "Fedovik", "vocab": int(pick([51, 97, 130, 255])), "width": width,
            "embedding": {"scale": float(pick([1.0, 0.5, 4.0]))}, "norm": {"eps": float(pick([1e-6, 1e-5, 1e-3]))},
            "layers": layers, "loop": loop}


@pytest.mark.parametrize("seed", range(8))
def test_configurations_drawn_at_random(tmp_path, seed):
    """Whatever config.json says is what runs: random sizes, layer orders, loops and constants, in float32 (sharp) and
    bfloat16, through portions and a mixed batch."""
    cfg = random_fedovik_config(seed)
    folder = write_model(copy.deepcopy(cfg), str(tmp_path / "m"), seed=40 + seed)
    reqs = rh.random_requests(cfg["vocab"], [37, 5, 70], seed=seed)
    steps = rh.trace_mixed(reqs, {r: rh.cut(t, [11, 2, 1, 30, 1, 1]) for r, t in reqs.items()}, max_live=2, seed=seed)
    whole = rh.trace_alone(reqs, {r: [(0, len(t))] for r, t in reqs.items()})
    cache = {}
    for dtype in ("float32", "bfloat16"):
        runner = make_runner(folder, dtype, pool_tokens=192, max_requests=2)
        runner.decode_graphs = True
        check_logits(folder, reqs, whole, rh.run_in_process(runner, whole), dtype, cache)
        check_logits(folder, reqs, steps, rh.run_in_process(runner, steps), dtype, cache)
