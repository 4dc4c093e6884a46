"""Kigalix on the GPU against the plain implementation (plain_kigalix.py): each mechanism alone, prompts against
token-by-token decoding, portions down to two tokens, unequal batches, pages and slots used again, a key far back at a
page's border, a state that must survive portions and slots, the first tokens, long decoding, generation through the
engine and through bin/trace_run."""
import copy
import math

import numpy as np
import pytest
import torch

import plain_kigalix as pk
import replay_helpers as rh
from kigalix_helpers import CONFIGS, check_logits, delta_layer, dense, latent_layer, moe, without_experts, write_model
from test_parts_gpu import DEV, OneMixer, rel, runtime
from vt_transformer_amd.config.base import PartSpec

pytestmark = pytest.mark.gpu
PART_TOL = {torch.float32: 2e-5, torch.bfloat16: 2.5e-2}
LATENT_NAMES = {"q": "q", "dkv": "dkv", "dkv_norm": "dkv.norm", "uk": "uk", "uv": "uv", "o": "o", "g": "g"}
CUTS = [(0, 20), (20, 21), (21, 23), (23, 70), (70, 71), (71, 83)]


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    root = tmp_path_factory.mktemp("kigalix")
    # (model A is written with the idle second sublayer's tensors of its layer without a feed-forward)
    out = {k: write_model(copy.deepcopy(cfg), str(root / k), seed=41 + i, idle=k == "A")
           for i, (k, cfg) in enumerate(CONFIGS.items())}
    # the same layers with dense feed-forwards: what bfloat16 compares to a sequence's end
    out.update({k + "-dense": write_model(without_experts(cfg), str(root / (k + "d")), seed=51 + i)
                for i, (k, cfg) in enumerate(CONFIGS.items())})
    return out


def make_runner(folder, dtype, pool_tokens, max_requests=4, page_size=16, max_seq_len=None):
    from vt_transformer_amd.engine import load_model, make_runner as mk
    model = load_model(folder, dtype, page_size=page_size)
    return mk(model, pool_tokens=pool_tokens, page_size=page_size, max_requests=max_requests,
              max_seq_len=max_seq_len or pool_tokens)


def weights_for(part, seed, scale):
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, decl in part.tensors().items():
        if decl.role == "matrix32":
            t = torch.randn(decl.shape, generator=g) * 2.0 / decl.shape[-1] ** 0.5
        else:
            t = torch.randn(decl.shape, generator=g) * (scale if decl.role == "matrix" else 0.4)
        if decl.role == "gain":
            t += 1.0
        out[name] = t.to(torch.bfloat16).float()
    return out


def step_part(runner, mixer, x, cuts, rid="r"):
    """The mixer alone over x [T, width] of one request, in the portions `cuts`."""
    from vt_transformer_amd.engine.step import StepEntry
    runner.admit(rid)
    outs = []
    for a, b in cuts:
        assert runner.cache.reserve([(rid, b)])
        if runner.cache.get(rid).fresh and runner.storage.state:
            runner.storage.clear_state([runner.cache.get(rid).slot])
        ctx = runner.build_context([StepEntry(rid, [0] * (b - a), [])])
        caches = runner.storage.layer_caches(ctx.block_tables)
        state = runner.storage.state[0] if runner.storage.state else None
        outs.append(mixer.forward(x[a:b].to(DEV).contiguous(), ctx, caches[0] if caches else None, state).float().cpu().clone())
        runner.cache.commit(rid, b)
    runner.release(rid)
    return torch.cat(outs)


# ---------------------------------------------------------------------------
# the mechanisms alone
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nh,dn,dr,dv,rank,base,scaling,gate", [
    (4, 16, 16, 24, 32, 1e4, None, False),                   # sizes that suit the matrix-core kernels
    (3, 20, 12, 10, 24, 300.0, (4.0, 64, 16.0, 2.0), True),  # no multiples of 16; stretched frequencies, some pairs in between
    (8, 8, 32, 16, 32, 500.0, (8.0, 32, 4.0, 1.0), True),    # eight heads on the one cache
    (1, 8, 16, 8, 16, 50.0, (2.0, 1000, 32.0, 1.0), False),  # one head; a stretch that reaches no pair fully
    (2, 24, 0, 40, 48, 0.0, None, True),                     # nothing rotated
    (20, 16, 16, 8, 16, 1e6, None, True),                    # more heads than the 16 rows of a decoding product
])
def test_latent_attention_with_neighbouring_pairs(dtype, nh, dn, dr, dv, rank, base, scaling, gate):
    from vt_transformer_amd.engine.step import ModelRunner
    from vt_transformer_amd.parts import MIXERS
    rt = runtime(dtype)
    width, t = 72, 83
    sc = dict(zip(("factor", "original", "fast", "slow"), scaling)) if scaling else None
    pos_spec = PartSpec("rotary", {"theta": base, "dim": dr, "scaling": sc}) if dr else None
    mixer = MIXERS.build(PartSpec("latent_attention", dict(
        num_heads=nh, plain_dim=dn, rot_dim=dr, value_dim=dv, rank=rank, norm_eps=1e-5, position=pos_spec, scale=0.3,
        window=0, sink=False, out_gate=gate, rot_pairs="neighbours", names=dict(LATENT_NAMES))), rt=rt, width=width,
        prefix="a.", shared={})
    w = weights_for(mixer, 3, 0.3)
    mixer.load(w.__getitem__, rt)
    runner = ModelRunner(OneMixer(mixer), rt, 16, 256, 4, 256)
    x = (torch.randn(t, width, generator=torch.Generator().manual_seed(4)) * 0.7).to(dtype)
    got = step_part(runner, mixer, x, CUTS)
    m = {"heads": nh, "dim": dn, "rot_dim": dr, "vdim": dv, "kv_rank": rank, "scale": 0.3}
    if dr:
        m["rot"] = {"dims": dr, "base": base}
        if sc:
            m["rot"]["scaling"] = sc
    ref = pk.latent_attention_mixer(x.double(), {k: v.double() for k, v in w.items()}, "a.", m, 1e-5, torch.arange(t), gated=gate)
    assert rel(got, ref) < PART_TOL[dtype]
    if dtype == torch.float32:      # the same operations whatever the cut
        assert torch.equal(got, step_part(runner, mixer, x, [(0, t)]))
        assert torch.equal(got, step_part(runner, mixer, x, [(0, 50)] + [(i, i + 1) for i in range(50, t)]))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nh", [2, 4])
def test_one_key_far_back_at_a_page_border(dtype, nh):
    """The whole latent mixer with weights that pass its input through: one token's low-rank vector points along
    element 0 and every query asks for element 0, so every later position returns that vector, hundreds of keys on,
    and no earlier one sees anything of it; the token sits in the last slot of a page; in one portion, in portions
    that end before, at and behind it, and decoded one by one."""
    from vt_transformer_amd.engine.step import ModelRunner
    from vt_transformer_amd.parts import MIXERS
    rt = runtime(dtype)
    rank, dr, t, star = 16, 16, 420, 31
    qcols = ccol = nh * (rank + dr)
    gcol = ccol + rank + dr
    width = gcol + nh * rank
    mixer = MIXERS.build(PartSpec("latent_attention", dict(
        num_heads=nh, plain_dim=rank, rot_dim=dr, value_dim=rank, rank=rank, norm_eps=1e-6, scale=1.0, window=0,
        position=PartSpec("rotary", {"theta": 100.0, "dim": dr, "scaling": None}), sink=False, out_gate=True,
        rot_pairs="neighbours", names=dict(LATENT_NAMES))), rt=rt, width=width, prefix="a.", shared={})
    eye = torch.eye(width)
    w = {"a.q": eye[:qcols], "a.dkv": eye[ccol:gcol], "a.g": eye[gcol:], "a.dkv.norm": torch.ones(rank),
         "a.uk": torch.eye(rank).repeat(nh, 1), "a.uv": torch.eye(rank).repeat(nh, 1),
         "a.o": torch.cat([torch.eye(nh * rank), torch.zeros(width - nh * rank, nh * rank)])}
    mixer.load(w.__getitem__, rt)
    runner = ModelRunner(OneMixer(mixer), rt, 16, 512, 2, 512)
    g = torch.Generator().manual_seed(6)
    x = torch.zeros(t, width)
    for hh in range(nh):
        x[:, hh * (rank + dr)] = 6.0                     # every head's query: element 0 of the unrotated part
    x[:, ccol + 1:ccol + rank] = torch.randn(t, rank - 1, generator=g)      # low-rank vectors without element 0 ...
    x[star, ccol:ccol + rank] = 0.0
    x[star, ccol] = 1.0                                                      # ... but one, which is nothing else
    x[:, gcol:] = 30.0                                                       # gates wide open
    x = x.to(dtype)
    height = math.sqrt(rank)                # what the norm makes of it
    for cuts in ([(0, t)], [(0, star), (star, star + 1), (star + 1, star + 3), (star + 3, 300), (300, t)],
                 [(0, 32)] + [(i, i + 1) for i in range(32, 80)] + [(80, 399)] + [(i, i + 1) for i in range(399, t)]):
        got = step_part(runner, mixer, x, cuts).reshape(t, -1)[:, :nh * rank].reshape(t, nh, rank)
        assert float(got[star:, :, 0].min()) > 0.97 * height, "a position lost the key"
        assert float(got[:star, :, 0].abs().max()) < 0.05


def _delta_rows(t, nh, d, star, star2):
    """Rows [r | k | v | a] and decay logits for the delta rule's kernel, made so that the answer is known: every
    read-out vector is element 0; token `star` writes 2 e0 v*^T, token `star2` removes along e0 at rate 1 and writes
    3 e0 v2^T; all other keys have no element 0.  Head 0 keeps its state (decay 1), head 1 decays element 0 by
    exp(-c) a token."""
    g = torch.Generator().manual_seed(8)
    kd = nh * d
    r = torch.zeros(t, nh, d)
    r[:, :, 0] = 1.0
    k = torch.randn(t, nh, d, generator=g) * 0.3
    k[:, :, 0] = 0.0
    v = torch.randn(t, nh, d, generator=g)
    a = torch.full((t, nh, d), -30.0)
    z = torch.full((t, nh, d), -30.0)
    z[:, 1, 0] = 30.0
    for s_, height in ((star, 2.0), (star2, 3.0)):
        k[s_] = 0.0
        k[s_, :, 0] = height
    a[star2, :, 0] = 30.0
    x = torch.cat([r.reshape(t, kd), k.reshape(t, kd), v.reshape(t, kd), a.reshape(t, kd)], dim=1)
    return x, z.reshape(t, kd), v


@pytest.mark.parametrize("d,dv", [(48, 48), (80, 48), (112, 48), (176, 48), (144, 128)])
@pytest.mark.parametrize("nh", [2, 4, 8])
def test_matrix_core_attention_whose_key_size_is_no_multiple_of_32(nh, d, dv):
    """The kernel for portions of prompts, alone (heads that are no multiple of four) and with four heads of a block
    sharing the keys they read, against the kernel with a block per token and head: key sizes that end in half a
    step of the wide matrix product (a low-rank vector of 48 or 64 with a rotated part of 32 or 16 behind it)."""
    from vt_transformer_amd.engine.step import ModelRunner, StepEntry
    from vt_transformer_amd.kernels import ops
    from vt_transformer_amd.parts import MIXERS
    from vt_transformer_amd.parts.masked_attention import TILES_KEY
    rt = runtime(torch.bfloat16)
    mixer = MIXERS.build(PartSpec("masked_attention", dict(num_heads=nh, num_kv_heads=1, key_dim=d, value_dim=dv, scale=0.2)),
                         rt=rt, width=8, prefix="a.", shared={})
    runner = ModelRunner(OneMixer(mixer), rt, 16, 256, 2, 256)
    t = 83
    y = torch.randn(t, (nh + 1) * d + dv, generator=torch.Generator().manual_seed(5)).to(DEV).to(torch.bfloat16)
    runner.admit("r")
    assert runner.cache.reserve([("r", t)])
    ctx = runner.build_context([StepEntry("r", [0] * t, [])])
    cache = runner.storage.layer_caches(ctx.block_tables)[0]
    q = torch.empty(t, nh * d, dtype=torch.bfloat16, device=DEV)
    got, ref = torch.empty(t, nh * dv, dtype=torch.bfloat16, device=DEV), torch.empty(t, nh * dv, dtype=torch.bfloat16, device=DEV)
    ops.qk_prepare(y, None, None, ctx.positions, ctx.tok_entry, cache.block_table, q, cache["k"], cache["v"], nh, 1, d, dv, None)
    ops.attention_masked_mfma(q, cache["k"], cache["v"], ctx.positions, ctx.tok_entry, cache.block_table, ctx.extra[TILES_KEY],
                              got, nh, 1, d, dv, 0.2)
    ops.attention_masked(q, cache["k"], cache["v"], ctx.positions, ctx.tok_entry, cache.block_table, ref, nh, 1, d, dv, 0.2)
    runner.release("r")
    assert rel(got, ref) < 1.5e-2


@pytest.mark.parametrize("cuts", ["whole", "portions", "single"])
def test_delta_rule_keeps_decays_and_removes_what_it_should(cuts):
    """Known answers from the kernel itself, through a request's state slot: a row written once is read hundreds of
    tokens later unchanged (or decayed by exp(-c) a token), and a removal at rate 1 along the same unit key takes all
    of it away in the same step that writes the next.  A state that is lost between portions, cleared late or decayed
    on the wrong channel shows.  The slot is used by another request in between."""
    from vt_transformer_amd.engine.step import ModelRunner, StepEntry
    from vt_transformer_amd.kernels import ops
    from vt_transformer_amd.parts import MIXERS
    rt = runtime(torch.float32)
    nh, d, t, star, star2 = 2, 16, 330, 5, 290
    c = math.exp(-0.5)
    mixer = MIXERS.build(PartSpec("general_delta", dict(num_heads=nh, key_dim=d, decay_rank=4, norm_eps=1e-6)), rt=rt,
                         width=8, prefix="a.", shared={})
    runner = ModelRunner(OneMixer(mixer), rt, 16, 512, 1, 512)
    x, z, v = _delta_rows(t, nh, d, star, star2)
    portions = {"whole": [(0, t)], "portions": [(0, star), (star, star + 1), (star + 1, star + 3), (star + 3, star2), (star2, t)],
                "single": [(0, 3)] + [(i, i + 1) for i in range(3, 40)] + [(40, 280)] + [(i, i + 1) for i in range(280, t)]}[cuts]
    for rid in ("first", "second"):          # the second request takes the slot that the first one left full
        runner.admit(rid)
        outs = []
        for a, b in portions:
            assert runner.cache.reserve([(rid, b)])
            if runner.cache.get(rid).fresh:
                runner.storage.clear_state([runner.cache.get(rid).slot])
            ctx = runner.build_context([StepEntry(rid, [0] * (b - a), [])])
            out = torch.empty(b - a, nh * d, device=DEV)
            kd = nh * d
            ops.general_delta(x[a:b].to(DEV).contiguous(), 0, kd, 2 * kd, 3 * kd, z[a:b].to(DEV).contiguous(), None,
                              runner.storage.state[0], ctx.entry_start, ctx.state_slots, out, nh, d, d, c, 1e-6)
            outs.append(out.cpu())
            runner.cache.commit(rid, b)
        runner.release(rid)
        got = torch.cat(outs).reshape(t, nh, d)
        assert float(got[:star].abs().max()) < 1e-5, "something was in the state before the first write"
        for p in (star, star + 1, 39, 40, 150, 279, 280, star2 - 1):
            assert torch.allclose(got[p, 0], 2.0 * v[star, 0], rtol=1e-4, atol=1e-5), p
            assert torch.allclose(got[p, 1], 2.0 * v[star, 1] * math.exp(-c * (p - star)), rtol=1e-3, atol=1e-30), p
        for p in (star2, star2 + 1, t - 1):
            assert torch.allclose(got[p, 0], 3.0 * v[star2, 0], rtol=1e-4, atol=1e-4), p
            assert torch.allclose(got[p, 1], 3.0 * v[star2, 1] * math.exp(-c * (p - star2)), rtol=1e-3, atol=1e-30), p


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nh,d,low", [(3, 20, 12), (1, 64, 4), (2, 128, 32), (5, 16, 16), (6, 48, 1)])
def test_general_delta_part(dtype, nh, d, low):
    from vt_transformer_amd.engine.step import ModelRunner
    from vt_transformer_amd.parts import MIXERS
    rt = runtime(dtype)
    width, t = 72, 83
    mixer = MIXERS.build(PartSpec("general_delta", dict(num_heads=nh, key_dim=d, decay_rank=low, norm_eps=1e-5)), rt=rt,
                         width=width, prefix="a.", shared={})
    assert mixer.cache_need() is None and mixer.state_need().shape == (nh * d * d,)
    w = weights_for(mixer, 5, 0.3)
    mixer.load(w.__getitem__, rt)
    runner = ModelRunner(OneMixer(mixer), rt, 16, 256, 2, 256)
    x = (torch.randn(t, width, generator=torch.Generator().manual_seed(7)) * 0.9).to(dtype)
    got = step_part(runner, mixer, x, CUTS)
    ref = pk.general_delta_mixer(x.double(), {k: v.double() for k, v in w.items()}, "a.", {"heads": nh, "dim": d}, 1e-5)
    assert rel(got, ref) < PART_TOL[dtype]
    if dtype == torch.float32:
        assert torch.equal(got, step_part(runner, mixer, x, [(0, t)]))
        assert torch.equal(got, step_part(runner, mixer, x, [(0, 50)] + [(i, i + 1) for i in range(50, t)]))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("experts,top,inter,width", [(5, 2, 40, 96), (3, 1, 64, 72), (16, 4, 16, 128), (4, 4, 24, 80),
                                                     (9, 3, 32, 80), (2, 1, 200, 128), (8, 2, 20, 36)])
def test_expert_mixture_part(dtype, experts, top, inter, width):
    """Few rows (a kernel that walks a token's choices) and many (pairs sorted by expert, products on the matrix
    cores): the same answer, the plain implementation's."""
    from vt_transformer_amd.parts import FEED_FORWARDS
    rt = runtime(dtype)
    ff = FEED_FORWARDS.build(PartSpec("expert_mixture", dict(num_experts=experts, top=top, intermediate_size=inter,
                                                             score="sigmoid", renormalize=False, weight_on="input",
                                                             activation="silu")), rt=rt, width=width, prefix="f.")
    w = weights_for(ff, 12, 0.3)
    ff.load(w.__getitem__, rt)
    wd = {k: v.double() for k, v in w.items()}
    for rows in (1, 3, 7, 30, 150, 700):
        x = (torch.randn(rows, width, generator=torch.Generator().manual_seed(rows)) * 1.2).to(dtype)
        got = ff.forward(x.to(DEV)).float().cpu().clone()
        ref = pk.expert_mixture(x.double(), wd, "f.", experts, top)
        assert rel(got, ref) < PART_TOL[dtype], rows
        if rows == 150:                      # every expert was somebody's choice
            chosen = torch.topk(torch.sigmoid(x.double() @ wd["f.router"].T), top, dim=-1).indices
            assert len(set(chosen.flatten().tolist())) == experts


def test_the_router_decides_and_the_score_scales_the_input():
    """A router whose rows are unit vectors: token t, which is e_j times a size, goes to expert j alone, with the score
    sigmoid(size) on its input (an expert is not linear, so a score on the output would give another number)."""
    from vt_transformer_amd.parts import FEED_FORWARDS
    rt = runtime(torch.float32)
    experts, width, inter = 6, 32, 24
    ff = FEED_FORWARDS.build(PartSpec("expert_mixture", dict(num_experts=experts, top=1, intermediate_size=inter)), rt=rt,
                             width=width, prefix="f.")
    w = weights_for(ff, 2, 0.6)
    w["f.router"] = torch.eye(width)[:experts].clone()
    ff.load(w.__getitem__, rt)
    for rows in (6, 60):
        x = torch.zeros(rows, width)
        sizes = torch.linspace(0.5, 3.0, rows)
        for i in range(rows):
            x[i, i % experts] = sizes[i]
        got = ff.forward(x.to(DEV)).double().cpu()
        for i in range(rows):
            e, s = i % experts, torch.sigmoid(sizes[i].double())
            xe = s * x[i].double()
            gt = xe @ w[f"f.e{e}.gate"].double().T
            want = ((gt * torch.sigmoid(gt)) * (xe @ w[f"f.e{e}.up"].double().T)) @ w[f"f.e{e}.down"].double().T
            assert torch.allclose(got[i], want, rtol=1e-4, atol=1e-6), i


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows", [1, 5, 70, 300])
def test_gated_unit_with_the_tanh_form_of_gelu(dtype, rows):
    from vt_transformer_amd.parts import FEED_FORWARDS
    rt = runtime(dtype)
    width, inter = 72, 104
    ff = FEED_FORWARDS.build(PartSpec("gated_mlp", dict(intermediate_size=inter, activation="gelu_tanh", weight_suffix="",
                                                        names={"gate": "gate", "up": "up", "down": "down"})),
                             rt=rt, width=width, prefix="f.")
    w = weights_for(ff, 12, 0.3)
    ff.load(w.__getitem__, rt)
    x = (torch.randn(rows, width, generator=torch.Generator().manual_seed(13)) * 1.5).to(dtype)
    got = ff.forward(x.to(DEV))
    assert rel(got, pk.dense_mlp(x.double(), {k: v.double() for k, v in w.items()}, "f.")) < PART_TOL[dtype]


@pytest.mark.parametrize("streams,width", [(1, 40), (2, 192), (3, 96), (4, 2048), (8, 100), (2, 4100)])
def test_streams_are_read_mixed_and_written(streams, width):
    """The kernels around a sublayer against their formulas: the weighted sum of the streams through the norm (whole
    batch and chosen rows), and the gated result going back into every stream while the streams are mixed."""
    from vt_transformer_amd.kernels import ops
    g = torch.Generator().manual_seed(streams * 1000 + width)
    n = 37
    x = torch.randn(n, streams, width, generator=g)
    w_in, w_out = torch.rand(streams, generator=g) + 0.3, torch.rand(streams, generator=g) + 0.3
    mix = torch.eye(streams) * 0.8 + torch.randn(streams, streams, generator=g) * 0.25
    gain = 1.0 + torch.randn(width, generator=g) * 0.3
    rows = torch.tensor([36, 0, 5, 5, 17], dtype=torch.int32)
    xd = x.to(DEV)
    for out_dtype in (torch.float32, torch.bfloat16):
        u = torch.einsum("s,nsw->nw", w_in.double(), x.double())
        ref = u * torch.rsqrt((u * u).mean(-1, keepdim=True) + 1e-5) * gain.double()
        got = ops.streams_read(xd, w_in.to(DEV), gain.to(DEV), torch.empty(n, width, dtype=out_dtype, device=DEV), 1e-5)
        assert rel(got, ref) < PART_TOL[out_dtype]
        got = ops.streams_read(xd, w_in.to(DEV), gain.to(DEV), torch.empty(5, width, dtype=out_dtype, device=DEV), 1e-5,
                               rows=rows.to(DEV))
        assert rel(got, ref[rows.long()]) < PART_TOL[out_dtype]
    for y_dtype in (torch.float32, torch.bfloat16):
        y, gate = torch.randn(n, width, generator=g).to(y_dtype), torch.randn(n, width, generator=g).to(y_dtype)
        for gt in (gate, None):
            yy = y.double() * (torch.sigmoid(gate.double()) if gt is not None else 1.0)
            ref = torch.einsum("st,nsw->ntw", mix.double(), x.double()) + w_out.double()[None, :, None] * yy[:, None, :]
            xc = xd.clone()
            ops.streams_write(xc, mix.to(DEV), w_out.to(DEV), y.to(DEV), gt.to(DEV) if gt is not None else None)
            assert rel(xc, ref) < 3e-6


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_token_shift_across_portions_and_entries(dtype):
    """Three requests side by side in portions of unequal sizes (single tokens among them): every token blends with
    the one before it in its own sequence, across steps through the request's state row, and a sequence's first token
    with zeros, also in a slot that another request has just left."""
    from vt_transformer_amd.engine.step import ModelRunner, StepEntry
    from vt_transformer_amd.kernels import ops
    from vt_transformer_amd.parts import MIXERS
    rt = runtime(dtype)
    width = 40
    mixer = MIXERS.build(PartSpec("general_delta", dict(num_heads=1, key_dim=8, decay_rank=2, norm_eps=1e-6)), rt=rt,
                         width=width, prefix="a.", shared={})           # (any mixer with a state row; the first 40 floats are used)
    runner = ModelRunner(OneMixer(mixer), rt, 16, 256, 3, 256)
    g = torch.Generator().manual_seed(1)
    mu = torch.rand(width, generator=g)
    seqs = {r: torch.randn(n, width, generator=g).to(dtype) for r, n in (("a", 23), ("b", 9), ("c", 14), ("d", 6))}
    plan = [[("a", 5), ("b", 1)], [("a", 1), ("b", 2), ("c", 7)], [("b", 6), ("c", 1)], [("a", 17), ("c", 6), ("d", 2)],
            [("d", 1)], [("d", 3)]]
    done = {r: 0 for r in seqs}
    got = {r: [] for r in seqs}
    live = set()
    for step in plan:
        for r, _ in step:
            if r not in live:
                assert runner.admit(r)
                live.add(r)
        assert runner.cache.reserve([(r, done[r] + n) for r, n in step])
        fresh = [runner.cache.get(r).slot for r, _ in step if runner.cache.get(r).fresh]
        if fresh:
            runner.storage.clear_state(fresh)
        ctx = runner.build_context([StepEntry(r, [0] * n, []) for r, n in step])
        h = torch.cat([seqs[r][done[r]:done[r] + n] for r, n in step]).to(DEV).contiguous()
        out = ops.token_shift(h, mu.to(DEV), runner.storage.state[0][:, :width], ctx.tok_entry, ctx.entry_start, ctx.state_slots,
                              torch.empty_like(h)).float().cpu()
        at = 0
        for r, n in step:
            got[r].append(out[at:at + n])
            at += n
            done[r] += n
            runner.cache.commit(r, done[r])
            if done[r] == len(seqs[r]):
                runner.release(r)
                live.discard(r)
    for r, h in seqs.items():
        assert rel(torch.cat(got[r]), pk.token_shift(h.double(), mu.double())) < (1e-6 if dtype == torch.float32 else 1e-2), r


# ---------------------------------------------------------------------------
# whole models: schedules against the plain implementation
# ---------------------------------------------------------------------------
LENGTHS = [61, 1, 23, 90, 2, 47]


@pytest.mark.parametrize("name,dtype", [(n, d) for n in "ABCD" for d in ("float32", "bfloat16")]
                         + [(n + "-dense", "bfloat16") for n in "ABCD"])
def test_schedules(folders, name, dtype):
    """Whole prompts; most of a prompt and then its last tokens one by one; portions of changing sizes down to two
    tokens; unequal requests side by side with three slots and few pages, so that both are used again."""
    folder, vocab = folders[name], CONFIGS[name[0]]["vocab"]
    reqs = rh.random_requests(vocab, LENGTHS, seed=3)
    cache = {}
    runner = make_runner(folder, dtype, pool_tokens=256, max_requests=3)
    runner.decode_graphs = True
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
        # a position's logits do not depend on the cut, the batch, the pages or the slots
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
                assert float(np.abs(rows[0] - r).max()) <= 2e-5 * float(np.abs(rows[0]).max()), f"{key} depends on the schedule"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_across_pages(folders, dtype):
    folder, vocab = folders["A" if dtype == "float32" else "A-dense"], CONFIGS["A"]["vocab"]
    reqs = rh.random_requests(vocab, [150], seed=9)
    steps = rh.trace_alone(reqs, {"r0": [(0, 5)] + [(i, i + 1) for i in range(5, 150)]})
    runner = make_runner(folder, dtype, pool_tokens=192, max_requests=1)
    runner.decode_graphs = True
    check_logits(folder, reqs, steps, rh.run_in_process(runner, steps), dtype)
    assert sum(runner.cache.available_pages()) == sum(p.num_pages for p in runner.cache.pools)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_many_tokens_at_once_take_the_grouped_experts(tmp_path, dtype):
    """A prompt of some hundred tokens (experts on the matrix cores in bfloat16, many keys behind every query, a delta
    rule over many tokens in one launch) against the same prompt in small portions."""
    cfg = {"architecture": "Kigalix", "vocab": 90, "width": 64, "streams": 2, "norm": {"eps": 1e-6},
           "layers": [delta_layer(heads=2, dim=32, rank=8, mlp=moe(8, 2, 24)),
                      latent_layer(heads=4, dim=16, rot_dim=16, vdim=16, rank=32, mlp=moe(4, 1, 48)),
                      latent_layer(heads=2, dim=32, rot_dim=8, vdim=24, rank=16, gated=True, scaling=(4.0, 128, 8.0, 1.0),
                                   mlp=dense(96))]}
    folder = write_model(cfg, str(tmp_path / "m"), seed=77)
    reqs = rh.random_requests(90, [300, 170], seed=2)
    runner = make_runner(folder, dtype, pool_tokens=512, max_requests=2)
    cache = {}
    whole = rh.trace_alone(reqs, {r: [(0, len(t))] for r, t in reqs.items()})
    check_logits(folder, reqs, whole, rh.run_in_process(runner, whole), dtype, cache)
    mixed = rh.trace_mixed(reqs, {r: rh.cut(t, [130, 2, 1, 64, 1, 1, 50]) for r, t in reqs.items()}, max_live=2, seed=4)
    check_logits(folder, reqs, mixed, rh.run_in_process(runner, mixed), dtype, cache)


def test_captured_decoding_steps_equal_launched_ones(folders):
    """bfloat16: the same decoding steps through captured graphs and launch by launch, bit for bit (two requests: the
    state rows and tables of two entries are in play)."""
    folder, vocab = folders["A"], CONFIGS["A"]["vocab"]
    reqs = rh.random_requests(vocab, [40, 25], seed=19)
    portions = {r: [(0, len(t) - 16)] + [(i, i + 1) for i in range(len(t) - 16, len(t))] for r, t in reqs.items()}
    steps = rh.trace_mixed(reqs, portions, max_live=2, seed=1, skip_prob=0.0)
    got = []
    for graphs in (False, True):
        runner = make_runner(folder, "bfloat16", pool_tokens=128, max_requests=2)
        runner.decode_graphs = graphs
        got.append(rh.run_in_process(runner, steps))
        assert bool(runner._graphs) == graphs
    assert all(np.array_equal(got[0][k], got[1][k]) for k in got[0])
    check_logits(folder, reqs, steps, got[1], "bfloat16")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_generation_through_the_engine(folders, dtype):
    """Greedy tokens through Engine.generate (scheduler with short portions, two slots for three requests)."""
    from vt_transformer_amd.engine import Engine
    from vt_transformer_amd.sampling import SamplingParams
    folder = folders["C" if dtype == "float32" else "C-dense"]
    cfg, w = pk.read_folder(folder)
    prompts = [r for r in rh.random_requests(cfg["vocab"], [19, 3, 41], seed=21).values()]
    eng = Engine(folder, dtype=dtype, num_pages=16, max_running_reqs=2, max_seq_len=128, chunk_size=16, max_extend_tokens=24)
    got = eng.generate(prompts, SamplingParams(max_tokens=8, ignore_eos=True))
    for p, g in zip(prompts, got):
        assert len(g) == 8
        if dtype == "float32":
            assert g == pk.greedy(cfg, w, p, 8)
        else:
            logits = pk.forward(cfg, w, p + g)
            for i, tok in enumerate(g):
                row = logits[len(p) - 1 + i]
                assert float(row.max() - row[tok]) <= 3e-2 * float(row.abs().max())


def test_trace_run_with_a_kigalix_folder(folders, tmp_path):
    folder, vocab = folders["B"], CONFIGS["B"]["vocab"]
    reqs = rh.random_requests(vocab, [40, 9, 27], seed=17)
    steps = rh.trace_mixed(reqs, {r: rh.cut(t, [6, 2, 11, 1]) for r, t in reqs.items()}, max_live=2, seed=2)
    got = rh.run_trace_run(folder, "float32", steps, str(tmp_path / "out"), rh.max_live_tokens(steps), vocab,
                           extra_args=("--max-requests", "2"))
    check_logits(folder, reqs, steps, got, "float32")


# ---------------------------------------------------------------------------
# configurations drawn at random
# ---------------------------------------------------------------------------
def random_kigalix_config(seed: int) -> dict:
    rs = np.random.RandomState(seed)
    pick = lambda xs: xs[rs.randint(len(xs))]      # noqa: E731
    width = int(pick([24, 40, 52, 64, 96, 100, 136]))       # (52, 100: no multiples of 8)
    layers = []
    for _ in range(rs.randint(2, 6)):
        kind = pick([None, "dense", "moe", "moe"])
        if kind == "dense":
            mlp = dense(int(pick([24, 56, 100])))
        elif kind == "moe":
            experts = int(pick([1, 2, 3, 8, 12]))
            mlp = moe(experts, int(pick([k for k in (1, 2, 3, 4) if k <= experts])), int(pick([8, 24, 40, 52])))
        else:
            mlp = None
        u = rs.rand()
        if u < 0.4:
            layers.append(delta_layer(heads=int(pick([1, 2, 3, 6])), dim=int(pick([8, 16, 20, 32, 64])),
                                      rank=int(pick([1, 4, 16, 24])), mlp=mlp))
        else:
            rot_dim = int(pick([0, 4, 16, 32]))
            dim = int(pick([8, 16, 20, 64]))
            layers.append(latent_layer(heads=int(pick([1, 2, 4, 5, 8])), dim=dim, rot_dim=rot_dim, vdim=int(pick([8, 12, 32, 80])),
                                       rank=int(pick([12, 16, 32, 48, 80])),
                                       scale=float(pick([0.5, 1.0, 2.0])) / math.sqrt(dim + rot_dim),
                                       base=float(pick([10.0, 1e4, 5e5])), gated=u > 0.7,
                                       scaling=(float(pick([2.0, 8.0, 32.0])), int(pick([16, 64, 1024])), float(pick([4.0, 32.0])),
                                                float(pick([1.0, 2.0]))) if u > 0.7 and rot_dim else None, mlp=mlp))
    cfg = {"architecture": "Kigalix", "vocab": int(pick([17, 100, 257])), "width": width,
           "norm": {"eps": float(pick([1e-6, 1e-5, 1e-3]))}, "layers": layers}
    streams = pick([None, 1, 2, 3, 4, 5])
    if streams is not None:
        cfg["streams"] = int(streams)
    return cfg


@pytest.mark.parametrize("seed", range(8))
def test_configurations_drawn_at_random(tmp_path, seed):
    cfg = random_kigalix_config(seed)
    folder = write_model(cfg, str(tmp_path / "m"), seed=100 + seed, idle=bool(seed % 2))
    dense_folder = write_model(without_experts(cfg), str(tmp_path / "d"), seed=200 + seed)
    reqs = rh.random_requests(cfg["vocab"], [70, 33, 5], seed=seed)
    for folder, dtype in ((folder, "float32"), (folder, "bfloat16"), (dense_folder, "bfloat16")):
        runner = make_runner(folder, dtype, pool_tokens=192, max_requests=2)
        runner.decode_graphs = True
        cache = {}
        whole = rh.trace_alone(reqs, {r: [(0, len(t))] for r, t in reqs.items()})
        check_logits(folder, reqs, whole, rh.run_in_process(runner, whole), dtype, cache)
        mixed = rh.trace_mixed(reqs, {r: rh.cut(t, [11, 2, 1, 1, 17, 1, 1, 3]) for r, t in reqs.items()}, max_live=2, seed=seed)
        check_logits(folder, reqs, mixed, rh.run_in_process(runner, mixed), dtype, cache)
