"""Gabelorn on the GPU against the plain implementation (plain_gabelorn.py): each mechanism alone, prompts against
token-by-token decoding, portions down to two tokens, unequal batches, pages and slots used again, keys far back and at
the edges of windows and pages, sinks, long decoding, generation through the engine and through bin/trace_run."""
import copy
import math
from types import SimpleNamespace

import numpy as np
import pytest
import torch

import plain_gabelorn as pg
import replay_helpers as rh
from gabelorn_helpers import CONFIGS, TOL, attention_layer, check_logits, latent_layer, write_model
from test_parts_gpu import DEV, OneMixer, rel, runtime
from vt_transformer_amd.config.base import PartSpec, ScheduleEntry

pytestmark = pytest.mark.gpu
PART_TOL = {torch.float32: 1e-5, torch.bfloat16: 2.5e-2}
LATENT_NAMES = {"q": "q", "dkv": "dkv", "dkv_norm": "dkv.norm", "uk": "uk", "uv": "uv", "o": "o", "g": "g", "sink": "sink"}
ATTN_NAMES = {"q": "q", "k": "k", "v": "v", "o": "o", "sink": "sink", "vmix": "vmix"}
CUTS = [(0, 20), (20, 21), (21, 23), (23, 70), (70, 71), (71, 83)]


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    root = tmp_path_factory.mktemp("gabelorn")
    return {k: write_model(copy.deepcopy(cfg), str(root / k), seed=31 + i) for i, (k, cfg) in enumerate(CONFIGS.items())}


def make_runner(folder, dtype, pool_tokens, max_requests=4, page_size=16, max_seq_len=None):
    from vt_transformer_amd.engine import load_model, make_runner as mk
    model = load_model(folder, dtype, page_size=page_size)
    return mk(model, pool_tokens=pool_tokens, page_size=page_size, max_requests=max_requests,
              max_seq_len=max_seq_len or pool_tokens)


def weights_for(part, seed, scale):
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, decl in part.tensors().items():
        t = torch.randn(decl.shape, generator=g) * (scale if decl.role == "matrix" else 0.4)
        if decl.role == "gain":
            t += 1.0
        if name.endswith("sink"):
            t = t * 3.0 + 1.0
        if name.endswith("vmix"):
            t = torch.rand(decl.shape, generator=g) * 0.8 + 0.1
        out[name] = t.to(torch.bfloat16).float()
    return out


class Mixers:
    """The least a ModelRunner needs to give some mixers, one per layer, caches and a context."""

    def __init__(self, mixers, vocab=100):
        self.schedule = [ScheduleEntry(i) for i in range(len(mixers))]
        self.layers = [SimpleNamespace(mixer=m) for m in mixers]
        self.spec = SimpleNamespace(vocab_size=vocab)


def step_parts(runner, mixers, xs, cuts):
    """Mixer i over xs[i] [T, width] of one request, all in the same steps, in the portions `cuts`."""
    from vt_transformer_amd.engine.step import StepEntry
    runner.admit("r")
    outs = [[] for _ in mixers]
    for a, b in cuts:
        assert runner.cache.reserve([("r", b)])
        ctx = runner.build_context([StepEntry("r", [0] * (b - a), [])])
        caches = runner.storage.layer_caches(ctx.block_tables)
        for i, m in enumerate(mixers):
            outs[i].append(m.forward(xs[i][a:b].to(DEV).contiguous(), ctx, caches[i], None).float().cpu().clone())
        runner.cache.commit("r", b)
    runner.release("r")
    return [torch.cat(o) for o in outs]


# ---------------------------------------------------------------------------
# the mechanisms alone
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nh,dn,dr,dv,rank,rot,window,sink,gate", [
    (8, 16, 16, 24, 32, 8, 20, True, True),      # eight heads on one cache: a block's waves share keys; half the part rotated
    (3, 20, 12, 10, 24, 12, 0, True, True),      # sizes that are no multiples of 16, every earlier key
    (5, 48, 16, 40, 48, 16, 37, False, False),   # no sink, no gate
    (1, 8, 16, 8, 16, 16, 1, True, False),       # one head that sees itself alone
    (2, 24, 0, 40, 48, 0, 16, True, True),       # nothing rotated
    (2, 16, 32, 8, 320, 32, 50, True, True),     # a low-rank vector wider than the matrix-core kernels take
    (20, 16, 16, 8, 16, 16, 30, True, True),     # more heads than the 16 rows of a decoding product: two tiles of heads
])
def test_latent_attention_part(dtype, nh, dn, dr, dv, rank, rot, window, sink, gate):
    from vt_transformer_amd.engine.step import ModelRunner
    from vt_transformer_amd.parts import MIXERS
    rt = runtime(dtype)
    width, t = 72, 83
    pos_spec = PartSpec("rotary", {"theta": 300.0, "dim": rot, "scaling": None}) if rot else None
    mixer = MIXERS.build(PartSpec("latent_attention", dict(
        num_heads=nh, plain_dim=dn, rot_dim=dr, value_dim=dv, rank=rank, norm_eps=1e-5, position=pos_spec, scale=0.3,
        window=window, sink=sink, out_gate=gate, names=dict(LATENT_NAMES))), rt=rt, width=width, prefix="a.", shared={})
    assert mixer.cache_need().tensors[0].token_shape == (1, rank + dr) and mixer.cache_need().tensors[1].token_shape == (1, rank)
    assert mixer.cache_need().window == window
    w = weights_for(mixer, 3, 0.3)
    mixer.load(w.__getitem__, rt)
    runner = ModelRunner(OneMixer(mixer), rt, 16, 256, 4, 256)
    x = (torch.randn(t, width, generator=torch.Generator().manual_seed(4)) * 0.7).to(dtype)
    got = step_parts(runner, [mixer], [x], CUTS)[0]
    wd = {k: v.double() for k, v in w.items()}
    factor = 1.0
    if not gate:            # the plain mixer always gates: a gate of zeros halves, and the output product is linear
        wd["a.g"], factor = torch.zeros(nh * dv, width, dtype=torch.float64), 2.0
    m = {"heads": nh, "dim": dn, "rot_dim": dr, "vdim": dv, "kv_rank": rank, "scale": 0.3}
    if window:
        m["mask"] = {"size": window}
    if rot:
        m["rot"] = {"dims": rot, "base": 300.0}
    ref = factor * pg.latent_attention_mixer(x.double(), wd, "a.", m, 1e-5, torch.arange(t))
    assert rel(got, ref) < PART_TOL[dtype]
    if dtype == torch.float32:      # the same operations whatever the cut
        assert torch.equal(got, step_parts(runner, [mixer], [x], [(0, t)])[0])
        assert torch.equal(got, step_parts(runner, [mixer], [x], [(0, 50)] + [(i, i + 1) for i in range(50, t)])[0])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nh,kvh,d,dv,q_temp", [
    (4, 2, 32, 48, (0.3, 5)),
    (6, 6, 16, 16, (0.6, 1)),
    (8, 2, 32, 48, None),          # four query heads to a key/value head: a block's waves share keys
    (2, 1, 24, 40, (0.2, 64)),     # heads that are no multiples of 16
])
def test_slope_attention_with_sinks_and_mixed_values(dtype, nh, kvh, d, dv, q_temp):
    """Three layers on the same steps: the first leaves its values, the second and third mix them into theirs."""
    from vt_transformer_amd.engine.step import ModelRunner
    from vt_transformer_amd.parts import MIXERS
    rt = runtime(dtype)
    width, t = 72, 83
    mixers, ws = [], []
    for i, role in enumerate(["source", "mix", "mix"]):
        mx = MIXERS.build(PartSpec("masked_attention", dict(
            num_heads=nh, num_kv_heads=kvh, key_dim=d, value_dim=dv, scale=0.4, sink=True, distance_slopes=8.0,
            q_temp={"coef": q_temp[0], "every": q_temp[1]} if q_temp else None, value_mix=role, names=dict(ATTN_NAMES))),
            rt=rt, width=width, prefix=f"m{i}.", shared={})
        w = weights_for(mx, 10 + i, 0.3)
        mx.load(w.__getitem__, rt)
        mixers.append(mx)
        ws.append(w)
    runner = ModelRunner(Mixers(mixers), rt, 16, 256, 4, 256)
    g = torch.Generator().manual_seed(4)
    xs = [(torch.randn(t, width, generator=g) * 0.7).to(dtype) for _ in mixers]
    got = step_parts(runner, mixers, xs, CUTS)
    m = {"heads": nh, "kv_heads": kvh, "dim": d, "vdim": dv, "scale": 0.4, "v_mix": True}
    if q_temp:
        m["q_temp"] = {"coef": q_temp[0], "every": q_temp[1]}
    shared = {}
    for i in range(3):
        wd = {k: v.double() for k, v in ws[i].items()}
        ref = pg.slope_attention_mixer(xs[i].double(), wd, f"m{i}.", m, torch.arange(t), shared)
        assert rel(got[i], ref) < PART_TOL[dtype], f"layer {i}"
    if dtype == torch.float32:
        again = step_parts(runner, mixers, xs, [(0, 50)] + [(i, i + 1) for i in range(50, t)])
        assert all(torch.equal(a, b) for a, b in zip(got, again))


def _attention_rows(y, nh, kvh, d, dv, sink, slopes, window):
    """Plain attention over prepared rows y [T, q heads | k heads | v heads] in float64."""
    t = y.shape[0]
    yd = y.double()
    q = yd[:, :nh * d].reshape(t, nh, d)
    k = yd[:, nh * d:(nh + kvh) * d].reshape(t, kvh, d).repeat_interleave(nh // kvh, dim=1)
    v = yd[:, (nh + kvh) * d:].reshape(t, kvh, dv).repeat_interleave(nh // kvh, dim=1)
    dist = torch.arange(t)[:, None] - torch.arange(t)[None, :]
    seen = dist >= 0
    if window:
        seen = seen & (dist < window)
    s = torch.einsum("ihd,jhd->hij", q, k)
    if slopes is not None:
        s = s - slopes.double()[:, None, None] * dist.double()[None]
    a = pg.sink_softmax(s, seen, sink.double() if sink is not None else None)
    return torch.einsum("hij,jhd->ihd", a, v).reshape(t, nh * dv)


@pytest.mark.parametrize("dtype,matrix", [(torch.float32, False), (torch.bfloat16, False), (torch.bfloat16, True)])
def test_one_key_far_back_against_a_sink_and_slopes(dtype, matrix):
    """Queries and keys are made so that one key far back (the last slot of the second page, hundreds of keys before
    the end) takes all the weight that the sink leaves it: the sink equals that key's score, so a position d behind
    it gets value / (1 + exp(slope_h d)), in a prompt's portion and decoded alone.  A sink left out doubles the result,
    a slope left out flattens it, a key lost zeroes it."""
    from vt_transformer_amd.engine.step import ModelRunner, StepEntry
    from vt_transformer_amd.kernels import ops
    from vt_transformer_amd.parts import MIXERS
    from vt_transformer_amd.parts.masked_attention import TILES_KEY, head_slopes
    rt = runtime(dtype)
    nh, kvh, d, dv = (4 if matrix else 2), 1, 16, 16
    mixer = MIXERS.build(PartSpec("masked_attention", dict(num_heads=nh, num_kv_heads=kvh, key_dim=d, value_dim=dv, scale=1.0)),
                         rt=rt, width=8, prefix="a.", shared={})
    runner = ModelRunner(OneMixer(mixer), rt, 16, 1024, 2, 1024)
    t, star = 700, 31
    g = torch.Generator().manual_seed(5)
    y = torch.randn(t, (nh + kvh) * d + kvh * dv, generator=g) * 0.1
    y[:, :nh * d] = 0
    for hh in range(nh):
        y[:, hh * d] = 6.0                 # every query points along element 0 ...
    y[star, nh * d] = 6.0                  # ... and so does the one key: score 36 against about 0
    y[star, (nh + kvh) * d:] = 50.0
    sink = torch.full((nh,), 36.0, device=DEV)
    slopes = torch.from_numpy(head_slopes(nh, 8.0)).to(DEV)
    for cuts in ([(0, t)], [(0, 300), (300, 463), (463, 464), (464, 465), (465, 466), (466, t)]):
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
            if matrix and b - a > 1:
                ops.attention_masked_mfma(q, cache["k"], cache["v"], ctx.positions, ctx.tok_entry, cache.block_table,
                                          ctx.extra[TILES_KEY], out, nh, kvh, d, dv, 1.0, sink=sink, slopes=slopes)
            elif matrix:                    # single tokens: the kernel whose rows are heads and whose keys are dealt out
                for splits in (1, 3):
                    part = torch.empty(ops.attention_masked_decode_scratch(1, nh, kvh, dv, splits), device=DEV)
                    ops.attention_masked_decode(q, cache["k"], cache["v"], ctx.positions, ctx.tok_entry, cache.block_table,
                                                out, part, splits, nh, kvh, d, dv, 1.0, sink=sink, slopes=slopes)
                    if splits == 1:
                        first = out.clone()
                assert float((out.float() - first.float()).abs().max()) < 0.3       # (however the keys are dealt out)
            else:
                ops.attention_masked(q, cache["k"], cache["v"], ctx.positions, ctx.tok_entry, cache.block_table, out, nh, kvh,
                                     d, dv, 1.0, sink=sink, slopes=slopes)
            outs.append(out.float().cpu())
            runner.cache.commit("r", b)
        runner.release("r")
        got = torch.cat(outs).reshape(t, nh, dv)
        for hh in range(nh):
            for p in (star, star + 1, 464, 465, t - 1):
                want = 50.0 / (1.0 + math.exp(float(slopes[hh]) * (p - star)))
                assert abs(float(got[p, hh, 0]) - want) < 0.03 * want + 0.02, (hh, p, float(got[p, hh, 0]), want)
        assert float(got[:star].abs().max()) < 1.0
        ref = _attention_rows(y.to(dtype), nh, kvh, d, dv, sink.cpu(), slopes.cpu(), 0)
        assert rel(got.reshape(t, -1), ref) < PART_TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nh", [2, 4])       # (four heads on the one cache: the matrix-core kernel whose waves share keys)
def test_latent_window_edges_at_a_page_border(dtype, nh):
    """The whole latent mixer with weights that pass its input through: one token's low-rank vector points along
    element 0 and every query asks for element 0, so the positions that still see it return it and the first one
    outside the window returns nothing of it; the token sits in the last slot of a page and the window ends inside
    another; in one portion, in portions that end at both edges, and decoded one by one."""
    from vt_transformer_amd.engine.step import ModelRunner
    from vt_transformer_amd.parts import MIXERS
    rt = runtime(dtype)
    rank, dr, window, t, star = 16, 16, 40, 150, 47
    qcols, ccol = nh * (rank + dr), nh * (rank + dr)
    gcol = ccol + rank + dr
    width = gcol + nh * rank
    mixer = MIXERS.build(PartSpec("latent_attention", dict(
        num_heads=nh, plain_dim=rank, rot_dim=dr, value_dim=rank, rank=rank, norm_eps=1e-6, scale=1.0, window=window,
        position=PartSpec("rotary", {"theta": 100.0, "dim": dr, "scaling": None}), sink=True, out_gate=True,
        names=dict(LATENT_NAMES))), rt=rt, width=width, prefix="a.", shared={})
    eye = torch.eye(width)
    w = {"a.q": eye[:qcols], "a.dkv": eye[ccol:gcol], "a.g": eye[gcol:], "a.dkv.norm": torch.ones(rank),
         "a.uk": torch.eye(rank).repeat(nh, 1), "a.uv": torch.eye(rank).repeat(nh, 1), "a.sink": torch.full((nh,), -20.0),
         "a.o": torch.cat([torch.eye(nh * rank), torch.zeros(width - nh * rank, nh * rank)])}
    mixer.load(w.__getitem__, rt)
    runner = ModelRunner(OneMixer(mixer), rt, 16, 256, 2, 256)
    g = torch.Generator().manual_seed(6)
    x = torch.zeros(t, width)
    for hh in range(nh):
        x[:, hh * (rank + dr)] = 6.0                     # every head's query: element 0 of the unrotated part
    x[:, ccol + 1:ccol + rank] = torch.randn(t, rank - 1, generator=g)      # low-rank vectors without element 0 ...
    x[star, ccol:ccol + rank] = 0.0
    x[star, ccol] = 1.0                                                      # ... but one, which is nothing else
    x[:, gcol:] = 30.0                                                       # gates wide open
    x = x.to(dtype)
    last = star + window - 1                # the last position that sees it
    height = math.sqrt(rank)                # what the norm makes of it
    for cuts in ([(0, t)], [(0, 30), (30, last), (last, last + 1), (last + 1, last + 3), (last + 3, t)],
                 [(0, 60)] + [(i, i + 1) for i in range(60, 100)] + [(100, t)]):
        got = step_parts(runner, [mixer], [x], cuts)[0].reshape(t, -1)[:, :nh * rank].reshape(t, nh, rank)
        assert float(got[star:last + 1, :, 0].min()) > 0.97 * height, "a position inside the window lost the key"
        assert float(got[last + 1:, :, 0].abs().max()) < 0.05, "a position outside the window saw the key"
        assert float(got[:star, :, 0].abs().max()) < 0.05


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n,heads,n_in,n_out,transposed,gated", [
    (1, 3, 20, 24, False, True), (9, 8, 128, 48, False, False), (70, 2, 16, 100, True, True), (33, 5, 44, 12, True, False),
    (200, 4, 64, 64, False, True), (2100, 16, 128, 40, False, True), (1030, 32, 100, 48, False, False),   # (many tokens: 32 to a wave)
])
def test_per_head_products(dtype, n, heads, n_in, n_out, transposed, gated):
    """One small matrix per head, from and into columns of wider rows, in either orientation, with and without the gate;
    float32 inputs to 16-bit results as well (what a few-row product hands on)."""
    from vt_transformer_amd.kernels import ops
    g = torch.Generator().manual_seed(n + heads)
    x_cols, y_cols, x_head, y_head = 8 + heads * (n_in + 4), 4 + heads * (n_out + 8), n_in + 4, n_out + 8
    w = (torch.randn(heads, n_out, n_in, generator=g) / n_in ** 0.5).to(torch.bfloat16).float()
    gate = torch.randn(n, 12 + heads * n_out, generator=g)
    for x_dtype in ({torch.float32, dtype}):
        x = torch.randn(n, x_cols, generator=g).to(x_dtype)
        y = torch.zeros(n, y_cols, dtype=dtype, device=DEV)
        wd = (w.transpose(1, 2).contiguous() if transposed else w).reshape(-1, n_out if transposed else n_in).to(dtype).to(DEV)
        ops.head_linear(x.to(DEV), 8, x_head, wd, transposed, y, 4, y_head, heads, n_in, n_out,
                        gate=gate.to(x_dtype).to(DEV) if gated else None, gate_column=12)
        xs = x.double()[:, 8:8 + heads * x_head].reshape(n, heads, x_head)[:, :, :n_in]
        ref = torch.einsum("hoi,nhi->nho", w.double(), xs)
        if gated:
            ref = ref * torch.sigmoid(gate.to(x_dtype).double()[:, 12:12 + heads * n_out].reshape(n, heads, n_out))
        got = y.float().cpu()[:, 4:4 + heads * y_head].reshape(n, heads, y_head)
        assert rel(got[:, :, :n_out], ref) < PART_TOL[dtype]
        assert float(got[:, :, n_out:].abs().max()) == 0.0 and float(y[:, :4].abs().max()) == 0.0    # nothing beside its columns


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows", [1, 5, 70, 300])
def test_bounded_gated_feed_forward(dtype, rows):
    from vt_transformer_amd.parts import FEED_FORWARDS
    rt = runtime(dtype)
    width, inter = 72, 104
    ff = FEED_FORWARDS.build(PartSpec("gated_mlp", dict(
        intermediate_size=inter, act_alpha=1.702, act_limit=0.9, up_shift=1.0, weight_suffix="", bias_suffix=".b",
        names={"gate": "gate", "up": "up", "down": "down"})), rt=rt, width=width, prefix="f.")
    w = weights_for(ff, 12, 0.3)
    ff.load(w.__getitem__, rt)
    x = (torch.randn(rows, width, generator=torch.Generator().manual_seed(13)) * 1.5).to(dtype)
    got = ff.forward(x.to(DEV))
    ref = pg.clamped_gated_mlp(x.double(), {k: v.double() for k, v in w.items()}, "f.", 0.9)
    assert rel(got, ref) < PART_TOL[dtype]
    gate = x.double() @ w["f.gate"].double().t() + w["f.gate.b"].double()
    assert float((gate > 0.9).double().mean()) > 0.02       # the bound did cut


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_capped_logits(dtype):
    from vt_transformer_amd.parts import HEADS
    rt = runtime(dtype)
    head = HEADS.build(PartSpec("linear_head", {"name": "head", "softcap": 2.0}), rt=rt, width=64, vocab_size=301)
    w = {"head": (torch.randn(301, 64, generator=torch.Generator().manual_seed(1)) * 0.5).to(torch.bfloat16).float()}
    head.load(w.__getitem__, rt, shared={})
    x = torch.randn(70, 64, generator=torch.Generator().manual_seed(2)).to(dtype)
    got = head.forward(x.to(DEV))
    ref = 2.0 * torch.tanh(x.double() @ w["head"].double().t() / 2.0)
    assert float(got.abs().max()) <= 2.0 and rel(got, ref) < PART_TOL[dtype]


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
            assert len(rows) == 4 and all(np.array_equal(rows[0], r) for r in rows[1:]), f"{key} depends on the schedule"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_across_windows_and_pages(folders, dtype):
    folder, vocab = folders["A"], CONFIGS["A"]["vocab"]
    reqs = rh.random_requests(vocab, [150], seed=9)
    steps = rh.trace_alone(reqs, {"r0": [(0, 5)] + [(i, i + 1) for i in range(5, 150)]})
    runner = make_runner(folder, dtype, pool_tokens=192, max_requests=1)
    runner.decode_graphs = True
    check_logits(folder, reqs, steps, rh.run_in_process(runner, steps), dtype)
    assert sum(runner.cache.available_pages()) == sum(p.num_pages for p in runner.cache.pools)


def test_pages_behind_a_window_are_given_back(tmp_path):
    """A model of latent layers alone runs a request longer than its pool of pages, because a token that no later
    position can see is dead; the plain logits still come out."""
    cfg = {"architecture": "Gabelorn", "vocab": 61, "width": 48, "norm": {"eps": 1e-5},
           "layers": [latent_layer(heads=2, dim=8, rot_dim=8, vdim=8, rank=16, window=23, ff=40),
                      latent_layer(heads=3, dim=16, rot_dim=4, vdim=12, rank=20, window=23)]}
    folder = write_model(cfg, str(tmp_path / "w"), seed=4)
    reqs = rh.random_requests(61, [140], seed=13)
    steps = rh.trace_alone(reqs, {"r0": rh.cut(reqs["r0"], [10])})
    runner = make_runner(folder, "float32", pool_tokens=96, max_requests=1, max_seq_len=160)
    check_logits(folder, reqs, steps, rh.run_in_process(runner, steps), "float32")


def test_captured_decoding_steps_equal_launched_ones(folders):
    """bfloat16: the same decoding steps through captured graphs and launch by launch, bit for bit (two requests, so
    that the value-mixing buffer and the tables of two entries are in play)."""
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
    folder = folders["C"]
    cfg, w = pg.read_folder(folder)
    prompts = [r for r in rh.random_requests(cfg["vocab"], [19, 3, 41], seed=21).values()]
    eng = Engine(folder, dtype=dtype, num_pages=16, max_running_reqs=2, max_seq_len=128, chunk_size=16, max_extend_tokens=24)
    got = eng.generate(prompts, SamplingParams(max_tokens=8, ignore_eos=True))
    for p, g in zip(prompts, got):
        assert len(g) == 8
        if dtype == "float32":
            assert g == pg.greedy(cfg, w, p, 8)
        else:
            logits = pg.forward(cfg, w, p + g)
            for i, tok in enumerate(g):
                row = logits[len(p) - 1 + i]
                assert float(row.max() - row[tok]) <= 3e-2 * float(row.abs().max())


def test_trace_run_with_a_gabelorn_folder(folders, tmp_path):
    folder, vocab = folders["B"], CONFIGS["B"]["vocab"]
    reqs = rh.random_requests(vocab, [40, 9, 27], seed=17)
    steps = rh.trace_mixed(reqs, {r: rh.cut(t, [6, 2, 11, 1]) for r, t in reqs.items()}, max_live=2, seed=2)
    got = rh.run_trace_run(folder, "float32", steps, str(tmp_path / "out"), rh.max_live_tokens(steps), vocab,
                           extra_args=("--max-requests", "2"))
    check_logits(folder, reqs, steps, got, "float32")


# ---------------------------------------------------------------------------
# configurations drawn at random
# ---------------------------------------------------------------------------
def random_gabelorn_config(seed: int) -> dict:
    rs = np.random.RandomState(seed)
    pick = lambda xs: xs[rs.randint(len(xs))]      # noqa: E731
    layers = []
    kv, vdim = pick([1, 2, 3]), pick([8, 16, 24, 40])
    for _ in range(rs.randint(2, 6)):
        ff = pick([None, 24, 56, 100])
        if rs.rand() < 0.45:
            rot_dim = pick([0, 4, 16, 32])
            dim = pick([8, 16, 20, 64])
            layers.append(latent_layer(heads=pick([1, 2, 4, 5, 8]), dim=dim, rot_dim=rot_dim,
                                       vdim=pick([8, 12, 32]), rank=pick([12, 16, 32, 48, 80]),
                                       scale=float(pick([0.5, 1.0, 2.0])) / math.sqrt(dim + rot_dim),
                                       window=pick([0, 1, 2, 15, 16, 17, 50, 400]),
                                       rot_dims=pick([d for d in (2, 4, 8, 16, 32) if d <= rot_dim]) if rot_dim else None,
                                       base=float(pick([10.0, 1e4, 1e6])), ff=ff, limit=float(pick([0.5, 1.5, 7.0])))
            )
        else:
            mix = bool(rs.rand() < 0.6)
            dim = pick([8, 16, 24, 64, 128])
            # (scores of about unit size at these weights: sharper ones magnify what bfloat16 rounds away)
            layers.append(attention_layer(heads=kv * pick([1, 2, 4]) if mix else pick([1, 3, 4, 8]),
                                          kv_heads=kv if mix else 1, dim=dim,
                                          vdim=vdim if mix else pick([8, 16, 48]), scale=float(pick([0.5, 1.0, 2.0])) / math.sqrt(dim),
                                          q_temp=pick([None, (0.2, 1), (0.25, 16), (1.0, 50)]), v_mix=mix, ff=ff,
                                          limit=float(pick([0.5, 1.5, 7.0]))))
    cfg = {"architecture": "Gabelorn", "vocab": int(pick([17, 100, 257])), "width": int(pick([24, 40, 64, 100])),
           "norm": {"eps": float(pick([1e-6, 1e-5, 1e-3]))}, "layers": layers}
    if rs.rand() < 0.7:
        cfg["logit_softcap"] = float(pick([5.0, 30.0]))
    return cfg


@pytest.mark.parametrize("seed", range(8))
def test_configurations_drawn_at_random(tmp_path, seed):
    cfg = random_gabelorn_config(seed)
    folder = write_model(cfg, str(tmp_path / "m"), seed=100 + seed)
    reqs = rh.random_requests(cfg["vocab"], [70, 33, 5], seed=seed)
    for dtype in ("float32", "bfloat16"):
        runner = make_runner(folder, dtype, pool_tokens=192, max_requests=2)
        runner.decode_graphs = True
        cache = {}
        whole = rh.trace_alone(reqs, {r: [(0, len(t))] for r, t in reqs.items()})
        check_logits(folder, reqs, whole, rh.run_in_process(runner, whole), dtype, cache)
        mixed = rh.trace_mixed(reqs, {r: rh.cut(t, [11, 2, 1, 1, 17, 1, 1, 3]) for r, t in reqs.items()}, max_live=2, seed=seed)
        check_logits(folder, reqs, mixed, rh.run_in_process(runner, mixed), dtype, cache)
