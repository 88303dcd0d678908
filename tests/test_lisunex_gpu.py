"""Lisunex on the GPU against the plain implementation (plain_lisunex.py): each mechanism alone, prompts against
token-by-token decoding, portions down to two tokens, unequal batches, pages and slots used again, chunk edges, long
decoding, generation through the engine and through bin/trace_run."""
import copy
import math

import numpy as np
import pytest
import torch

import plain_lisunex as pl
import replay_helpers as rh
from lisunex_helpers import CONFIGS, TOL, attention_layer, check_logits, delta_layer, write_model
from test_parts_gpu import DEV, OneMixer, rel, runtime
from vt_transformer_amd.config.base import PartSpec

pytestmark = pytest.mark.gpu
PART_TOL = {torch.float32: 1e-5, torch.bfloat16: 2.5e-2}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    root = tmp_path_factory.mktemp("lisunex")
    return {k: write_model(copy.deepcopy(cfg), str(root / k), seed=11 + i) for i, (k, cfg) in enumerate(CONFIGS.items())}


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
        out[name] = t.to(torch.bfloat16).float()
    return out


def step_part(runner, mixer, x, cuts, state=False):
    """The mixer alone over x [T, width] of one request, in the portions `cuts`."""
    from vt_transformer_amd.engine.step import StepEntry
    runner.admit("r")
    outs = []
    for a, b in cuts:
        assert runner.cache.reserve([("r", b)])
        if runner.cache.get("r").fresh:
            runner.storage.clear_state([runner.cache.get("r").slot])
        ctx = runner.build_context([StepEntry("r", [0] * (b - a), [])])
        cache = runner.storage.layer_caches(ctx.block_tables)[0]
        outs.append(mixer.forward(x[a:b].to(DEV).contiguous(), ctx, cache, runner.storage.state[0]).float().cpu().clone())
        runner.cache.commit("r", b)
    runner.release("r")
    return torch.cat(outs)


# ---------------------------------------------------------------------------
# each mechanism alone
# ---------------------------------------------------------------------------
def test_stretched_rotary_table():
    from vt_transformer_amd.parts import POSITIONS
    sc = {"factor": 8.0, "original": 256, "fast": 16.0, "slow": 2.0}
    rot = POSITIONS.build(PartSpec("rotary", {"theta": 3000.0, "dim": 24, "scaling": sc}), rt=runtime(torch.float32))
    cos, sin = rot.rotary_tables(500)
    f, mag = pl.yarn_frequencies(24, 3000.0, sc)
    ang = torch.arange(500, dtype=torch.float64)[:, None] * f[None, :]
    assert abs(mag - (0.1 * math.log(8.0) + 1)) < 1e-12
    assert float((cos.cpu().double() - torch.cos(ang) * mag).abs().max()) < 2e-7
    assert float((sin.cpu().double() - torch.sin(ang) * mag).abs().max()) < 2e-7
    # the fastest pair keeps its frequency, the slowest is divided by the factor, some pair lies between
    plain = torch.pow(torch.tensor(3000.0, dtype=torch.float64), -2.0 * torch.arange(12, dtype=torch.float64) / 24)
    ratio = f / plain
    assert ratio[0] == 1.0 and abs(float(ratio[-1]) - 1 / 8) < 1e-12 and ((ratio < 1) & (ratio > 1 / 8)).any()


def test_embedding_scale_and_stream_offsets():
    from vt_transformer_amd.kernels import ops
    from vt_transformer_amd.parts import EMBEDDINGS
    rt = runtime(torch.bfloat16)
    emb = EMBEDDINGS.build(PartSpec("embedding", {"name": "e", "scale": 2.75}), rt=rt, width=40, vocab_size=50)
    w = torch.randn(50, 40, generator=torch.Generator().manual_seed(1)).to(torch.bfloat16)
    emb.load({"e": w}.__getitem__, rt)
    ids = torch.tensor([3, 49, 0, 3], dtype=torch.int32, device=DEV)
    h = emb.forward(ids)
    ref = w.float()[ids.cpu().long()] * 2.75
    assert torch.equal(h.cpu(), ref)                 # the product is float32: bfloat16 * 2.75 rounded once
    row = torch.randn(40, generator=torch.Generator().manual_seed(2))
    delta = torch.randn(4, 40, generator=torch.Generator().manual_seed(3)).to(torch.bfloat16)
    ops.add_row(h, delta.to(DEV), row.to(DEV))
    assert float((h.cpu() - (ref + delta.float() + row)).abs().max()) < 1e-5
    ops.add_row(h, None, row.to(DEV))
    assert float((h.cpu() - (ref + delta.float() + 2 * row)).abs().max()) < 1e-5


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nh,kvh,d,dv,rot,chunk,window,cap,gate,unit", [
    (4, 2, 32, 48, 8, 24, 0, 15.0, True, True),      # everything on
    (3, 3, 16, 16, 16, 7, 0, 0.0, False, False),     # whole head rotated, nothing else but the chunks
    (6, 1, 40, 24, 0, 0, 0, 5.0, True, True),        # no rotation, every earlier key
    (2, 1, 24, 136, 12, 50, 20, 0.0, True, False),   # window inside chunks, values larger than keys
    (2, 1, 64, 96, 16, 50, 20, 10.0, True, True),    # the same on the matrix cores (heads in multiples of 16)
    (8, 2, 32, 48, 8, 24, 0, 15.0, True, True),      # four query heads to a key/value head: a block's waves share keys
    (4, 1, 16, 16, 16, 7, 11, 0.0, False, True),     # ... with a window inside small chunks
])
def test_masked_attention_part(dtype, nh, kvh, d, dv, rot, chunk, window, cap, gate, unit):
    from vt_transformer_amd.engine.step import ModelRunner
    from vt_transformer_amd.parts import MIXERS
    rt = runtime(dtype)
    width, t = 72, 83
    sc = {"factor": 4.0, "original": 32, "fast": 4.0, "slow": 1.0}
    pos_spec = PartSpec("rotary", {"theta": 1e4, "dim": rot, "scaling": sc}) if rot else None
    mixer = MIXERS.build(PartSpec("masked_attention", dict(
        num_heads=nh, num_kv_heads=kvh, key_dim=d, value_dim=dv, qkv_bias=True, position=pos_spec, scale=0.4, softcap=cap,
        window=window, chunk=chunk, unit_rms_eps=1e-5 if unit else None, head_gate=gate)), rt=rt, width=width, prefix="a.",
        shared={})
    w = weights_for(mixer, 3, 0.3)
    mixer.load(w.__getitem__, rt)
    runner = ModelRunner(OneMixer(mixer), rt, 16, 256, 4, 256)
    x = (torch.randn(t, width, generator=torch.Generator().manual_seed(4)) * 0.7).to(dtype)
    got = step_part(runner, mixer, x, [(0, 20), (20, 21), (21, 23), (23, 70), (70, 71), (71, 83)])
    xd, wd = x.double(), {k: v.double() for k, v in w.items()}
    pos = torch.arange(t)
    q = (xd @ wd["a.q_proj.weight"].t() + wd["a.q_proj.bias"]).reshape(t, nh, d)
    k = (xd @ wd["a.k_proj.weight"].t() + wd["a.k_proj.bias"]).reshape(t, kvh, d)
    v = (xd @ wd["a.v_proj.weight"].t() + wd["a.v_proj.bias"]).reshape(t, kvh, dv)
    if rot:
        q, k = pl.rotate_part(q, pos, rot, 1e4, sc), pl.rotate_part(k, pos, rot, 1e4, sc)
    if unit:
        q, k = pl.rms_unit(q, 1e-5), pl.rms_unit(k, 1e-5)
    o = chunk_window_attention(q, k, v, pos, 0.4, cap, chunk, window)
    if gate:
        o = o * torch.sigmoid(xd @ wd["a.g_proj.weight"].t())[:, :, None]
    ref = o.reshape(t, nh * dv) @ wd["a.o_proj.weight"].t()
    assert rel(got, ref) < PART_TOL[dtype]


def chunk_window_attention(q, k, v, pos, scale, cap, chunk, window):
    """pl.chunk_attention with a window on top (the design has none; the part takes one)."""
    if not window:
        return pl.chunk_attention(q, k, v, pos, scale, cap, chunk)
    t, h, _ = q.shape
    out = torch.zeros(t, h, v.shape[-1], dtype=torch.float64)
    for i in range(t):
        lo = max(0, i - window + 1, (i // chunk) * chunk if chunk else 0)
        out[i] = _one_row(q[i], k[lo:i + 1], v[lo:i + 1], scale, cap)
    return out


def _one_row(q, k, v, scale, cap):
    h, g = q.shape[0], k.shape[1]
    out = torch.zeros(h, v.shape[-1], dtype=torch.float64)
    for hh in range(h):
        s = (k[:, hh // (h // g)] @ q[hh]) * scale
        if cap > 0:
            s = cap * torch.tanh(s / cap)
        out[hh] = torch.softmax(s, dim=0) @ v[:, hh // (h // g)]
    return out


@pytest.mark.parametrize("dtype,matrix", [(torch.float32, False), (torch.bfloat16, False), (torch.bfloat16, True)])
def test_one_key_that_stands_out_at_chunk_and_page_edges(dtype, matrix):
    """Queries and keys are made so that one key far back (hundreds of keys away, the last slot of a page, the last
    position of a chunk) takes nearly all the weight from whoever sees it: the positions just inside its chunk must
    return its value, the first position of the next chunk must not, in a prompt's portion and decoded alone."""
    from vt_transformer_amd.engine.step import ModelRunner, StepEntry
    from vt_transformer_amd.kernels import ops
    from vt_transformer_amd.parts import MIXERS
    rt = runtime(dtype)
    nh, kvh, d, dv, chunk = (4 if matrix else 2), 1, 16, 16, 320      # (four heads to a key/value head: the kernel whose waves share keys)
    mixer = MIXERS.build(PartSpec("masked_attention", dict(num_heads=nh, num_kv_heads=kvh, key_dim=d, value_dim=dv,
                                                           scale=1.0, chunk=chunk)), rt=rt, width=8, prefix="a.", shared={})
    runner = ModelRunner(OneMixer(mixer), rt, 16, 1024, 2, 1024)
    t, star = 700, 31                      # the key that stands out: the last slot of the second page
    g = torch.Generator().manual_seed(5)
    y = torch.randn(t, (nh + kvh) * d + kvh * dv, generator=g) * 0.1
    y[:, :nh * d] = 0
    for hh in range(nh):
        y[:, hh * d] = 6.0                 # every query points along element 0 ...
    y[star, nh * d] = 6.0                  # ... and so does the one key: score 36 against about 0
    y[star, (nh + kvh) * d:] = 50.0
    far = chunk - 1                        # the last position that sees it
    for cuts in ([(0, t)], [(0, 300), (300, far), (far, far + 1), (far + 1, far + 2), (far + 2, t)]):
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
            if matrix and b - a > 1:        # (the mixer sends steps of single tokens to the other kernel)
                ops.attention_masked_mfma(q, cache["k"], cache["v"], ctx.positions, ctx.tok_entry, cache.block_table,
                                          ctx.extra[("masked_attention.tiles", 16)], out, nh, kvh, d, dv, 1.0, 0.0, 0, chunk)
            else:
                ops.attention_masked(q, cache["k"], cache["v"], ctx.positions, ctx.tok_entry, cache.block_table, out, nh, kvh,
                                     d, dv, 1.0, 0.0, 0, chunk)
            outs.append(out.float().cpu())
            runner.cache.commit("r", b)
        runner.release("r")
        got = torch.cat(outs)
        assert float(got[star:far + 1].min()) > 49.0, "a position inside the chunk lost the key that stands out"
        assert float(got[far + 1:].abs().max()) < 1.0, "a position of the next chunk saw a key of the chunk before"
        assert float(got[:star].abs().max()) < 1.0
        yd = y.to(dtype).double()
        ref = pl.chunk_attention(yd[:, :nh * d].reshape(t, nh, d), yd[:, nh * d:(nh + kvh) * d].reshape(t, kvh, d),
                                 yd[:, (nh + kvh) * d:].reshape(t, kvh, dv), torch.arange(t), 1.0, 0.0, chunk)
        assert rel(got, ref.reshape(t, nh * dv)) < PART_TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nh,kvh,d,dv,taps", [(4, 2, 16, 24, 3), (2, 2, 20, 72, 5), (3, 1, 64, 16, 2), (1, 1, 8, 130, 4),
                                              (2, 1, 12, 8, 1)])
def test_gated_delta_part(dtype, nh, kvh, d, dv, taps):
    """Prompt in one step, in portions (down to one and two tokens, shorter than the convolution), and token by token,
    all against the plain recurrence."""
    from vt_transformer_amd.engine.step import ModelRunner
    from vt_transformer_amd.parts import MIXERS
    rt = runtime(dtype)
    width, t = 56, 70
    mixer = MIXERS.build(PartSpec("gated_delta", dict(num_heads=nh, num_kv_heads=kvh, key_dim=d, value_dim=dv,
                                                      conv_taps=taps, norm_eps=1e-5)), rt=rt, width=width, prefix="m.", shared={})
    w = weights_for(mixer, 7, 0.25)
    w["m.A_log"] = torch.log(torch.linspace(0.02, 1.5, nh)).to(torch.bfloat16).float()
    mixer.load(w.__getitem__, rt)
    runner = ModelRunner(OneMixer(mixer), rt, 16, 256, 3, 256)
    assert runner.storage.state[0].shape == (3 + 1, (taps - 1) * (2 * kvh * d + nh * dv) + nh * d * dv)
    x = (torch.randn(t, width, generator=torch.Generator().manual_seed(8)) * 0.8).to(dtype)
    wd = {k[2:].replace("_proj.weight", "").replace("_conv.weight", ".conv").replace("norm.weight", "norm"): v.double()
          for k, v in w.items()}
    ref = pl.delta_mixer(x.double(), wd, "", dict(heads=nh, kv_heads=kvh, dim=d, vdim=dv), 1e-5)
    whole = step_part(runner, mixer, x, [(0, t)])
    assert rel(whole, ref) < PART_TOL[dtype]
    cut = step_part(runner, mixer, x, [(0, 1), (1, 3), (3, 4), (4, 6), (6, 37), (37, 38), (38, 40), (40, 57), (57, t)])
    steps = step_part(runner, mixer, x, [(i, i + 1) for i in range(t)])
    assert rel(cut, ref) < PART_TOL[dtype] and rel(steps, ref) < PART_TOL[dtype]
    if dtype == torch.float32:
        assert torch.equal(whole, cut) and torch.equal(whole, steps)      # the same operations whatever the cut


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
def test_long_decoding_across_chunks_and_pages(folders, dtype):
    folder, vocab = folders["A"], CONFIGS["A"]["vocab"]
    reqs = rh.random_requests(vocab, [150], seed=9)
    steps = rh.trace_alone(reqs, {"r0": [(0, 5)] + [(i, i + 1) for i in range(5, 150)]})
    runner = make_runner(folder, dtype, pool_tokens=192, max_requests=1)
    check_logits(folder, reqs, steps, rh.run_in_process(runner, steps), dtype)
    assert sum(runner.cache.available_pages()) == sum(p.num_pages for p in runner.cache.pools)


def test_pages_behind_a_chunk_are_given_back(folders):
    """A request longer than the pool of the attention layers' pages runs, because keys that no later position can
    see are dead; the plain logits still come out."""
    folder, vocab = folders["B"], CONFIGS["B"]["vocab"]       # chunks of 7 and 40 positions
    reqs = rh.random_requests(vocab, [140], seed=13)
    steps = rh.trace_alone(reqs, {"r0": rh.cut(reqs["r0"], [10])})
    runner = make_runner(folder, "float32", pool_tokens=96, max_requests=1, max_seq_len=160)
    check_logits(folder, reqs, steps, rh.run_in_process(runner, steps), "float32")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_generation_through_the_engine(folders, dtype):
    """Greedy tokens through Engine.generate (scheduler with short portions, two slots for three requests)."""
    from vt_transformer_amd.engine import Engine
    from vt_transformer_amd.sampling import SamplingParams
    folder = folders["C"]
    cfg, w = pl.read_folder(folder)
    prompts = [r for r in rh.random_requests(cfg["vocab"], [19, 3, 41], seed=21).values()]
    eng = Engine(folder, dtype=dtype, num_pages=16, max_running_reqs=2, max_seq_len=128, chunk_size=16, max_extend_tokens=24)
    got = eng.generate(prompts, SamplingParams(max_tokens=8, ignore_eos=True))
    for p, g in zip(prompts, got):
        assert len(g) == 8
        if dtype == "float32":
            assert g == pl.greedy(cfg, w, p, 8)
        else:
            logits = pl.forward(cfg, w, p + g)
            for i, tok in enumerate(g):
                row = logits[len(p) - 1 + i]
                assert float(row.max() - row[tok]) <= 3e-2 * float(row.abs().max())


def test_trace_run_with_a_lisunex_folder(folders, tmp_path):
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


def random_lisunex_config(seed: int) -> dict:
    """Sizes, orders and constants drawn at random, odd ones on purpose."""
    rs = np.random.RandomState(seed)
    pick = lambda xs: xs[rs.randint(len(xs))]
    width = int(pick([40, 72, 100, 136, 200]))
    layers = []
    for _ in range(rs.randint(2, 6)):
        heads = int(pick([1, 2, 3, 4, 6, 8]))
        kv = int(pick([k for k in (1, 2, 3, 4) if heads % k == 0]))
        ff = int(pick([0, 24, 100, 136]))
        if rs.rand() < 0.5:
            dim = int(pick([8, 16, 24, 40, 64]))
            layers.append(attention_layer(heads=heads, kv_heads=kv, dim=dim, vdim=int(pick([8, 16, 32, 40, 80, 144])),
                                          scale=float(pick([0.05, 0.3, 1.0])), softcap=float(pick([0.0, 2.0, 30.0])),
                                          chunk=int(pick([1, 3, 16, 50, 1000])), rot_dims=int(pick([d for d in (2, 4, 8, 16, 24, 40, 64) if d <= dim])),
                                          base=float(pick([100.0, 1e4, 1e6])), scaling=bool(rs.rand() < 0.6), ff=ff or None))
        else:
            layers.append(delta_layer(heads=heads, kv_heads=kv, dim=int(pick([8, 12, 32, 72, 128])),
                                      vdim=int(pick([8, 20, 64, 80])), conv=int(pick([2, 3, 4, 6])), ff=ff or None))
    n = len(layers)
    loop = None
    if rs.rand() < 0.6:
        a = int(rs.randint(0, n))
        loop = {"start": a, "stop": int(rs.randint(a + 1, n + 1)), "times": int(rs.randint(1, 4))}
    return {"architecture": "Lisunex", "vocab": int(pick([51, 97, 130, 255])), "width": width,
            "embedding": {"scale": float(pick([1.0, 0.5, 9.0]))}, "norm": {"eps": float(pick([1e-6, 1e-5, 1e-3]))},
            "layers": layers, "loop": loop}


@pytest.mark.parametrize("seed", range(8))
def test_configurations_drawn_at_random(tmp_path, seed):
    """Whatever config.json says is what runs: random sizes, layer orders, loops and constants, in float32 (sharp) and
    bfloat16, through portions and a mixed batch."""
    cfg = random_lisunex_config(seed)
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
