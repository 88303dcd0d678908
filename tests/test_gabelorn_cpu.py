"""Gabelorn without a GPU: the configuration (keys, parts, tensors, errors) and the plain implementation's mechanisms on
cases with known answers."""
import copy
import math

import pytest
import torch

import plain_gabelorn as pg
from gabelorn_helpers import CFG_A, CFG_B, CFG_C, attention_layer, latent_layer, make_weights, write_model


def spec_of(cfg):
    from vt_transformer_amd.config import config_from_dict
    return config_from_dict(copy.deepcopy(cfg)).to_spec()


def test_configuration_becomes_parts():
    from vt_transformer_amd.config import GabelornConfig, architectures, config_from_dict
    assert "Gabelorn" in architectures()
    cfg = config_from_dict(copy.deepcopy(CFG_A))
    assert isinstance(cfg, GabelornConfig) and cfg.vocab_size == 203
    spec = cfg.to_spec()
    assert [e.layer for e in spec.schedule] == list(range(6)) and spec.stream_offsets is None
    kinds = [ls.mixer.kind for ls in spec.layers]
    assert kinds == ["masked_attention", "latent_attention", "masked_attention", "masked_attention", "latent_attention",
                     "masked_attention"]
    # the first layer that mixes values is their source, the later ones mix, a layer that says no does neither
    assert [ls.mixer.params.get("value_mix") for ls in spec.layers] == ["source", None, "off", "mix", None, "mix"]
    a = spec.layers[3].mixer.params
    assert (a["num_heads"], a["num_kv_heads"], a["key_dim"], a["value_dim"]) == (6, 2, 32, 48)
    assert a["q_temp"] == {"coef": 0.7, "every": 1} and a["distance_slopes"] == 8.0 and a["sink"] is True
    assert spec.layers[2].mixer.params["q_temp"] is None
    lat = spec.layers[1].mixer.params
    assert (lat["num_heads"], lat["plain_dim"], lat["rot_dim"], lat["value_dim"], lat["rank"]) == (8, 16, 16, 24, 32)
    assert lat["window"] == 20 and lat["position"].params["dim"] == 8 and lat["sink"] and lat["out_gate"]
    assert spec.layers[4].mixer.params["window"] == 0
    ff = spec.layers[0].feed_forward.params
    assert ff["act_limit"] == 0.8 and ff["act_alpha"] == 1.702 and ff["up_shift"] == 1.0 and ff["bias_suffix"] == ".b"
    assert spec.layers[2].feed_forward is None and "post_mixer" not in spec.layers[2].norms
    assert spec.head.params["softcap"] == 12.0 and spec_of(CFG_B).head.params["softcap"] == 0.0
    assert spec_of(CFG_C).layers[1].mixer.params["position"] is None       # nothing to rotate
    assert config_from_dict(cfg.to_dict()).to_spec() == spec


def test_declared_tensors():
    from vt_transformer_amd.config import config_from_dict
    from vt_transformer_amd.weights.random_init import declared_tensors
    t = declared_tensors(config_from_dict(copy.deepcopy(CFG_A)))
    assert t["embed"].shape == (203, 96) and t["head"].shape == (203, 96) and t["final.norm"].shape == (96,)
    assert t["l1.mix.q"].shape == (8 * 32, 96) and t["l1.mix.dkv"].shape == (48, 96) and t["l1.mix.dkv.norm"].shape == (32,)
    assert t["l1.mix.uk"].shape == (8 * 16, 32) and t["l1.mix.uv"].shape == (8 * 24, 32) and t["l1.mix.sink"].shape == (8,)
    assert t["l1.mix.g"].shape == (8 * 24, 96) and t["l1.mix.o"].shape == (96, 8 * 24)
    assert t["l0.mix.q"].shape == (128, 96) and t["l0.mix.k"].shape == (64, 96) and t["l0.mix.v"].shape == (96, 96)
    assert t["l0.mix.o"].shape == (96, 4 * 48) and t["l0.mix.sink"].shape == (4,)
    assert t["l3.mix.vmix"].shape == () and not t["l3.mix.vmix"].optional and t["l0.mix.vmix"].optional
    assert t["l2.mix.vmix"].optional and "l2.norm2" not in t and "l2.mlp.gate" not in t    # (tolerated, never read)
    assert t["l0.mlp.gate.b"].shape == (80,) and t["l0.mlp.down.b"].shape == (96,) and t["l0.mlp.up"].shape == (80, 96)
    assert not any(".b" == n[-2:] for n in t if ".mix." in n)        # no biases in the mixers


@pytest.mark.parametrize("change,message", [
    (lambda c: c["layers"][0].__setitem__("type", "conv"), "not known"),
    (lambda c: c["layers"][0]["mixer"].__setitem__("kv_heads", 3), "multiple"),
    (lambda c: c["layers"][1]["mixer"]["rot"].__setitem__("dims", 18), "rot_dim"),
    (lambda c: c["layers"][1]["mixer"]["rot"].__setitem__("dims", 7), "even"),
    (lambda c: c["layers"][1]["mixer"].pop("kv_rank"), "kv_rank"),
    (lambda c: c["layers"][0]["mlp"].pop("limit"), "limit"),
    (lambda c: c["layers"][0]["mlp"].__setitem__("kind", "routed"), "not known"),
    (lambda c: c["layers"][3]["mixer"].__setitem__("vdim", 40), "v_mix"),
    (lambda c: c["layers"][0]["mixer"]["q_temp"].__setitem__("every", 0), "positive"),
    (lambda c: c.pop("norm"), "norm"),
    (lambda c: c.__setitem__("logit_softcap", -1.0), "negative"),
])
def test_configuration_errors(change, message):
    from vt_transformer_amd.config import ConfigError, config_from_dict
    cfg = copy.deepcopy(CFG_A)
    change(cfg)
    with pytest.raises(ConfigError, match=message):
        config_from_dict(cfg)


def test_model_folder_round_trip(tmp_path):
    """A folder written with the tests' weights is read back by the plain reader and checked by the engine's loader;
    the command line's random model has every tensor the parts declare (a number without axes among them)."""
    from vt_transformer_amd.config import config_from_dict, load_config
    from vt_transformer_amd.weights.loader import check_tensors
    from vt_transformer_amd.weights.random_init import declared_tensors, write_random_model
    from vt_transformer_amd.weights.safetensors_io import WeightStore
    folder = write_model(copy.deepcopy(CFG_C), str(tmp_path / "c"), seed=1)
    cfg, w = pg.read_folder(folder)
    assert cfg["layers"][1]["mixer"]["kv_rank"] == 48 and w["l2.mix.vmix"].shape == ()
    store = WeightStore(folder)
    check_tensors(declared_tensors(load_config(folder)), {n: store.info(n) for n in store.names()}, folder)
    store.close()
    rnd = write_random_model(config_from_dict(copy.deepcopy(CFG_C)), str(tmp_path / "r"), seed=5)
    store = WeightStore(rnd)
    check_tensors(declared_tensors(load_config(rnd)), {n: store.info(n) for n in store.names()}, rnd)
    assert store.info("l3.mix.vmix")[1] == () and "l2.mix.vmix" not in store.names()
    store.close()


# ---------------------------------------------------------------------------
# the plain mechanisms on cases with known answers
# ---------------------------------------------------------------------------
def test_plain_rotation():
    x = torch.zeros(3, 1, 6, dtype=pg.DT)
    x[:, 0, 0] = 1.0
    x[:, 0, 5] = 7.0
    y = pg.rotate_half_split(x, torch.tensor([0, 1, 2]), 4, 100.0)
    for p in range(3):      # pair (0, 2) turns by p radians, pair (1, 3) by p / 10; elements 4 and 5 pass
        assert torch.allclose(y[p, 0], torch.tensor([math.cos(p), 0.0, math.sin(p), 0.0, 0.0, 7.0], dtype=pg.DT))
    z = torch.randn(5, 2, 8, dtype=pg.DT)
    assert torch.allclose(pg.rotate_half_split(z, torch.arange(5), 8, 50.0).norm(dim=-1), z.norm(dim=-1))


def test_plain_sink_softmax():
    s = torch.zeros(1, 2, 2, dtype=pg.DT)
    seen = torch.tensor([[True, False], [True, True]])
    # a sink of 0 counts like one more key with score 0 and no value
    a = pg.sink_softmax(s, seen, torch.zeros(1, dtype=pg.DT))
    assert torch.allclose(a[0], torch.tensor([[0.5, 0.0], [1 / 3, 1 / 3]], dtype=pg.DT))
    a = pg.sink_softmax(s, seen, torch.tensor([math.log(2.0)], dtype=pg.DT))
    assert torch.allclose(a[0, 1], torch.tensor([0.25, 0.25], dtype=pg.DT))
    assert torch.allclose(pg.sink_softmax(s, seen, None)[0, 1], torch.tensor([0.5, 0.5], dtype=pg.DT))
    a = pg.sink_softmax(s, seen, torch.tensor([800.0], dtype=pg.DT))      # a huge sink swallows everything, no overflow
    assert float(a.abs().max()) < 1e-300 or float(a.abs().max()) == 0.0


def test_plain_slopes_and_query_factor():
    assert torch.allclose(pg.head_slopes(4), torch.tensor([0.25, 0.0625, 0.015625, 0.00390625], dtype=pg.DT))
    assert torch.allclose(pg.head_slopes(1), torch.tensor([2.0 ** -8], dtype=pg.DT))
    f = pg.query_temperature(torch.tensor([0, 2, 3, 6, 7]), 0.5, 4)
    assert torch.allclose(f, torch.tensor([1.0, 1.0, 1 + 0.5 * math.log(2), 1 + 0.5 * math.log(2), 1 + 0.5 * math.log(3)], dtype=pg.DT))


def test_plain_slope_attention_prefers_near_keys_and_mixes_values():
    """One head, queries and keys of zero: the scores are the slopes times the distance alone; with a sink of minus
    infinity weights are exp(-slope d) normalised.  The second layer keeps (1 - lambda) v + lambda v_first."""
    t, width = 4, 2
    m = {"heads": 1, "kv_heads": 1, "dim": 2, "vdim": 2, "scale": 1.0, "v_mix": True}
    w = {"q": torch.zeros(2, width), "k": torch.zeros(2, width), "v": torch.eye(2), "o": torch.eye(2),
         "sink": torch.tensor([-1e9]), "vmix": torch.tensor(0.25)}
    w = {k: v.to(pg.DT) for k, v in w.items()}
    h = torch.tensor([[1.0, 0.0], [0.0, 1.0], [2.0, 0.0], [0.0, 3.0]], dtype=pg.DT)
    shared = {}
    out = pg.slope_attention_mixer(h, w, "", m, torch.arange(t), shared)
    s = 2.0 ** -8
    wts = torch.tensor([math.exp(-2 * s), math.exp(-s), 1.0], dtype=pg.DT)
    assert torch.allclose(out[2], (wts[:, None] * h[:3]).sum(0) / wts.sum())
    assert torch.equal(shared["v_first"][:, 0], h)
    h2 = h.flip(0)
    out2 = pg.slope_attention_mixer(h2, w, "", m, torch.arange(t), shared)
    assert torch.allclose(out2[0], 0.75 * h2[0] + 0.25 * h[0])


def test_plain_latent_attention_window_and_sink():
    """Keys of zero rank part and no rotated part: every seen key weighs the same, so a position's output is the mean
    of the values inside its window, shrunk by the sink's share; the gate of zero halves it."""
    t, width, rank = 6, 3, 2
    m = {"heads": 1, "dim": 2, "rot_dim": 0, "vdim": 2, "kv_rank": rank, "scale": 1.0, "mask": {"size": 3}}
    w = {"q": torch.zeros(2, width), "dkv": torch.tensor([[1.0, 0, 0], [0, 1.0, 0]]), "dkv.norm": torch.ones(rank),
         "uk": torch.zeros(2, rank), "uv": torch.eye(2), "sink": torch.tensor([0.0]), "g": torch.zeros(2, width),
         "o": torch.eye(2)}
    w = {k: v.to(pg.DT) for k, v in w.items()}
    h = torch.randn(t, width, dtype=pg.DT)
    out = pg.latent_attention_mixer(h, w, "", m, 0.0, torch.arange(t))
    c = h[:, :2] * torch.rsqrt((h[:, :2] ** 2).mean(-1, keepdim=True))
    assert torch.allclose(out[0], 0.5 * c[0] / 2)                       # itself and the sink
    assert torch.allclose(out[5], 0.5 * c[3:6].sum(0) / 4)              # three keys and the sink; key 2 is outside
    m2 = dict(m)
    m2.pop("mask")
    assert torch.allclose(pg.latent_attention_mixer(h, w, "", m2, 0.0, torch.arange(t))[5], 0.5 * c.sum(0) / 7)


def test_plain_feed_forward_bounds():
    w = {"gate": torch.eye(2), "gate.b": torch.zeros(2), "up": torch.eye(2), "up.b": torch.tensor([0.0, -9.0]),
         "down": torch.eye(2), "down.b": torch.tensor([0.5, 0.0])}
    w = {k: v.to(pg.DT) for k, v in w.items()}
    y = pg.clamped_gated_mlp(torch.tensor([[10.0, 1.0]], dtype=pg.DT), w, "", 2.0)
    g0 = 2.0 / (1 + math.exp(-1.702 * 2.0)) * (2.0 + 1.0)             # gate and up cut to 2
    g1 = 1.0 / (1 + math.exp(-1.702)) * (-2.0 + 1.0)                  # up cut to -2
    assert torch.allclose(y, torch.tensor([[g0 + 0.5, g1]], dtype=pg.DT))


def test_plain_forward_shapes_and_cap():
    cfg = copy.deepcopy(CFG_A)
    w = {k: v.double() for k, v in make_weights(cfg, 2).items()}
    streams = []
    logits = pg.forward(cfg, w, [3, 1, 4, 1, 5, 9, 2, 6], streams)
    assert logits.shape == (8, 203) and len(streams) == 6 and streams[0].shape == (8, 96)
    assert float(logits.abs().max()) < 12.0
    # causal: a longer sequence does not change earlier positions
    assert torch.allclose(pg.forward(cfg, w, [3, 1, 4, 1, 5])[:5], logits[:5], atol=1e-12)
    assert len(pg.greedy(cfg, w, [1, 2, 3], 3)) == 3


def test_command_line_writes_a_random_model(tmp_path):
    """`--write-random-model` with a Gabelorn config.json: the folder holds the configuration back and every tensor the
    parts need."""
    import json
    import os
    import subprocess
    import sys
    from vt_transformer_amd.weights.safetensors_io import WeightStore
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    cfg_path, out = tmp_path / "c.json", tmp_path / "m"
    cfg_path.write_text(json.dumps(CFG_B))
    r = subprocess.run([sys.executable, "-m", "vt_transformer_amd", "--write-random-model", str(out), "--config", str(cfg_path),
                        "--seed", "9"], capture_output=True, text=True, env=dict(os.environ, PYTHONPATH=root), timeout=300)
    assert r.returncode == 0, r.stderr
    cfg = json.loads((out / "config.json").read_text())
    assert cfg["architecture"] == "Gabelorn" and cfg["layers"] == CFG_B["layers"] and "logit_softcap" not in cfg
    store = WeightStore(str(out))
    names = set(store.names())
    assert {"embed", "head", "final.norm", "l0.mix.dkv.norm", "l0.mix.uk", "l1.mix.sink", "l2.mix.g", "l1.mlp.down.b"} <= names
    assert "l3.norm2" not in names and "l1.mix.vmix" not in names       # no feed-forward; the one mixing layer's number is not needed
    store.close()
