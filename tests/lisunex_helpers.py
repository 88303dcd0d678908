"""Small Lisunex configurations, weights that make every mechanism matter, and the comparison of logits with the
plain implementation (plain_lisunex.py)."""
from __future__ import annotations

import copy
import json
import os
from typing import Dict, List

import numpy as np
import torch

import plain_lisunex as pl

# root mean square of a row's error (its mean taken off) over the root mean square of the row's logits (theirs too):
# bfloat16 rounds every activation to eight bits, about 4e-3 each, through up to seven layer runs of these weights; a
# portion of more than 64 tokens also gets its projections' results in 16 bits (the GEMM library's), the logits of the
# delta rule's decay among them, which these weights make steep
TOL = {"float32": 3e-5, "bfloat16": 3e-2}


def attention_layer(heads=4, kv_heads=2, dim=32, vdim=48, scale=0.2, softcap=15.0, chunk=24, rot_dims=8, base=10000.0,
                    scaling=True, ff=None):
    rot = {"dims": rot_dims, "base": base}
    if scaling:
        rot["scaling"] = {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 1.0}
    return {"type": "attention",
            "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "softcap": softcap,
                      "mask": {"size": chunk}, "rot": rot},
            "mlp": {"kind": "dense", "ff": ff} if ff else None}


def delta_layer(heads=4, kv_heads=2, dim=16, vdim=24, conv=3, ff=None):
    return {"type": "delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv},
            "mlp": {"kind": "dense", "ff": ff} if ff else None}


# delta first, a loop from layer 0 run three times, grouped heads in both mixers, a chunk that is no multiple of a page
CFG_A = {"architecture": "Lisunex", "vocab": 203, "width": 96, "embedding": {"scale": 3.5}, "norm": {"eps": 1e-5},
         "layers": [delta_layer(ff=80), attention_layer(), delta_layer(heads=2, kv_heads=1, dim=20, vdim=72, conv=5)],
         "loop": {"start": 0, "stop": 2, "times": 3}}
# no loop, as many key heads as query heads, one key head for all, whole head rotated without scaling, no cap, chunk 7,
# two taps, a feed-forward behind every kind of mixer, scale and embedding factor of 1
CFG_B = {"architecture": "Lisunex", "vocab": 131, "width": 80, "embedding": {"scale": 1.0}, "norm": {"eps": 1e-6},
         "layers": [attention_layer(heads=3, kv_heads=3, dim=16, vdim=16, scale=1.0, softcap=0.0, chunk=7, rot_dims=16,
                                    base=500.0, scaling=False, ff=112),
                    delta_layer(heads=3, kv_heads=3, dim=64, vdim=16, conv=2, ff=64),
                    attention_layer(heads=5, kv_heads=1, dim=48, vdim=80, scale=0.05, softcap=3.0, chunk=40, rot_dims=24),
                    delta_layer(heads=1, kv_heads=1, dim=8, vdim=8, conv=4)],
         "loop": None}
# a loop in the middle that runs once, then layers behind it
CFG_C = {"architecture": "Lisunex", "vocab": 97, "width": 64, "embedding": {"scale": 8.0}, "norm": {"eps": 1e-5},
         "layers": [attention_layer(heads=2, kv_heads=1, dim=24, vdim=40, chunk=16, rot_dims=4, ff=96),
                    delta_layer(heads=4, kv_heads=4, dim=12, vdim=20, conv=4),
                    attention_layer(heads=2, kv_heads=2, dim=64, vdim=8, chunk=33, rot_dims=64, ff=48)],
         "loop": {"start": 1, "stop": 2, "times": 1}}
CONFIGS = {"A": CFG_A, "B": CFG_B, "C": CFG_C}


def make_weights(cfg: dict, seed: int) -> Dict[str, torch.Tensor]:
    """Weights at scales at which every mechanism shows in the logits (projections that keep activations near 1,
    biases, decays spread between 0.5 and 0.999, gains away from 1), rounded to bfloat16."""
    from vt_transformer_amd.config import config_from_dict
    from vt_transformer_amd.weights.random_init import declared_tensors
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, decl in declared_tensors(config_from_dict(copy.deepcopy(cfg))).items():
        shape = tuple(decl.shape)
        leaf = name.split(".")[-1]
        if leaf == "A_log":
            t = torch.log(torch.rand(shape, generator=g) * 2.0 + 0.01)
        elif leaf == "dt_bias":
            t = torch.randn(shape, generator=g) * 1.5 - 1.0
        elif leaf == "conv":
            t = torch.randn(shape, generator=g) * 0.6
        elif leaf == "step":
            t = torch.randn(shape, generator=g) * 0.5
        elif decl.role == "gain":
            t = 1.0 + torch.randn(shape, generator=g) * 0.3
        elif decl.role == "bias":
            t = torch.randn(shape, generator=g) * 0.3
        elif name == "embed":
            t = torch.randn(shape, generator=g)
        else:
            t = torch.randn(shape, generator=g) / shape[-1] ** 0.5
        out[name] = t.to(torch.bfloat16)
    return out


def write_model(cfg: dict, folder: str, seed: int) -> str:
    from vt_transformer_amd.weights.safetensors_io import write_safetensors
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    write_safetensors(os.path.join(folder, "model.safetensors"), make_weights(cfg, seed).items(), metadata={"format": "pt"})
    return folder


def check_logits(model_dir: str, reqs: Dict[str, List[int]], steps: List[dict], got: Dict[int, np.ndarray], dtype: str,
                 cache: dict = None) -> float:
    """Every wanted row against the plain implementation's logits at that place; raises at the first row beyond
    tolerance, naming step, request and position.  Returns the worst error."""
    cfg, w = pl.read_folder(model_dir)
    cache = cache if cache is not None else {}
    ref = {}
    for rid, toks in reqs.items():
        key = (model_dir, tuple(toks))
        if key not in cache:
            cache[key] = pl.forward(cfg, w, toks).numpy()
        ref[rid] = cache[key]
    pos = {r: 0 for r in reqs}
    worst, over, count = 0.0, 0, 0
    for s in steps:
        row = 0
        for e in s["entries"]:
            for wi in e["want"]:
                p = pos[e["id"]] + wi
                r = ref[e["id"]][p]
                gl = got[s["step"]][row].astype(np.float64)
                assert np.isfinite(gl).all(), f"step {s['step']} request {e['id']} position {p}: logits are not finite"
                diff = gl - r
                err = float(np.sqrt(np.mean((diff - diff.mean()) ** 2)) / max(np.sqrt(np.mean((r - r.mean()) ** 2)), 1e-30))
                # float32: every position within the tolerance.  bfloat16: a position whose logits lie close together
                # magnifies the rounding it has inherited, so one position in fifty (or one) may be up to half again over
                hard = TOL[dtype] * (1.5 if dtype == "bfloat16" else 1.0)
                assert err < hard, (f"step {s['step']} request {e['id']} position {p} "
                                    f"(portion starts at {pos[e['id']]}): error {err:.3e} > {hard:.1e}")
                over += err >= TOL[dtype]
                count += 1
                worst = max(worst, err)
                row += 1
            pos[e["id"]] += len(e["tokens"])
    assert over <= max(1, count // 50), f"{over} of {count} positions are over {TOL[dtype]:.0e} (worst {worst:.3e})"
    return worst
