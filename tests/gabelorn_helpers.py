"""Small Gabelorn configurations, weights that make every mechanism matter, and the comparison of logits with the
plain implementation (plain_gabelorn.py)."""
from __future__ import annotations

import copy
import json
import os
from typing import Dict, List

import numpy as np
import torch

import plain_gabelorn as pg

# root mean square of a row's error (its mean taken off) over the root mean square of the row's logits (theirs too)
TOL = {"float32": 3e-5, "bfloat16": 3e-2}


def latent_layer(heads=4, dim=16, rot_dim=16, vdim=24, rank=32, scale=0.2, window=20, rot_dims=None, base=10000.0, ff=None,
                 limit=1.0):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": rank, "scale": scale}
    if window:
        m["mask"] = {"size": window}
    if rot_dim:
        m["rot"] = {"dims": rot_dims or rot_dim, "base": base}
    return {"type": "latent_attention", "mixer": m, "mlp": {"kind": "dense", "ff": ff, "limit": limit} if ff else None}


def attention_layer(heads=4, kv_heads=2, dim=32, vdim=48, scale=0.2, q_temp=(0.3, 5), v_mix=True, ff=None, limit=1.0):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "v_mix": v_mix}
    if q_temp:
        m["q_temp"] = {"coef": q_temp[0], "every": q_temp[1]}
    return {"type": "attention", "mixer": m, "mlp": {"kind": "dense", "ff": ff, "limit": limit} if ff else None}


# value mixing from the first layer on, with a layer that does not mix in between; eight latent heads (the kernel whose
# waves share keys), a window that is no multiple of a page, part of the rotated part rotated; a latent layer whose
# sizes are no multiples of 16 and that sees every key; a layer without a feed-forward
CFG_A = {"architecture": "Gabelorn", "vocab": 203, "width": 96, "norm": {"eps": 1e-5}, "logit_softcap": 12.0,
         "layers": [attention_layer(ff=80, limit=0.8),
                    latent_layer(heads=8, rot_dims=8, ff=64),
                    attention_layer(heads=2, kv_heads=1, dim=24, vdim=40, q_temp=None, v_mix=False),
                    attention_layer(heads=6, q_temp=(0.7, 1), ff=48, limit=2.5),
                    latent_layer(heads=3, dim=20, rot_dim=12, vdim=10, rank=24, window=0, ff=72),
                    attention_layer(heads=2, dim=16, scale=0.35)]}
# a latent layer first, one head, a window of one position; a single value-mixing layer (it only leaves its values);
# as many key/value heads as query heads; no cap on the logits; a window of 33 in heads of 64 + 32
CFG_B = {"architecture": "Gabelorn", "vocab": 131, "width": 80, "norm": {"eps": 1e-6},
         "layers": [latent_layer(heads=1, dim=8, rot_dim=16, vdim=8, rank=16, window=1, ff=112),
                    attention_layer(heads=3, kv_heads=3, dim=16, vdim=16, scale=0.3, q_temp=(0.5, 7), ff=64, limit=3.0),
                    latent_layer(heads=5, dim=48, rot_dim=32, vdim=80, rank=64, scale=0.05, window=33, base=500.0),
                    attention_layer(heads=4, kv_heads=1, dim=64, vdim=16, v_mix=False, q_temp=(0.1, 64))]}
# no rotated part at all in the latent layer, value mixing that starts in the middle
CFG_C = {"architecture": "Gabelorn", "vocab": 97, "width": 64, "norm": {"eps": 1e-5}, "logit_softcap": 30.0,
         "layers": [attention_layer(heads=2, kv_heads=2, dim=8, vdim=8, v_mix=False, ff=96),
                    latent_layer(heads=2, dim=24, rot_dim=0, vdim=40, rank=48, window=16, ff=48),
                    attention_layer(heads=4, kv_heads=4, dim=16, vdim=32, scale=0.25),
                    attention_layer(heads=8, kv_heads=4, dim=16, vdim=32, scale=0.25, ff=32)]}
CONFIGS = {"A": CFG_A, "B": CFG_B, "C": CFG_C}


def make_weights(cfg: dict, seed: int) -> Dict[str, torch.Tensor]:
    """Weights at scales at which every mechanism shows in the logits (projections that keep activations near 1,
    biases, sinks around the scores' size, mixing numbers between 0.1 and 0.9, gains away from 1), rounded to bfloat16."""
    from vt_transformer_amd.config import config_from_dict
    from vt_transformer_amd.weights.random_init import declared_tensors
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, decl in declared_tensors(config_from_dict(copy.deepcopy(cfg))).items():
        shape = tuple(decl.shape)
        leaf = name.split(".")[-1]
        if leaf == "sink":
            t = torch.randn(shape, generator=g) * 1.5 + 1.0
        elif leaf == "vmix":
            t = torch.rand(shape, generator=g) * 0.8 + 0.1
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
    cfg, w = pg.read_folder(model_dir)
    cache = cache if cache is not None else {}
    ref = {}
    for rid, toks in reqs.items():
        key = (model_dir, tuple(toks))
        if key not in cache:
            cache[key] = pg.forward(cfg, w, toks).numpy()
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
                # float32: every position within the tolerance.  bfloat16: one position in fifty (or one) may be up to
                # half again over
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
