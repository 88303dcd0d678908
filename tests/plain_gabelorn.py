"""Plain, slow implementation of the Gabelorn decoder: whole sequences, no
cache, one function per mechanism, in float64 on the CPU.  It shares no code
with the engine; the tests compare the engine against it.

Gabelorn stacks two kinds of attention around a float32 residual stream.
"latent_attention" keeps one low-rank vector and one rotated key part per
token: every head's unrotated keys and its values are projections of the
low-rank vector, the rotated key part is shared by the heads, positions see a
sliding window, the softmax has a learned sink per head, and the heads'
outputs pass an elementwise sigmoid gate.  "attention" has grouped key/value
heads without any rotation: the queries grow with the logarithm of the
position, the scores lose a per-head slope times the distance, the softmax
has a sink, and the values are mixed with those of the first such layer.  The
feed-forward is a clamped gated unit with biases; the logits are capped by a
tanh.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

from plain_model import read_folder  # noqa: F401  (own safetensors reader of the tests)

DT = torch.float64


def rmsnorm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) * w over the last axis."""
    return x * torch.rsqrt((x * x).mean(dim=-1, keepdim=True) + eps) * w


def rotate_half_split(x: torch.Tensor, positions: torch.Tensor, dims: int, base: float) -> torch.Tensor:
    """x [T, ..., D]: the first `dims` elements of the last axis rotated, element i with element i + dims/2, by the
    angle position * base^(-2i/dims); the rest passes."""
    half = dims // 2
    f = torch.pow(torch.tensor(base, dtype=DT), -2.0 * torch.arange(half, dtype=DT) / dims)
    ang = positions.to(DT)[:, None] * f[None, :]
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [half]
    c, s = torch.cos(ang).reshape(shape), torch.sin(ang).reshape(shape)
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], dim=-1)


def sink_softmax(scores: torch.Tensor, seen: torch.Tensor, sink: Optional[torch.Tensor]) -> torch.Tensor:
    """scores [H, T, T], seen [T, T] (bool), sink [H] or None -> weights [H, T, T].  The sink adds exp(sink_h) to
    every row's denominator and nothing to the numerators."""
    s = scores.masked_fill(~seen[None], -math.inf)
    if sink is None:
        return torch.softmax(s, dim=-1)
    m = torch.maximum(s.max(dim=-1, keepdim=True).values, sink[:, None, None])
    e = torch.exp(s - m)
    return e / (e.sum(dim=-1, keepdim=True) + torch.exp(sink[:, None, None] - m))


def latent_attention_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: dict, eps: float,
                           positions: torch.Tensor) -> torch.Tensor:
    """h [T, width] -> [T, width].  Keys and values of every head are made anew from the low-rank vectors here (the
    engine never forms them)."""
    t = h.shape[0]
    heads, dim, rot_dim, vdim, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    rot = m.get("rot") or {}
    q = (h @ w[p + "q"].T).reshape(t, heads, dim + rot_dim)
    q_plain, q_rot = q[..., :dim], q[..., dim:]
    dkv = h @ w[p + "dkv"].T
    c = rmsnorm(dkv[:, :rank], w[p + "dkv.norm"], eps)
    k_rot = dkv[:, rank:]
    if rot:
        q_rot = rotate_half_split(q_rot, positions, int(rot["dims"]), float(rot["base"]))
        k_rot = rotate_half_split(k_rot, positions, int(rot["dims"]), float(rot["base"]))
    k_plain = (c @ w[p + "uk"].T).reshape(t, heads, dim)
    v = (c @ w[p + "uv"].T).reshape(t, heads, vdim)
    scores = (torch.einsum("ihd,jhd->hij", q_plain, k_plain) + torch.einsum("ihd,jd->hij", q_rot, k_rot)) * m["scale"]
    dist = positions[:, None] - positions[None, :]
    seen = dist >= 0
    if m.get("mask"):
        seen = seen & (dist < int(m["mask"]["size"]))
    a = sink_softmax(scores, seen, w.get(p + "sink"))
    o = torch.einsum("hij,jhd->ihd", a, v).reshape(t, heads * vdim)
    o = o * torch.sigmoid(h @ w[p + "g"].T)
    return o @ w[p + "o"].T


def query_temperature(positions: torch.Tensor, coef: float, every: int) -> torch.Tensor:
    """1 + coef ln(floor((p + 1) / every) + 1) per position."""
    return 1.0 + coef * torch.log(torch.div(positions + 1, every, rounding_mode="floor").to(DT) + 1.0)


def head_slopes(heads: int) -> torch.Tensor:
    """2^(-8 (h + 1) / heads) for h = 0 .. heads - 1."""
    return torch.pow(torch.tensor(2.0, dtype=DT), -8.0 * (torch.arange(heads, dtype=DT) + 1.0) / heads)


def mix_values(v: torch.Tensor, v_first: torch.Tensor, lam: torch.Tensor) -> torch.Tensor:
    return (1.0 - lam) * v + lam * v_first


def slope_attention_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, m: dict, positions: torch.Tensor,
                          shared: dict) -> torch.Tensor:
    """h [T, width] -> [T, width].  shared: carries the values of the first value-mixing layer to the later ones."""
    t = h.shape[0]
    heads, kv, dim, vdim = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w[p + "q"].T).reshape(t, heads, dim)
    k = (h @ w[p + "k"].T).reshape(t, kv, dim)
    v = (h @ w[p + "v"].T).reshape(t, kv, vdim)
    qt = m.get("q_temp")
    if qt:
        q = q * query_temperature(positions, float(qt["coef"]), int(qt["every"]))[:, None, None]
    if m.get("v_mix"):
        if "v_first" in shared:
            v = mix_values(v, shared["v_first"], w[p + "vmix"])
        else:
            shared["v_first"] = v
    group = heads // kv
    kh, vh = k.repeat_interleave(group, dim=1), v.repeat_interleave(group, dim=1)
    dist = (positions[:, None] - positions[None, :])
    scores = torch.einsum("ihd,jhd->hij", q, kh) * m["scale"] - head_slopes(heads)[:, None, None] * dist.to(DT)[None]
    a = sink_softmax(scores, dist >= 0, w.get(p + "sink"))
    o = torch.einsum("hij,jhd->ihd", a, vh).reshape(t, heads * vdim)
    return o @ w[p + "o"].T


def clamped_gated_mlp(x: torch.Tensor, w: Dict[str, torch.Tensor], p: str, limit: float) -> torch.Tensor:
    """g = min(gate(x), limit), u = clamp(up(x), -limit, limit), down(g sigmoid(1.702 g) (u + 1)); biases on all three."""
    g = torch.clamp(x @ w[p + "gate"].T + w[p + "gate.b"], max=limit)
    u = torch.clamp(x @ w[p + "up"].T + w[p + "up.b"], min=-limit, max=limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ w[p + "down"].T + w[p + "down.b"]


def forward(cfg: dict, w: Dict[str, torch.Tensor], ids: List[int], streams: Optional[list] = None) -> torch.Tensor:
    """Logits [T, vocab] of one sequence from position 0.  streams: a list that receives the residual stream after
    every layer."""
    w = {k: v.to(DT) for k, v in w.items()}
    eps = float(cfg["norm"]["eps"])
    positions = torch.arange(len(ids))
    x = w["embed"][torch.tensor(ids, dtype=torch.long)]
    shared: dict = {}
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        hn = rmsnorm(x, w[p + "norm1"], eps)
        if layer["type"] == "latent_attention":
            x = x + latent_attention_mixer(hn, w, p + "mix.", layer["mixer"], eps, positions)
        elif layer["type"] == "attention":
            x = x + slope_attention_mixer(hn, w, p + "mix.", layer["mixer"], positions, shared)
        else:
            raise ValueError(f"layer type {layer['type']!r}")
        mlp = layer.get("mlp")
        if mlp is not None:
            x = x + clamped_gated_mlp(rmsnorm(x, w[p + "norm2"], eps), w, p + "mlp.", float(mlp["limit"]))
        if streams is not None:
            streams.append(x.clone())
    logits = rmsnorm(x, w["final.norm"], eps) @ w["head"].T
    cap = cfg.get("logit_softcap")
    if cap:
        logits = float(cap) * torch.tanh(logits / float(cap))
    return logits


def greedy(cfg: dict, w: Dict[str, torch.Tensor], prompt: List[int], n_new: int) -> List[int]:
    ids = list(prompt)
    for _ in range(n_new):
        ids.append(int(torch.argmax(forward(cfg, w, ids)[-1])))
    return ids[len(prompt):]
