"""Plain, slow implementation of the Lisunex decoder: whole sequences, no
cache, one function per mechanism, in float64 on the CPU.  It shares no code
with the engine; the tests compare the engine against it.

Lisunex stacks two kinds of token mixers around a float32 residual stream:
attention over the keys of the token's own chunk of positions (rotary on part
of each head with YaRN-scaled frequencies, unit-RMS queries and keys, a
tanh cap on the scores, one sigmoid gate per head) and a gated delta rule (a
matrix state per head that decays, is corrected towards the new value and is
read in the same step; short causal convolutions in front).  A run of layers
may be repeated with shared weights and a per-pass offset vector.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

from plain_model import read_folder  # noqa: F401  (own safetensors reader of the tests)

DT = torch.float64


def rms_unit(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x * torch.rsqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def rmsnorm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    return rms_unit(x, eps) * w


def silu(x: torch.Tensor) -> torch.Tensor:
    return x * torch.sigmoid(x)


def softplus(x: torch.Tensor) -> torch.Tensor:
    return torch.where(x > 30, x, torch.log1p(torch.exp(torch.clamp(x, max=30))))


def yarn_frequencies(dims: int, base: float, scaling: Optional[dict]):
    """(frequency per pair [dims/2], factor on cos and sin).  Pair i has f_i = base^(-2i/dims); with scaling the
    slow pairs (few turns within `original` positions) are divided by `factor`, the fast ones kept, a linear ramp in
    the pair's index between the two."""
    half = dims // 2
    i = torch.arange(half, dtype=DT)
    f = torch.pow(torch.tensor(base, dtype=DT), -2.0 * i / dims)
    if not scaling:
        return f, 1.0
    factor, orig = float(scaling["factor"]), float(scaling["original"])

    def at(turns):
        return dims * math.log(orig / (2 * math.pi * turns)) / (2 * math.log(base))
    lo = max(math.floor(at(float(scaling["fast"]))), 0)
    hi = min(math.ceil(at(float(scaling["slow"]))), dims - 1)
    ramp = torch.clamp((i - lo) / max(hi - lo, 0.001), 0, 1)
    return f / factor * ramp + f * (1 - ramp), 0.1 * math.log(factor) + 1.0


def rotate_part(x: torch.Tensor, positions: torch.Tensor, dims: int, base: float, scaling: Optional[dict]) -> torch.Tensor:
    """x [T, heads, D]: the first `dims` of each head rotated, element i with element i + dims/2."""
    f, mag = yarn_frequencies(dims, base, scaling)
    ang = positions.to(DT)[:, None] * f[None, :]
    c, s = (torch.cos(ang) * mag)[:, None, :], (torch.sin(ang) * mag)[:, None, :]
    half = dims // 2
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], dim=-1)


def chunk_attention(q, k, v, positions, scale: float, softcap: float, chunk: int) -> torch.Tensor:
    """q [T, H, D], k [T, G, D], v [T, G, Dv] of one sequence at `positions`; key j is seen from i if j <= i and both lie
    in the same chunk of `chunk` positions (0: every earlier key).  -> [T, H, Dv]"""
    t, h, _ = q.shape
    g = k.shape[1]
    out = torch.zeros(t, h, v.shape[-1], dtype=DT)
    pi, pj = positions[:, None], positions[None, :]
    seen = pj <= pi
    if chunk > 0:
        seen = seen & ((pi // chunk) == (pj // chunk))
    for hh in range(h):
        kv = hh // (h // g)
        s = (q[:, hh] @ k[:, kv].t()) * scale
        if softcap > 0:
            s = softcap * torch.tanh(s / softcap)
        s = s.masked_fill(~seen, float("-inf"))
        out[:, hh] = torch.softmax(s, dim=-1) @ v[:, kv]
    return out


def attention_mixer(x, w: Dict[str, torch.Tensor], p: str, m: dict, eps: float, positions) -> torch.Tensor:
    t = x.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (x @ w[p + "q"].t() + w[p + "q.b"]).reshape(t, H, D)
    k = (x @ w[p + "k"].t() + w[p + "k.b"]).reshape(t, G, D)
    v = (x @ w[p + "v"].t() + w[p + "v.b"]).reshape(t, G, Dv)
    rot = m.get("rot")
    if rot:
        q = rotate_part(q, positions, rot["dims"], rot["base"], rot.get("scaling"))
        k = rotate_part(k, positions, rot["dims"], rot["base"], rot.get("scaling"))
    q, k = rms_unit(q, eps), rms_unit(k, eps)
    chunk = (m.get("mask") or {}).get("size", 0)
    o = chunk_attention(q, k, v, positions, m["scale"], m.get("softcap", 0.0), chunk)
    gate = torch.sigmoid(x @ w[p + "g"].t())            # [T, H]
    o = o * gate[:, :, None]
    return o.reshape(t, H * Dv) @ w[p + "o"].t()


def short_conv(x: torch.Tensor, taps: torch.Tensor) -> torch.Tensor:
    """x [T, C], taps [C, K]: y[t, c] = sum_j taps[c, j] x[t - (K-1) + j, c], zeros before the start."""
    t, c = x.shape
    kk = taps.shape[1]
    pad = torch.cat([torch.zeros(kk - 1, c, dtype=DT), x], dim=0)
    y = torch.zeros(t, c, dtype=DT)
    for j in range(kk):
        y += pad[j:j + t] * taps[:, j][None, :]
    return y


def delta_rule(q, k, v, beta, g) -> torch.Tensor:
    """Per head, token by token: S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q.
    q, k [T, H, D], v [T, H, Dv], beta, g [T, H] -> [T, H, Dv]"""
    t, h, d = q.shape
    dv = v.shape[-1]
    out = torch.zeros(t, h, dv, dtype=DT)
    for hh in range(h):
        S = torch.zeros(d, dv, dtype=DT)
        for i in range(t):
            S = S * g[i, hh]
            u = beta[i, hh] * (v[i, hh] - S.t() @ k[i, hh])
            S = S + torch.outer(k[i, hh], u)
            out[i, hh] = S.t() @ q[i, hh]
    return out


def delta_mixer(x, w: Dict[str, torch.Tensor], p: str, m: dict, eps: float) -> torch.Tensor:
    t = x.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(short_conv(x @ w[p + "q"].t(), w[p + "q.conv"])).reshape(t, G, D)
    k = silu(short_conv(x @ w[p + "k"].t(), w[p + "k.conv"])).reshape(t, G, D)
    v = silu(short_conv(x @ w[p + "v"].t(), w[p + "v.conv"])).reshape(t, H, Dv)
    q = q * torch.rsqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    k = k * torch.rsqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    rep = H // G
    q, k = q.repeat_interleave(rep, dim=1), k.repeat_interleave(rep, dim=1)
    beta = torch.sigmoid(x @ w[p + "b"].t())
    g = torch.exp(-torch.exp(w[p + "A_log"]) * softplus(x @ w[p + "a"].t() + w[p + "dt_bias"]))
    o = delta_rule(q, k, v, beta, g)
    o = rms_unit(o, eps) * w[p + "norm"]
    o = o * silu(x @ w[p + "g"].t()).reshape(t, H, Dv)
    return o.reshape(t, H * Dv) @ w[p + "o"].t()


def dense_mlp(x, w: Dict[str, torch.Tensor], p: str) -> torch.Tensor:
    return (silu(x @ w[p + "gate"].t()) * (x @ w[p + "up"].t())) @ w[p + "down"].t()


def layer_runs(cfg: dict) -> List[tuple]:
    """[(layer index, pass number or None if the layer starts no pass)] in the order they run."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, None) for i in range(n)]
    a, b, times = loop["start"], loop["stop"], loop["times"]
    runs = [(i, None) for i in range(a)]
    for t in range(times):
        runs += [(i, t if i == a else None) for i in range(a, b)]
    return runs + [(i, None) for i in range(b, n)]


def forward(cfg: dict, w: Dict[str, torch.Tensor], ids: List[int], streams: Optional[list] = None) -> torch.Tensor:
    """Logits [T, vocab] of one sequence from position 0.  streams: a list that gets the residual stream after every
    layer run."""
    eps = cfg["norm"]["eps"]
    pos = torch.arange(len(ids))
    x = w["embed"][torch.tensor(ids, dtype=torch.long)] * cfg["embedding"]["scale"]
    for i, t in layer_runs(cfg):
        if t is not None:
            x = x + w["loop.step"][t]
        L, p = cfg["layers"][i], f"l{i}."
        h = rmsnorm(x, w[p + "norm1"], eps)
        if L["type"] == "attention":
            x = x + attention_mixer(h, w, p + "mix.", L["mixer"], eps, pos)
        elif L["type"] == "delta":
            x = x + delta_mixer(h, w, p + "mix.", L["mixer"], eps)
        else:
            raise ValueError(L["type"])
        if L.get("mlp"):
            x = x + dense_mlp(rmsnorm(x, w[p + "norm2"], eps), w, p + "mlp.")
        if streams is not None:
            streams.append(x.clone())
    return rmsnorm(x, w["final.norm"], eps) @ w["head"].t()


def greedy(cfg: dict, w: Dict[str, torch.Tensor], prompt: List[int], n_new: int) -> List[int]:
    ids, out = list(prompt), []
    for _ in range(n_new):
        t = int(torch.argmax(forward(cfg, w, ids)[-1]))
        out.append(t)
        ids.append(t)
    return out
