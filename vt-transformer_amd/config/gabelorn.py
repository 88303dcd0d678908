"""Gabelorn: typed configuration read from the keys of its config.json.

A Gabelorn model is a list of pre-norm layers around a float32 residual stream.
Each layer names its mixer and may have a feed-forward.  Two mixers:

"latent_attention": the cache holds one low-rank vector and one rotated key part per token; per head the unrotated
keys and the values are projections of the low-rank vector; a query head is [dim unrotated | rot_dim rotated]; a
sliding window, a learned sink per head in the softmax's denominator, an elementwise sigmoid gate on the heads'
outputs (`parts/latent_attention.py`).

"attention": grouped key/value heads with separate key and value sizes and no rotation; queries times a factor that
grows with the logarithm of the position, scores less a per-head slope times the distance, every earlier key seen, a
sink per head, values mixed with those of the first layer that mixes values (`parts/masked_attention.py`).

The feed-forward is a gated unit with biases whose gate and up projections are bounded; the logits are bounded by a
tanh.

config.json:
  architecture            "Gabelorn"
  vocab, width            sizes of the vocabulary and of the stream
  norm.eps                eps of every RMS norm of the model (also of the low-rank vector's)
  logit_softcap           c: logits <- c tanh(logits / c) (absent or 0: not)
  layers[i].type          "latent_attention" | "attention"
  layers[i].mixer         latent_attention: heads, dim, rot_dim, vdim, kv_rank, scale, mask.size, rot.{dims, base}
                          attention:        heads, kv_heads, dim, vdim, scale, q_temp.{coef, every}, v_mix
  layers[i].mlp           null | {kind: "dense", ff, limit}

Tensor names: embed, head, final.norm, and per layer l<i>.norm1, l<i>.norm2, l<i>.mix.*, l<i>.mlp.*; a bias is the
matrix's name with ".b".

Fixed by the architecture: no biases in the mixers and biases on all three projections of the feed-forward; rotation
in half-split pairs; the slopes 2^(-8 (h + 1) / H); sinks in both mixers; the latent mixer's output gate; the
feed-forward's gate g sigmoid(1.702 g) (u + 1).
"""
from __future__ import annotations

import copy
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

from .base import (ConfigError, LayerSpec, ModelConfig, ModelSpec, PartSpec, ScheduleEntry, read_key, require_positive)

_LATENT_NAMES = {"q": "q", "dkv": "dkv", "dkv_norm": "dkv.norm", "uk": "uk", "uv": "uv", "o": "o", "g": "g", "sink": "sink"}
_ATTENTION_NAMES = {"q": "q", "k": "k", "v": "v", "o": "o", "sink": "sink", "vmix": "vmix"}
_MLP_NAMES = {"gate": "gate", "up": "up", "down": "down"}

SLOPE_STEEPNESS = 8.0       # head h's slope is 2^(-8 (h + 1) / H)
GATE_ALPHA = 1.702          # the feed-forward's gate: g sigmoid(1.702 g) (u + 1)
UP_SHIFT = 1.0


def _sub(d: Dict[str, Any], key: str, where: str, optional: bool = False) -> Optional[Dict[str, Any]]:
    v = d.get(key)
    if v is None:
        if optional:
            return None
        raise ConfigError(f"{where}: required key '{key}' is missing")
    if not isinstance(v, dict):
        raise ConfigError(f"{where}: key '{key}' must be an object, got {v!r}")
    return v


@dataclass
class GabelornConfig(ModelConfig):
    vocab: int
    width: int
    norm_eps: float
    layers: List[Dict[str, Any]]
    logit_softcap: float = 0.0
    max_positions: int = 1 << 20          # the design sets no limit; the engine's max_seq_len bounds what is run
    eos_token_id: List[int] = field(default_factory=list)

    architecture = "Gabelorn"

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "GabelornConfig":
        layers = d.get("layers")
        if not isinstance(layers, list) or not layers or not all(isinstance(x, dict) for x in layers):
            raise ConfigError("config.json: key 'layers' must be a non-empty list of objects")
        eos = d.get("eos_token_id")
        eos_list = [] if eos is None else ([eos] if isinstance(eos, int) else list(eos))
        cfg = cls(
            vocab=read_key(d, "vocab", int),
            width=read_key(d, "width", int),
            norm_eps=read_key(_sub(d, "norm", "config.json"), "eps", float, where="config.json: norm"),
            layers=copy.deepcopy(layers),
            logit_softcap=read_key(d, "logit_softcap", float, 0.0),
            max_positions=read_key(d, "max_positions", int, 1 << 20),
            eos_token_id=eos_list,
        )
        cfg.check()
        return cfg

    # ------------------------------------------------------------------
    def check(self) -> None:
        require_positive("vocab", self.vocab)
        require_positive("width", self.width)
        require_positive("norm.eps", self.norm_eps)
        if self.logit_softcap < 0:
            raise ConfigError("config.json: logit_softcap must not be negative")
        mixed_shape = None
        for i, L in enumerate(self.layers):
            where = f"config.json: layers[{i}]"
            kind = read_key(L, "type", str, where=where)
            m = _sub(L, "mixer", where)
            mw = where + ".mixer"
            for key in ("heads", "dim", "vdim"):
                require_positive(f"layers[{i}].mixer.{key}", read_key(m, key, int, where=mw))
            require_positive(f"layers[{i}].mixer.scale", read_key(m, "scale", float, where=mw))
            if kind == "latent_attention":
                require_positive(f"layers[{i}].mixer.kv_rank", read_key(m, "kv_rank", int, where=mw))
                rot_dim = read_key(m, "rot_dim", int, where=mw)
                if rot_dim < 0:
                    raise ConfigError(f"{mw}: rot_dim must not be negative")
                mask = _sub(m, "mask", mw, optional=True)
                if mask is not None:
                    require_positive(f"layers[{i}].mixer.mask.size", read_key(mask, "size", int, where=mw + ".mask"))
                rot = _sub(m, "rot", mw, optional=True)
                if rot is not None:
                    dims = read_key(rot, "dims", int, where=mw + ".rot")
                    if dims <= 0 or dims % 2 or dims > rot_dim:
                        raise ConfigError(f"{mw}.rot: dims {dims} must be even, positive and at most rot_dim {rot_dim}")
                    require_positive(f"layers[{i}].mixer.rot.base", read_key(rot, "base", float, where=mw + ".rot"))
            elif kind == "attention":
                heads, kv = m["heads"], read_key(m, "kv_heads", int, where=mw)
                if kv <= 0 or heads % kv:
                    raise ConfigError(f"{mw}: heads {heads} must be a positive multiple of kv_heads {kv}")
                qt = _sub(m, "q_temp", mw, optional=True)
                if qt is not None:
                    read_key(qt, "coef", float, where=mw + ".q_temp")
                    require_positive(f"layers[{i}].mixer.q_temp.every", read_key(qt, "every", int, where=mw + ".q_temp"))
                if read_key(m, "v_mix", bool, False, where=mw):
                    shape = (kv, m["vdim"])
                    if mixed_shape is not None and shape != mixed_shape:
                        raise ConfigError(f"{mw}: v_mix with {kv} key/value heads of {m['vdim']}, the first layer that "
                                          f"mixes values has {mixed_shape[0]} of {mixed_shape[1]}")
                    mixed_shape = shape
            else:
                raise ConfigError(f"{where}: mixer type '{kind}' is not known ('latent_attention' and 'attention' are)")
            mlp = _sub(L, "mlp", where, optional=True)
            if mlp is not None:
                if read_key(mlp, "kind", str, "dense", where=where + ".mlp") != "dense":
                    raise ConfigError(f"{where}.mlp: kind '{mlp['kind']}' is not known ('dense' is)")
                require_positive(f"layers[{i}].mlp.ff", read_key(mlp, "ff", int, where=where + ".mlp"))
                require_positive(f"layers[{i}].mlp.limit", read_key(mlp, "limit", float, where=where + ".mlp"))

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {
            "architecture": self.architecture, "vocab": self.vocab, "width": self.width,
            "norm": {"eps": self.norm_eps}, "layers": copy.deepcopy(self.layers),
        }
        if self.logit_softcap:
            d["logit_softcap"] = self.logit_softcap
        if self.max_positions != 1 << 20:
            d["max_positions"] = self.max_positions
        if self.eos_token_id:
            d["eos_token_id"] = list(self.eos_token_id)
        return d

    # ------------------------------------------------------------------
    def _mixer_spec(self, L: Dict[str, Any], value_mix: Optional[str]) -> PartSpec:
        m = L["mixer"]
        if L["type"] == "latent_attention":
            rot, mask = m.get("rot"), m.get("mask")
            position = None
            if rot is not None and int(m["rot_dim"]) > 0:
                position = PartSpec("rotary", {"theta": float(rot["base"]), "dim": int(rot["dims"]), "scaling": None})
            return PartSpec("latent_attention", {
                "num_heads": int(m["heads"]), "plain_dim": int(m["dim"]), "rot_dim": int(m["rot_dim"]),
                "value_dim": int(m["vdim"]), "rank": int(m["kv_rank"]), "norm_eps": self.norm_eps, "position": position,
                "scale": float(m["scale"]), "window": int(mask["size"]) if mask else 0, "sink": True, "out_gate": True,
                "names": dict(_LATENT_NAMES), "prefix": "mix.",
            })
        qt = m.get("q_temp")
        return PartSpec("masked_attention", {
            "num_heads": int(m["heads"]), "num_kv_heads": int(m["kv_heads"]), "key_dim": int(m["dim"]),
            "value_dim": int(m["vdim"]), "scale": float(m["scale"]), "sink": True, "distance_slopes": SLOPE_STEEPNESS,
            "q_temp": {"coef": float(qt["coef"]), "every": int(qt["every"])} if qt else None, "value_mix": value_mix,
            "fuse_norms": True, "names": dict(_ATTENTION_NAMES), "prefix": "mix.",
        })

    def to_spec(self) -> ModelSpec:
        layers = []
        seen_mixing = False
        for i, L in enumerate(self.layers):
            value_mix = "off" if L["type"] == "attention" else None
            if L["type"] == "attention" and L["mixer"].get("v_mix"):
                value_mix = "mix" if seen_mixing else "source"
                seen_mixing = True
            mlp = L.get("mlp")
            norms = {"input": PartSpec("rmsnorm", {"eps": self.norm_eps, "name": "norm1"})}
            ffn = None
            if mlp is not None:
                norms["post_mixer"] = PartSpec("rmsnorm", {"eps": self.norm_eps, "name": "norm2"})
                ffn = PartSpec("gated_mlp", {"intermediate_size": int(mlp["ff"]), "activation": "silu",
                                             "act_alpha": GATE_ALPHA, "act_limit": float(mlp["limit"]), "up_shift": UP_SHIFT,
                                             "names": dict(_MLP_NAMES), "weight_suffix": "", "bias_suffix": ".b",
                                             "prefix": "mlp."})
            layers.append(LayerSpec(block=PartSpec("prenorm", {}), mixer=self._mixer_spec(L, value_mix), feed_forward=ffn,
                                    norms=norms, prefix=f"l{i}."))
        spec = ModelSpec(
            architecture=self.architecture,
            vocab_size=self.vocab,
            hidden_size=self.width,
            embedding=PartSpec("embedding", {"name": "embed"}),
            layers=layers,
            schedule=[ScheduleEntry(i) for i in range(len(layers))],
            final_norm=PartSpec("rmsnorm", {"eps": self.norm_eps, "name": "final.norm"}),
            head=PartSpec("linear_head", {"name": "head", "tied_to": None, "softcap": self.logit_softcap}),
            max_positions=self.max_positions,
            eos_token_ids=list(self.eos_token_id),
        )
        spec.validate()
        return spec
