"""Lisunex: typed configuration read from the keys of its config.json.

A Lisunex model is a list of pre-norm layers around a float32 residual stream.
Each layer names its mixer ("attention": chunk-masked attention with partial
rotary encoding, unit-RMS queries and keys, capped scores and head gates;
"delta": the gated delta rule with short convolutions) and may or may not have
a gated feed-forward.  A run of layers can be repeated with shared weights;
every pass has caches and state of its own and starts by adding its own row of
the tensor `loop.step` to the stream.  The embedding is multiplied by a constant.

config.json:
  architecture            "Lisunex"
  vocab, width            sizes of the vocabulary and of the stream
  embedding.scale         factor on the embedding rows
  norm.eps                eps of every RMS norm of the model (also of the mixers' own)
  layers[i].type          "attention" | "delta"
  layers[i].mixer         attention: heads, kv_heads, dim, vdim, scale, softcap, mask.size,
                                     rot.{dims, base, scaling.{factor, original, fast, slow}}
                          delta:     heads, kv_heads, dim, vdim, conv
  layers[i].mlp           null | {kind: "dense", ff}
  loop                    null | {start, stop, times}

Tensor names: embed, head, final.norm, loop.step, and per layer l<i>.norm1, l<i>.norm2, l<i>.mix.*, l<i>.mlp.*;
a bias is the matrix's name with ".b", a convolution's taps the matrix's name with ".conv".

Fixed by the architecture: biases on q, k and v of attention and nowhere else; rotation in half-split pairs; SiLU
gates; 1e-6 inside the root of the delta rule's unit vectors (in the kernel).
"""
from __future__ import annotations

import copy
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

from .base import (ConfigError, LayerSpec, ModelConfig, ModelSpec, PartSpec, ScheduleEntry, read_key, require_positive)

_ATTENTION_NAMES = {"q": "q", "k": "k", "v": "v", "o": "o", "g": "g", "q_bias": "q.b", "k_bias": "k.b", "v_bias": "v.b"}
_DELTA_NAMES = {"q": "q", "k": "k", "v": "v", "g": "g", "o": "o", "q_conv": "q.conv", "k_conv": "k.conv", "v_conv": "v.conv",
                "b": "b", "a": "a", "A_log": "A_log", "dt_bias": "dt_bias", "norm": "norm"}
_MLP_NAMES = {"gate": "gate", "up": "up", "down": "down"}


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
class LisunexConfig(ModelConfig):
    vocab: int
    width: int
    embedding_scale: float
    norm_eps: float
    layers: List[Dict[str, Any]]
    loop: Optional[Dict[str, int]] = None
    max_positions: int = 1 << 20          # the design sets no limit; the engine's max_seq_len bounds what is run
    eos_token_id: List[int] = field(default_factory=list)

    architecture = "Lisunex"

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "LisunexConfig":
        layers = d.get("layers")
        if not isinstance(layers, list) or not layers or not all(isinstance(x, dict) for x in layers):
            raise ConfigError("config.json: key 'layers' must be a non-empty list of objects")
        eos = d.get("eos_token_id")
        eos_list = [] if eos is None else ([eos] if isinstance(eos, int) else list(eos))
        cfg = cls(
            vocab=read_key(d, "vocab", int),
            width=read_key(d, "width", int),
            embedding_scale=read_key(_sub(d, "embedding", "config.json", optional=True) or {}, "scale", float, 1.0,
                                     where="config.json: embedding"),
            norm_eps=read_key(_sub(d, "norm", "config.json"), "eps", float, where="config.json: norm"),
            layers=copy.deepcopy(layers),
            loop=copy.deepcopy(_sub(d, "loop", "config.json", optional=True)),
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
        for i, L in enumerate(self.layers):
            where = f"config.json: layers[{i}]"
            kind = read_key(L, "type", str, where=where)
            m = _sub(L, "mixer", where)
            mw = where + ".mixer"
            heads, kv = read_key(m, "heads", int, where=mw), read_key(m, "kv_heads", int, where=mw)
            for key in ("dim", "vdim"):
                require_positive(f"layers[{i}].mixer.{key}", read_key(m, key, int, where=mw))
            if heads <= 0 or kv <= 0 or heads % kv:
                raise ConfigError(f"{mw}: heads {heads} must be a positive multiple of kv_heads {kv}")
            if kind == "attention":
                require_positive(f"layers[{i}].mixer.scale", read_key(m, "scale", float, where=mw))
                if read_key(m, "softcap", float, 0.0, where=mw) < 0:
                    raise ConfigError(f"{mw}: softcap must not be negative")
                mask = _sub(m, "mask", mw, optional=True)
                if mask is not None:
                    require_positive(f"layers[{i}].mixer.mask.size", read_key(mask, "size", int, where=mw + ".mask"))
                rot = _sub(m, "rot", mw, optional=True)
                if rot is not None:
                    dims = read_key(rot, "dims", int, where=mw + ".rot")
                    if dims <= 0 or dims % 2 or dims > m["dim"]:
                        raise ConfigError(f"{mw}.rot: dims {dims} must be even, positive and at most dim {m['dim']}")
                    require_positive(f"layers[{i}].mixer.rot.base", read_key(rot, "base", float, where=mw + ".rot"))
                    sc = _sub(rot, "scaling", mw + ".rot", optional=True)
                    if sc is not None:
                        for key in ("factor", "original", "fast", "slow"):
                            require_positive(f"layers[{i}].mixer.rot.scaling.{key}",
                                             read_key(sc, key, float, where=mw + ".rot.scaling"))
            elif kind == "delta":
                require_positive(f"layers[{i}].mixer.conv", read_key(m, "conv", int, where=mw))
            else:
                raise ConfigError(f"{where}: mixer type '{kind}' is not known ('attention' and 'delta' are)")
            mlp = _sub(L, "mlp", where, optional=True)
            if mlp is not None:
                if read_key(mlp, "kind", str, "dense", where=where + ".mlp") != "dense":
                    raise ConfigError(f"{where}.mlp: kind '{mlp['kind']}' is not known ('dense' is)")
                require_positive(f"layers[{i}].mlp.ff", read_key(mlp, "ff", int, where=where + ".mlp"))
        if self.loop is not None:
            a, b = read_key(self.loop, "start", int, where="config.json: loop"), read_key(self.loop, "stop", int, where="config.json: loop")
            t = read_key(self.loop, "times", int, where="config.json: loop")
            if not (0 <= a < b <= len(self.layers)) or t < 1:
                raise ConfigError(f"config.json: loop {self.loop!r} does not name a run of the {len(self.layers)} layers "
                                  f"(0 <= start < stop <= layers, times >= 1)")

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {
            "architecture": self.architecture, "vocab": self.vocab, "width": self.width,
            "embedding": {"scale": self.embedding_scale}, "norm": {"eps": self.norm_eps},
            "layers": copy.deepcopy(self.layers), "loop": copy.deepcopy(self.loop),
        }
        if self.max_positions != 1 << 20:
            d["max_positions"] = self.max_positions
        if self.eos_token_id:
            d["eos_token_id"] = list(self.eos_token_id)
        return d

    # ------------------------------------------------------------------
    def _mixer_spec(self, L: Dict[str, Any]) -> PartSpec:
        m = L["mixer"]
        if L["type"] == "attention":
            rot, mask = m.get("rot"), m.get("mask")
            position = None
            if rot is not None:
                position = PartSpec("rotary", {"theta": float(rot["base"]), "dim": int(rot["dims"]),
                                               "scaling": dict(rot["scaling"]) if rot.get("scaling") else None})
            return PartSpec("masked_attention", {
                "num_heads": int(m["heads"]), "num_kv_heads": int(m["kv_heads"]), "key_dim": int(m["dim"]),
                "value_dim": int(m["vdim"]), "qkv_bias": True, "position": position, "scale": float(m["scale"]),
                "softcap": float(m.get("softcap") or 0.0), "chunk": int(mask["size"]) if mask else 0,
                "unit_rms_eps": self.norm_eps, "head_gate": True, "names": dict(_ATTENTION_NAMES), "prefix": "mix.",
            })
        return PartSpec("gated_delta", {
            "num_heads": int(m["heads"]), "num_kv_heads": int(m["kv_heads"]), "key_dim": int(m["dim"]),
            "value_dim": int(m["vdim"]), "conv_taps": int(m["conv"]), "norm_eps": self.norm_eps,
            "names": dict(_DELTA_NAMES), "prefix": "mix.",
        })

    def run_order(self) -> List[ScheduleEntry]:
        """The layers in the order they run: those in front of the loop, the looped run `times` times (each pass
        opens by adding its row of the offsets), the rest."""
        n = len(self.layers)
        if self.loop is None:
            return [ScheduleEntry(i) for i in range(n)]
        a, b, times = int(self.loop["start"]), int(self.loop["stop"]), int(self.loop["times"])
        order = [ScheduleEntry(i) for i in range(a)]
        for t in range(times):
            order += [ScheduleEntry(i, offset_row=t if i == a else None) for i in range(a, b)]
        return order + [ScheduleEntry(i) for i in range(b, n)]

    def to_spec(self) -> ModelSpec:
        layers = []
        for i, L in enumerate(self.layers):
            mlp = L.get("mlp")
            norms = {"input": PartSpec("rmsnorm", {"eps": self.norm_eps, "name": "norm1"})}
            ffn = None
            if mlp is not None:
                norms["post_mixer"] = PartSpec("rmsnorm", {"eps": self.norm_eps, "name": "norm2"})
                ffn = PartSpec("gated_mlp", {"intermediate_size": int(mlp["ff"]), "activation": "silu",
                                             "names": dict(_MLP_NAMES), "weight_suffix": "", "prefix": "mlp."})
            layers.append(LayerSpec(block=PartSpec("prenorm", {}), mixer=self._mixer_spec(L), feed_forward=ffn,
                                    norms=norms, prefix=f"l{i}."))
        spec = ModelSpec(
            architecture=self.architecture,
            vocab_size=self.vocab,
            hidden_size=self.width,
            embedding=PartSpec("embedding", {"name": "embed", "scale": self.embedding_scale}),
            layers=layers,
            schedule=self.run_order(),
            final_norm=PartSpec("rmsnorm", {"eps": self.norm_eps, "name": "final.norm"}),
            head=PartSpec("linear_head", {"name": "head", "tied_to": None}),
            max_positions=self.max_positions,
            eos_token_ids=list(self.eos_token_id),
            stream_offsets={"name": "loop.step", "rows": int(self.loop["times"])} if self.loop is not None else None,
        )
        spec.validate()
        return spec
