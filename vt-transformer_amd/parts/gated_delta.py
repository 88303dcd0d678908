"""Gated delta rule: a token mixer with a matrix state per head instead of a
cache of keys and values.

For every value head the mixer carries S [D, Dv] (float32) from token to token:

    S <- g S                      decay, g = exp(-exp(A_log) * softplus(a + dt_bias)) in (0, 1)
    u  = beta (v - S^T k)         what the state gets wrong about this key, times beta = sigmoid(b)
    S <- S + k u^T                corrected towards v
    o  = S^T q                    read out after the write

q and k (shared by the value heads of a group) are unit vectors, q also times
D^-1/2.  In front, q, k and v pass a short causal convolution over time per
channel and a SiLU; behind, each head's o is divided by its root mean square,
multiplied by a gain shared by the heads and by silu of a gate projection, and
projected back to the model's width.  Decay, beta, the unit lengths and the
state are float32 whatever the runtime's dtype.

A request's state slot holds the convolution's last taps - 1 inputs and the
heads' matrices; it has no pages.
"""
from __future__ import annotations

from typing import Callable, Dict, Optional

import torch

from ..kernels import ops
from .base import MIXERS, CacheNeed, Part, Runtime, StateNeed, TensorDecl
from .linear import linear


@MIXERS.register("gated_delta")
class GatedDeltaMixer(Part):
    replayable = True       # a decoding step's launches depend on the number of entries only; its state lies in device
                            # memory and is found by the slots of the step's metadata

    def __init__(self, *, rt: Runtime, width: int, prefix: str, num_heads: int, num_kv_heads: int, key_dim: int,
                 value_dim: int, conv_taps: int, norm_eps: float, shared: Optional[dict] = None,
                 names: Optional[Dict[str, str]] = None):
        """num_heads value heads of value_dim, num_kv_heads query/key heads of key_dim (value head h reads query/key
        head h // (num_heads / num_kv_heads)); conv_taps: length of the convolutions (1: a factor per channel); norm_eps: eps of
        the output's norm; names: tensor names behind the prefix for q, k, v, g, o (matrices), q_conv, k_conv, v_conv
        ([channels, taps], the last column is the current token's), b and a (write strength and decay, one row per
        head), A_log, dt_bias (per head) and norm (per value channel)."""
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} value heads are not a multiple of {num_kv_heads} query/key heads")
        self.rt, self.width = rt, int(width)
        self.nh, self.nkv, self.d, self.dv = int(num_heads), int(num_kv_heads), int(key_dim), int(value_dim)
        self.taps = int(conv_taps)
        self.eps = float(norm_eps)
        if not 1 <= self.d <= ops.DELTA_MAX_KEY_DIM:
            raise ValueError(f"key size {self.d}: the kernel takes up to {ops.DELTA_MAX_KEY_DIM}")
        if not 1 <= self.taps <= ops.CONV_MAX_TAPS:
            raise ValueError(f"{self.taps} taps: the convolution takes 1 to {ops.CONV_MAX_TAPS}")
        n = {"q": "q_proj.weight", "k": "k_proj.weight", "v": "v_proj.weight", "g": "g_proj.weight", "o": "o_proj.weight",
             "q_conv": "q_conv.weight", "k_conv": "k_conv.weight", "v_conv": "v_conv.weight", "b": "b_proj.weight",
             "a": "a_proj.weight", "A_log": "A_log", "dt_bias": "dt_bias", "norm": "norm.weight"}
        n.update(names or {})
        self.names = {k: prefix + v for k, v in n.items()}
        self.channels = 2 * self.nkv * self.d + self.nh * self.dv      # what the convolutions run over: q, k, v
        self.conv_floats = (self.taps - 1) * self.channels
        self.rule_floats = self.nh * self.d * self.dv
        self.w_in = self.p_in = self.w_o = self.p_o = None
        self.conv_w = self.a_log = self.dt_bias = self.norm_w = None

    def cache_need(self) -> Optional[CacheNeed]:
        return None

    def state_need(self) -> Optional[StateNeed]:
        """One float32 row per request: the convolutions' last taps - 1 inputs [taps - 1][channels], then the heads'
        matrices [H][Dv][D]."""
        return StateNeed((self.conv_floats + self.rule_floats,), torch.float32)

    def tensors(self) -> Dict[str, TensorDecl]:
        nm, kd, vd = self.names, self.nkv * self.d, self.nh * self.dv
        t = {
            nm["q"]: TensorDecl((kd, self.width), "matrix"),
            nm["k"]: TensorDecl((kd, self.width), "matrix"),
            nm["v"]: TensorDecl((vd, self.width), "matrix"),
            nm["g"]: TensorDecl((vd, self.width), "matrix"),
            nm["o"]: TensorDecl((self.width, vd), "matrix"),
            nm["b"]: TensorDecl((self.nh, self.width), "matrix"),
            nm["a"]: TensorDecl((self.nh, self.width), "matrix"),
            nm["A_log"]: TensorDecl((self.nh,), "bias"),
            nm["dt_bias"]: TensorDecl((self.nh,), "bias"),
            nm["norm"]: TensorDecl((self.dv,), "gain"),
        }
        # (with one tap the "convolution" is a factor per channel: the tensors are there all the same)
        t[nm["q_conv"]] = TensorDecl((kd, self.taps), "bias")
        t[nm["k_conv"]] = TensorDecl((kd, self.taps), "bias")
        t[nm["v_conv"]] = TensorDecl((vd, self.taps), "bias")
        return t

    def load(self, get: Callable[[str], torch.Tensor], rt: Runtime) -> None:
        nm = self.names
        # one product for everything that reads the mixer's input: q, k, v, the output's gate, and the logits of the
        # write strength and of the decay (what is computed from those two is float32)
        self.w_in = torch.cat([rt.place(get(nm[k]), "matrix") for k in ("q", "k", "v", "g", "b", "a")], dim=0).contiguous()
        self.w_o = rt.place(get(nm["o"]), "matrix")
        self.p_in, self.p_o = rt.pack(self.w_in), rt.pack(self.w_o)
        self.w_in, self.w_o = rt.row_major(self.w_in, self.p_in), rt.row_major(self.w_o, self.p_o)
        self.conv_w = torch.cat([rt.place(get(nm[k]), "bias") for k in ("q_conv", "k_conv", "v_conv")], dim=0).contiguous()
        self.a_log, self.dt_bias = rt.place(get(nm["A_log"]), "bias"), rt.place(get(nm["dt_bias"]), "bias")
        self.norm_w = rt.place(get(nm["norm"]), "gain")

    def forward(self, x, ctx, cache, state):
        rt, c = self.rt, self.channels
        n = x.shape[0]
        if state is None or state.dim() != 2 or state.shape[1] != self.conv_floats + self.rule_floats:
            raise RuntimeError("the gated delta mixer was given no state of its shape")
        conv_state, rule_state = state[:, :self.conv_floats], state[:, self.conv_floats:]
        y = linear(rt, x, self.w_in, None, "delta.in", packed=self.p_in)            # q, k, v, gate, b, a
        qkv = rt.buffer("delta.qkv", (n, c), rt.dtype)
        ops.short_conv(y, c, self.conv_w, conv_state, ctx.tok_entry, ctx.entry_start, ctx.state_slots, qkv)
        if self.taps > 1:
            ops.short_conv_carry(y, c, self.taps, conv_state, ctx.entry_start, ctx.state_slots)
        o = rt.buffer("delta.o", (n, self.nh * self.dv), torch.float32)
        ops.delta_rule(qkv, y, c + self.nh * self.dv, self.a_log, self.dt_bias, rule_state, ctx.entry_start, ctx.state_slots, o, self.nh,
                       self.nkv, self.d, self.dv)
        z = rt.buffer("delta.gated", (n, self.nh * self.dv), rt.dtype)
        ops.gated_rmsnorm(o, self.norm_w, y, c, z, self.nh, self.dv, self.eps)
        return linear(rt, z, self.w_o, None, "delta.o_proj", packed=self.p_o)
